// The gated delta rule, a linear-attention recurrence with a state S of dim x vdim floats per
// request and head:
//
//   S <- g_t S;  u = beta_t (v_t - S^T k_t);  S <- S + k_t u^T;  o_t = S^T q_t
//
// (the kernel forms the read-out as g_t S_(t-1)^T q_t + u (k_t . q_t), the same number, so that both
// sums over a column are taken from the state as the token finds it)
//
// with q and k made unit vectors per head first (x / sqrt(sum x^2 + unit_eps); q also times
// q_scale), beta_t = sigmoid(b_t), g_t = exp(-exp(A_log) * softplus(a_t + dt_bias)) per head, and
// every head's o_t divided by its root mean square (eps inside the root), times a weight shared by
// the heads, times silu of a gate.  Everything is float; only the result is rounded.
//
// One workgroup per (row of the step, head).  The state lives in registers for the whole row:
// thread (j, p) keeps a slice of R elements of column j of S (P slices a column, the P threads of
// a column side by side in one wave, so the two sums over dim end in a few lane exchanges).  The
// row's tokens go by in pieces of up to CT: the waves first prepare a piece (a wave a token: unit
// vectors, beta, decay and the values into LDS; in the code: a few threads a token, all tokens of the
// piece at once, the next piece's rows already on their way), then every thread walks the piece token by token
// with no barrier in between, then the waves norm and gate the piece's outputs.  The state is
// read from the request's slot at the start and written back at the end; it is kept transposed,
// [slot, head, vdim, dim], so that a thread's slice is contiguous.
//
// The columns of S never meet (u_j, S[:, j] and o_j depend on column j alone), so where rows are
// long and few the columns of a head are dealt to several workgroups (col_groups), each with more
// threads a column and fewer elements a thread: the chain of dependent instructions a token costs
// gets shorter and more compute units work.  The head's norm needs all its columns: the workgroups
// then leave o unnormed in a float buffer, and a second small kernel norms and gates it.
#include "common.h"

#define DR_PAD 4   // floats between two slices of q or k in LDS (keeps the slices' reads off one bank)
#define DR_HOLD 8  // elements of q, of k and of v that a thread may hold of the next piece

// The sum of v over the P lanes of a column (P a power of two; the lanes j * P .. j * P + P - 1 lie
// side by side), in every one of them.  Up to sixteen lanes it goes through the lanes' own
// data paths (quads swapped, halves of eight mirrored, the row of sixteen mirrored): no trip to LDS,
// which a wave alone on its SIMD would wait out; beyond that rows exchange through it.
template <int CTRL>
__device__ __forceinline__ float dr_moved(float v) {
  return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, 0xf, 0xf, true));
}
__device__ __forceinline__ float column_sum(float v, int P) {
  if (P >= 2) v += dr_moved<0xB1>(v);   // quad_perm [1, 0, 3, 2]
  if (P >= 4) v += dr_moved<0x4E>(v);   // quad_perm [2, 3, 0, 1]
  if (P >= 8) v += dr_moved<0x141>(v);  // row_half_mirror
  if (P >= 16) v += dr_moved<0x140>(v); // row_mirror
  for (int off = 16; off < P; off <<= 1) v += __shfl_xor(v, off, PYLON_WAVE);
  return v;
}

// The same for columns of at most sixteen lanes without a branch: all four steps are taken, and a step
// that would reach past the column adds its neighbour times zero (`steps` holds the four factors).
struct ColumnSteps {
  float f1, f2, f4, f8;
};
__device__ __forceinline__ ColumnSteps column_steps(int P) {
  return ColumnSteps{P >= 2 ? 1.f : 0.f, P >= 4 ? 1.f : 0.f, P >= 8 ? 1.f : 0.f, P >= 16 ? 1.f : 0.f};
}
__device__ __forceinline__ float column_sum(float v, const ColumnSteps& steps) {
  v = fmaf(dr_moved<0xB1>(v), steps.f1, v);
  v = fmaf(dr_moved<0x4E>(v), steps.f2, v);
  v = fmaf(dr_moved<0x141>(v), steps.f4, v);
  v = fmaf(dr_moved<0x140>(v), steps.f8, v);
  return v;
}

#define DR_C 16  // tokens of a piece in the chunked form

template <int RT, int MAXT, bool CHUNK, typename TO>
__global__ void __launch_bounds__(MAXT)
delta_rule_kernel(TO* __restrict__ out, long long out_stride, const float* __restrict__ qkv, long long qkv_stride,
                  int q_off, int k_off, int v_off, const float* __restrict__ proj, long long proj_stride, int g_off,
                  int b_off, int a_off, const float* __restrict__ a_log, const float* __restrict__ dt_bias,
                  const float* __restrict__ norm_w, float* __restrict__ state, const int* __restrict__ row_start,
                  const int* __restrict__ row_slots, int heads, int kv_heads, int dim, int vdim, int P, int R, int CT,
                  float eps, float unit_eps, float q_scale, int col_groups, float* __restrict__ raw, int TPT) {
  extern __shared__ __attribute__((aligned(16))) float dr_lds[];
  const int cg = blockIdx.x % col_groups, rh = blockIdx.x / col_groups;
  const int row = rh / heads, h = rh - row * heads;
  const int vg = vdim / col_groups, j0 = cg * vg;  // this workgroup's columns of S: j0 .. j0 + vg - 1
  const int hk = h / (heads / kv_heads);
  const int begin = row_start[row], end = row_start[row + 1];
  if (begin >= end) return;  // the whole workgroup
  const int tid = threadIdx.x, lane = tid & (PYLON_WAVE - 1), wave = tid / PYLON_WAVE;
  const int nwaves = blockDim.x / PYLON_WAVE;
  const int j = tid / P, p = tid - j * P;
  const bool owner = j < vg;
  const int KS = P * (RT + DR_PAD);
  float* qs = dr_lds;               // [CT][KS]
  float* ks = qs + CT * KS;         // [CT][KS]
  float* vs = ks + CT * KS;         // [CT][vg]
  float* os = vs + CT * vg;         // [CT][vg]
  float* betas = os + CT * vg;      // [CT]
  float* decays = betas + CT;       // [CT]; in the chunked form the decays' logarithms
  // chunked form only: A[t][s] = (G_t / G_s) k_s.k_t, B[t][s] = (G_t / G_s) k_s.q_t with G_t the product of
  // the piece's decays up to token t; G itself; G_last / G_s
  float* amat = decays + CT;        // [DR_C][DR_C]
  float* bmat = amat + DR_C * DR_C; // [DR_C][DR_C]
  float* gcum = bmat + DR_C * DR_C; // [DR_C]
  float* gend = gcum + DR_C;        // [DR_C]
  float* kqs = gend + DR_C;         // [CT <= DR_C]: the token's unit k times its scaled unit q

  float S[RT];
  float* st = state + ((static_cast<size_t>(row_slots[row]) * heads + h) * vdim + j0 + (owner ? j : 0)) * dim + p * R;
#pragma unroll
  for (int r = 0; r < RT; ++r) S[r] = (owner && r < R && p * R + r < dim) ? st[r] : 0.f;

  const float rate = expf(a_log[h]), shift = dt_bias[h];
  // A piece's rows are prepared by TPT threads a token, all tokens of the piece at once.  Where a
  // thread's share is at most DR_HOLD elements of q, of k and of v, the next piece's rows are fetched
  // into registers before the walk over this piece, so that their way from memory is hidden behind it.
  const int ti = tid / TPT, sub = tid - ti * TPT;
  const bool held = dim <= DR_HOLD * TPT && vg <= DR_HOLD * TPT;
  const ColumnSteps token_steps = column_steps(TPT);
  float rq[DR_HOLD], rk[DR_HOLD], rv[DR_HOLD], rb = 0.f, ra = 0.f;
  auto fetch = [&](int c0) {
    const int n = end - c0 < CT ? end - c0 : CT;
    if (ti >= n) return;
    const size_t t = static_cast<size_t>(c0 + ti);
    const float* qrow = qkv + t * qkv_stride + q_off + hk * dim;
    const float* krow = qkv + t * qkv_stride + k_off + hk * dim;
    const float* vrow = qkv + t * qkv_stride + v_off + h * vdim + j0;
#pragma unroll
    for (int e = 0; e < DR_HOLD; ++e) {
      const int d = sub + e * TPT;
      rq[e] = d < dim ? qrow[d] : 0.f;
      rk[e] = d < dim ? krow[d] : 0.f;
      rv[e] = d < vg ? vrow[d] : 0.f;
    }
    if (sub == 0) {
      rb = proj[t * proj_stride + b_off + h];
      ra = proj[t * proj_stride + a_off + h];
    }
  };
  // the slices' pads (and the elements past dim) stay zero: only real elements are ever written
  for (int e = tid; e < 2 * CT * KS; e += blockDim.x) qs[e] = 0.f;
  if (held) fetch(begin);
  __syncthreads();
  for (int c0 = begin; c0 < end; c0 += CT) {
    const int n = end - c0 < CT ? end - c0 : CT;
    if (ti < n) {
      const size_t t = static_cast<size_t>(c0 + ti);
      const float* qrow = qkv + t * qkv_stride + q_off + hk * dim;
      const float* krow = qkv + t * qkv_stride + k_off + hk * dim;
      const float* vrow = qkv + t * qkv_stride + v_off + h * vdim + j0;
      float sq = 0.f, sk = 0.f, qk = 0.f;
      if (held) {
#pragma unroll
        for (int e = 0; e < DR_HOLD; ++e) {
          sq = fmaf(rq[e], rq[e], sq);
          sk = fmaf(rk[e], rk[e], sk);
          qk = fmaf(rq[e], rk[e], qk);
        }
      } else {
        for (int d = sub; d < dim; d += TPT) {
          sq = fmaf(qrow[d], qrow[d], sq);
          sk = fmaf(krow[d], krow[d], sk);
          qk = fmaf(qrow[d], krow[d], qk);
        }
      }
      // the TPT threads of a token lie side by side in one wave
      if (TPT <= 16) {
        sq = column_sum(sq, token_steps), sk = column_sum(sk, token_steps), qk = column_sum(qk, token_steps);
      } else {
        sq = column_sum(sq, TPT), sk = column_sum(sk, TPT), qk = column_sum(qk, TPT);
      }
      const float iq = q_scale / sqrtf(sq + unit_eps);
      const float ik = 1.0f / sqrtf(sk + unit_eps);
      if (held) {
#pragma unroll
        for (int e = 0; e < DR_HOLD; ++e) {
          const int d = sub + e * TPT;
          if (d < dim) {
            const int at = ti * KS + (d / R) * (RT + DR_PAD) + d % R;
            qs[at] = rq[e] * iq;
            ks[at] = rk[e] * ik;
          }
          if (d < vg) vs[ti * vg + d] = rv[e];
        }
      } else {
        for (int d = sub; d < dim; d += TPT) {
          const int at = ti * KS + (d / R) * (RT + DR_PAD) + d % R;
          qs[at] = qrow[d] * iq;
          ks[at] = krow[d] * ik;
        }
        for (int d = sub; d < vg; d += TPT) vs[ti * vg + d] = vrow[d];
        if (sub == 0) {
          rb = proj[t * proj_stride + b_off + h];
          ra = proj[t * proj_stride + a_off + h];
        }
      }
      if (sub == 0) {
        kqs[ti] = qk * iq * ik;
        betas[ti] = 1.0f / (1.0f + expf(-rb));
        const float a = ra + shift;
        const float soft = a > 20.f ? a : log1pf(expf(a));
        decays[ti] = CHUNK ? -rate * soft : expf(-rate * soft);
      }
    }
    __syncthreads();
    if (held && c0 + CT < end) fetch(c0 + CT);  // on their way while this piece is walked
    if constexpr (CHUNK) {
      // The piece at once.  With G_t = g_1 ... g_t (the piece's decays) and S_0 the state before it:
      //   u_t = beta_t (v_t - G_t S_0^T k_t - sum_{s<t} A[t][s] u_s),
      //   o_t = G_t S_0^T q_t + sum_{s<=t} B[t][s] u_s,   S_n = G_n S_0 + sum_s (G_n / G_s) k_s u_s^T,
      // which is the token-by-token rule written out.  The products with S_0 and the sums over the
      // lanes of a column are independent over the piece's tokens, so their waits overlap; what is
      // left in order is a short chain of multiply-adds in registers.
      for (int idx = tid; idx < 2 * DR_C * DR_C; idx += blockDim.x) {
        const int which = idx / (DR_C * DR_C), ts = idx - which * DR_C * DR_C;
        const int t = ts / DR_C, sx = ts - t * DR_C;
        float value = 0.f;
        if (t < n && sx <= t) {
          const float4* a4 = reinterpret_cast<const float4*>(ks + sx * KS);
          const float4* b4 = reinterpret_cast<const float4*>((which ? qs : ks) + t * KS);
          float d0 = 0.f, d1 = 0.f, d2 = 0.f, d3 = 0.f;
#pragma unroll 8
          for (int e = 0; e < KS / 4; ++e) {  // the pads hold zeros; several reads of LDS in flight
            const float4 x = a4[e], y = b4[e];
            d0 = fmaf(x.x, y.x, d0);
            d1 = fmaf(x.y, y.y, d1);
            d2 = fmaf(x.z, y.z, d2);
            d3 = fmaf(x.w, y.w, d3);
          }
          d0 = (d0 + d1) + (d2 + d3);
          d1 = 0.f;
          float lg = 0.f;
          for (int r = sx + 1; r <= t; ++r) lg += decays[r];
          value = (d0 + d1) * expf(lg);
        }
        (which ? bmat : amat)[ts] = value;
      }
      if (tid < DR_C) {
        float lg = 0.f, all = 0.f;
        for (int r = 0; r < n; ++r) {
          all += decays[r];
          if (r <= tid) lg = all;
        }
        gcum[tid] = expf(lg);
        gend[tid] = expf(all - lg);
      }
      __syncthreads();
      if (owner) {
        const float* kbase = ks + p * (RT + DR_PAD);
        const float* qbase = qs + p * (RT + DR_PAD);
        float w[DR_C], y[DR_C], u[DR_C];
#pragma unroll
        for (int t = 0; t < DR_C; ++t) {
          w[t] = 0.f;
          y[t] = 0.f;
          if (t < n) {
            const float4* k4 = reinterpret_cast<const float4*>(kbase + t * KS);
            const float4* q4 = reinterpret_cast<const float4*>(qbase + t * KS);
            float w1 = 0.f, y1 = 0.f;
#pragma unroll
            for (int r = 0; r < RT / 4; ++r) {
              const float4 kv = k4[r], qv = q4[r];
              w[t] = fmaf(S[4 * r], kv.x, w[t]);
              w1 = fmaf(S[4 * r + 1], kv.y, w1);
              w[t] = fmaf(S[4 * r + 2], kv.z, w[t]);
              w1 = fmaf(S[4 * r + 3], kv.w, w1);
              y[t] = fmaf(S[4 * r], qv.x, y[t]);
              y1 = fmaf(S[4 * r + 1], qv.y, y1);
              y[t] = fmaf(S[4 * r + 2], qv.z, y[t]);
              y1 = fmaf(S[4 * r + 3], qv.w, y1);
            }
            w[t] += w1;
            y[t] += y1;
          }
        }
#pragma unroll
        for (int t = 0; t < DR_C; ++t) {
          w[t] = column_sum(w[t], P);
          y[t] = column_sum(y[t], P);
        }
#pragma unroll
        for (int t = 0; t < DR_C; ++t) {
          u[t] = 0.f;
          if (t < n) {
            const float gt = gcum[t];
            float acc = vs[t * vg + j] - gt * w[t];
            float o = gt * y[t];
            // row t of both matrices in 16-byte pieces, fetched before the chain that uses them
            float ar[DR_C], br[DR_C];
#pragma unroll
            for (int c = 0; c <= t / 4; ++c) {
              const float4 av = *reinterpret_cast<const float4*>(amat + t * DR_C + 4 * c);
              const float4 bv = *reinterpret_cast<const float4*>(bmat + t * DR_C + 4 * c);
              ar[4 * c] = av.x, ar[4 * c + 1] = av.y, ar[4 * c + 2] = av.z, ar[4 * c + 3] = av.w;
              br[4 * c] = bv.x, br[4 * c + 1] = bv.y, br[4 * c + 2] = bv.z, br[4 * c + 3] = bv.w;
            }
#pragma unroll
            for (int sx = 0; sx < t; ++sx) {
              acc = fmaf(-ar[sx], u[sx], acc);
              o = fmaf(br[sx], u[sx], o);
            }
            u[t] = betas[t] * acc;
            o = fmaf(br[t], u[t], o);
            if (p == 0) os[t * vg + j] = o;
          }
        }
        const float gn = gcum[n - 1];
#pragma unroll
        for (int r = 0; r < RT; ++r) S[r] *= gn;
#pragma unroll
        for (int t = 0; t < DR_C; ++t) {
          if (t < n) {
            const float c = gend[t] * u[t];
            const float4* k4 = reinterpret_cast<const float4*>(kbase + t * KS);
#pragma unroll
            for (int r = 0; r < RT / 4; ++r) {
              const float4 kv = k4[r];
              S[4 * r] = fmaf(kv.x, c, S[4 * r]);
              S[4 * r + 1] = fmaf(kv.y, c, S[4 * r + 1]);
              S[4 * r + 2] = fmaf(kv.z, c, S[4 * r + 2]);
              S[4 * r + 3] = fmaf(kv.w, c, S[4 * r + 3]);
            }
          }
        }
      }
    } else
    if (owner) {  // the P threads of a column are all here or all away
      if (RT <= 16 && P <= 16) {
        const ColumnSteps steps = column_steps(P);
        // short slices: the next token's keys, queries and numbers leave LDS while this token's chain runs
        const float* kb = ks + p * (RT + DR_PAD);
        const float* qb = qs + p * (RT + DR_PAD);
        float4 kn[RT / 4], qn[RT / 4];
        float gn = decays[0], bn = betas[0], vn = vs[j], cn = kqs[0];
#pragma unroll
        for (int r = 0; r < RT / 4; ++r) {
          kn[r] = reinterpret_cast<const float4*>(kb)[r];
          qn[r] = reinterpret_cast<const float4*>(qb)[r];
        }
        for (int i = 0; i < n; ++i) {
          float4 kc[RT / 4], qc[RT / 4];
#pragma unroll
          for (int r = 0; r < RT / 4; ++r) kc[r] = kn[r], qc[r] = qn[r];
          const float g = gn, b = bn, v = vn, kq = cn;
          {
            const int nx = i + 1 < n ? i + 1 : i;  // the last token fetches itself again: no branch
#pragma unroll
            for (int r = 0; r < RT / 4; ++r) {
              kn[r] = reinterpret_cast<const float4*>(kb + nx * KS)[r];
              qn[r] = reinterpret_cast<const float4*>(qb + nx * KS)[r];
            }
            gn = decays[nx], bn = betas[nx], vn = vs[nx * vg + j], cn = kqs[nx];
          }
          // both sums over the column before the state moves: S_t^T q = g S_(t-1)^T q + u (k.q), so the
          // read-out needs no second sum behind the update
          float a0 = 0.f, a1 = 0.f, y0 = 0.f, y1 = 0.f;
#pragma unroll
          for (int r = 0; r < RT / 4; ++r) {
            a0 = fmaf(S[4 * r], kc[r].x, a0);
            a1 = fmaf(S[4 * r + 1], kc[r].y, a1);
            a0 = fmaf(S[4 * r + 2], kc[r].z, a0);
            a1 = fmaf(S[4 * r + 3], kc[r].w, a1);
            y0 = fmaf(S[4 * r], qc[r].x, y0);
            y1 = fmaf(S[4 * r + 1], qc[r].y, y1);
            y0 = fmaf(S[4 * r + 2], qc[r].z, y0);
            y1 = fmaf(S[4 * r + 3], qc[r].w, y1);
          }
          const float a = column_sum(a0 + a1, steps), y = column_sum(y0 + y1, steps);
          const float u = b * (v - g * a);
          os[i * vg + j] = fmaf(u, kq, g * y);  // every lane of the column holds the same number
#pragma unroll
          for (int r = 0; r < RT / 4; ++r) {
            S[4 * r] = fmaf(kc[r].x, u, g * S[4 * r]);
            S[4 * r + 1] = fmaf(kc[r].y, u, g * S[4 * r + 1]);
            S[4 * r + 2] = fmaf(kc[r].z, u, g * S[4 * r + 2]);
            S[4 * r + 3] = fmaf(kc[r].w, u, g * S[4 * r + 3]);
          }
        }
      } else {
      for (int i = 0; i < n; ++i) {
        const float4* k4 = reinterpret_cast<const float4*>(ks + i * KS + p * (RT + DR_PAD));
        const float4* q4 = reinterpret_cast<const float4*>(qs + i * KS + p * (RT + DR_PAD));
        // chains of additions side by side, so that a sum does not wait for itself
        float a0 = 0.f, a1 = 0.f, y0 = 0.f, y1 = 0.f;
#pragma unroll
        for (int r = 0; r < RT / 4; ++r) {
          const float4 kv = k4[r], qv = q4[r];
          a0 = fmaf(S[4 * r], kv.x, a0);
          a1 = fmaf(S[4 * r + 1], kv.y, a1);
          a0 = fmaf(S[4 * r + 2], kv.z, a0);
          a1 = fmaf(S[4 * r + 3], kv.w, a1);
          y0 = fmaf(S[4 * r], qv.x, y0);
          y1 = fmaf(S[4 * r + 1], qv.y, y1);
          y0 = fmaf(S[4 * r + 2], qv.z, y0);
          y1 = fmaf(S[4 * r + 3], qv.w, y1);
        }
        const float a = column_sum(a0 + a1, P), y = column_sum(y0 + y1, P);
        const float g = decays[i];
        const float u = betas[i] * (vs[i * vg + j] - g * a);
        if (p == 0) os[i * vg + j] = fmaf(u, kqs[i], g * y);
#pragma unroll
        for (int r = 0; r < RT / 4; ++r) {
          const float4 w = k4[r];  // the keys once more from LDS: cheaper than holding them
          S[4 * r] = fmaf(w.x, u, g * S[4 * r]);
          S[4 * r + 1] = fmaf(w.y, u, g * S[4 * r + 1]);
          S[4 * r + 2] = fmaf(w.z, u, g * S[4 * r + 2]);
          S[4 * r + 3] = fmaf(w.w, u, g * S[4 * r + 3]);
        }
      }
      }
    }
    __syncthreads();
    if (raw != nullptr) {
      // the head's other columns are elsewhere: o as it is, for the kernel that norms and gates
      for (int e = tid; e < n * vg; e += blockDim.x) {
        const int i = e / vg, d = e - i * vg;
        raw[(static_cast<size_t>(c0 + i) * heads + h) * vdim + j0 + d] = os[e];
      }
      __syncthreads();
      continue;
    }
    // a wave a token: the head's norm, its weight, the gate
    for (int i = wave; i < n; i += nwaves) {
      const size_t t = static_cast<size_t>(c0 + i);
      float ss = 0.f;
      for (int d = lane; d < vdim; d += PYLON_WAVE) ss = fmaf(os[i * vdim + d], os[i * vdim + d], ss);
      const float inv = 1.0f / sqrtf(wave_sum(ss) / static_cast<float>(vdim) + eps);
      const float* gate = proj + t * proj_stride + g_off + h * vdim;
      TO* orow = out + t * out_stride + h * vdim;
      for (int d = lane; d < vdim; d += PYLON_WAVE) {
        const float z = gate[d];
        orow[d] = from_float<TO>(os[i * vdim + d] * inv * norm_w[d] * (z / (1.0f + expf(-z))));
      }
    }
    __syncthreads();  // the next piece overwrites what this one read
  }
  if (owner) {
#pragma unroll
    for (int r = 0; r < RT; ++r)
      if (r < R && p * R + r < dim) st[r] = S[r];
  }
}

// out[t, h, :] = raw[t, h, :] / rms(raw[t, h, :]) * norm_w * silu(gate[t, h, :]); a wave a (token, head).
template <typename TO>
__global__ void __launch_bounds__(256)
delta_rule_finish_kernel(TO* __restrict__ out, long long out_stride, const float* __restrict__ raw,
                         const float* __restrict__ proj, long long proj_stride, int g_off,
                         const float* __restrict__ norm_w, long long items, int heads, int vdim, float eps) {
  const int lane = threadIdx.x & (PYLON_WAVE - 1);
  const long long item = static_cast<long long>(blockIdx.x) * 4 + threadIdx.x / PYLON_WAVE;
  if (item >= items) return;  // whole waves leave; no barrier follows
  const size_t t = static_cast<size_t>(item / heads);
  const int h = static_cast<int>(item - static_cast<long long>(t) * heads);
  const float* o = raw + (t * heads + h) * vdim;
  float ss = 0.f;
  for (int d = lane; d < vdim; d += PYLON_WAVE) ss = fmaf(o[d], o[d], ss);
  const float inv = 1.0f / sqrtf(wave_sum(ss) / static_cast<float>(vdim) + eps);
  const float* gate = proj + t * proj_stride + g_off + h * vdim;
  TO* orow = out + t * out_stride + h * vdim;
  for (int d = lane; d < vdim; d += PYLON_WAVE) {
    const float z = gate[d];
    orow[d] = from_float<TO>(o[d] * inv * norm_w[d] * (z / (1.0f + expf(-z))));
  }
}

// How a head of dim x vdim is laid over a workgroup: P threads a column (a power of two of at most
// 64), R elements a thread.  Returns 0 if no layout fits.
static int delta_rule_layout(int dim, int vdim, int wide, int* P_out, int* R_out) {
  int P = 1;
  if (wide) {
    // as many threads a column (up to the sixteen of a row of lanes) as fill a workgroup of 256: short slices
    while (P * 2 <= 16 && P * 2 <= dim && vdim * P * 2 <= 256) P *= 2;
  } else {
    // token by token: up to four threads a column while a thread's slice is longer than 32 elements (the
    // sums over a column then end inside a quad of lanes)
    while (P < 4 && P * 2 <= dim && (dim + P - 1) / P > 32 && vdim * P * 2 <= 1024) P *= 2;
  }
  int R = (dim + P - 1) / P;
  while (R > 64 && P * 2 <= 64 && vdim * P * 2 <= 1024) {  // more threads a column where the registers ask for it
    P *= 2;
    R = (dim + P - 1) / P;
  }
  if (R > 128 || vdim * P > 1024 || (R > 64 && vdim * P > 256)) return 0;
  *P_out = P;
  *R_out = R;
  return 1;
}

// out: [tokens, heads * vdim] of out_dtype, rows out_stride apart.  qkv: float rows qkv_stride apart
// holding, after the short convolution and its activation, q at q_off ([kv_heads, dim]), k at k_off
// ([kv_heads, dim]) and v at v_off ([heads, vdim]); head h uses q/k head h / (heads / kv_heads).
// proj: float rows proj_stride apart holding the gate at g_off ([heads, vdim]) and per head the
// logits of beta at b_off and of the decay at a_off.  a_log, dt_bias: float [heads]; norm_w: float
// [vdim].  state: float [slots, heads, vdim, dim].  row_start: [rows + 1] prefix sums of the rows'
// token counts; row_slots: [rows] the rows' state slots (the host guarantees they are in range).
// col_groups > 1: a head's columns are dealt to that many workgroups, and raw (float [tokens, heads *
// vdim]) takes o before its norm; tokens: the rows of out.  chunked 1: sixteen tokens at a time where
// the sizes allow (same results up to the order of additions), else token by token.
extern "C" int pylon_delta_rule(void* out, int out_dtype, long long out_stride, const float* qkv, long long qkv_stride,
                                int q_off, int k_off, int v_off, const float* proj, long long proj_stride, int g_off,
                                int b_off, int a_off, const float* a_log, const float* dt_bias, const float* norm_w,
                                float* state, const int* row_start, const int* row_slots, int rows, int heads,
                                int kv_heads, int dim, int vdim, float eps, float unit_eps, float q_scale,
                                int col_groups, float* raw, int tokens, int chunked, hipStream_t stream) {
  PYLON_REQUIRE(pylon_valid_dtype(out_dtype), "delta_rule: unknown dtype");
  PYLON_REQUIRE(rows >= 0 && heads >= 1 && kv_heads >= 1 && heads % kv_heads == 0 && dim >= 1 && vdim >= 1,
                "delta_rule: %d heads over %d q/k heads of %d x %d", heads, kv_heads, dim, vdim);
  PYLON_REQUIRE(out != nullptr && qkv != nullptr && proj != nullptr && a_log != nullptr && dt_bias != nullptr &&
                    norm_w != nullptr && state != nullptr && row_start != nullptr && row_slots != nullptr,
                "delta_rule: every operand is required");
  PYLON_REQUIRE(out_stride >= static_cast<long long>(heads) * vdim, "delta_rule: rows of the output overlap");
  PYLON_REQUIRE(col_groups >= 1 && vdim % col_groups == 0, "delta_rule: %d columns in %d groups", vdim, col_groups);
  PYLON_REQUIRE((col_groups == 1) == (raw == nullptr), "delta_rule: columns dealt to several workgroups need the buffer for o");
  const int vg = vdim / col_groups;
  int P = 0, R = 0, RT = 4;
  // the chunked form where its layout fits 256 threads, slices of at most 32 elements and LDS
  if (chunked) {
    chunked = 0;
    if (delta_rule_layout(dim, vg, 1, &P, &R) && R <= 32 && vg * P <= 256) {
      while (RT < R) RT *= 2;
      chunked = sizeof(float) * (DR_C * (2 * P * (RT + DR_PAD) + 2 * vg + 2) + 2 * DR_C * DR_C + 3 * DR_C) <= 64 * 1024;
    }
  }
  // token by token: columns dealt to several workgroups take the wide layout too (measured: 10 heads of
  // 128 x 128 over 2,048 tokens, 16 columns and 16 threads a column 1.74 ms, 64 columns and 4 threads 2.24)
  if (!chunked)
    PYLON_REQUIRE(delta_rule_layout(dim, vg, col_groups > 1 ? 1 : 0, &P, &R),
                  "delta_rule: heads of %d x %d do not fit a workgroup", dim, vg);
  if (rows == 0) return 0;
  RT = 4;
  while (RT < R) RT *= 2;
  const int KS = P * (RT + DR_PAD);
  const int per_token = 2 * KS + 2 * vg + 2;
  int CT = chunked ? DR_C : 12000 / per_token;
  if (CT > 16) CT = 16;
  if (CT < 1) CT = 1;
  PYLON_REQUIRE(sizeof(float) * per_token <= 64 * 1024, "delta_rule: a token of %d x %d does not fit LDS", dim, vdim);
  const int threads = (vg * P + PYLON_WAVE - 1) / PYLON_WAVE * PYLON_WAVE;
  // threads that prepare one token of a piece: a power of two, all CT tokens at once
  if (CT > threads) CT = threads;
  int tpt = 1;
  while (tpt * 2 <= PYLON_WAVE && tpt * 2 * CT <= threads) tpt *= 2;
  PYLON_REQUIRE(static_cast<long long>(rows) * heads * col_groups < (1ll << 31), "delta_rule: too many rows");
  const size_t lds = sizeof(float) * (static_cast<size_t>(CT) * per_token + 2 * DR_C * DR_C + 3 * DR_C);
  dim3 grid(static_cast<unsigned>(rows * heads * col_groups)), block(threads);
#define GO(RTV, MAXT, TO)                                                                                     \
  GOC(RTV, MAXT, false, TO)
#define GOC(RTV, MAXT, CH, TO)                                                                                \
  hipLaunchKernelGGL((delta_rule_kernel<RTV, MAXT, CH, TO>), grid, block, lds, stream, (TO*)out, out_stride, qkv, \
                     qkv_stride, q_off, k_off, v_off, proj, proj_stride, g_off, b_off, a_off, a_log, dt_bias,   \
                     norm_w, state, row_start, row_slots, heads, kv_heads, dim, vdim, P, R, CT, eps, unit_eps,  \
                     q_scale, col_groups, raw, tpt)
  // up to 256 threads a workgroup may use all registers of a lane; more threads share them
#define BOTH(RTV, TO)                     \
  if (threads <= 256) GO(RTV, 256, TO);   \
  else GO(RTV, 1024, TO)
#define PICK(TO)                         \
  if (chunked) {                         \
    switch (RT) {                        \
      case 4: GOC(4, 256, true, TO); break;   \
      case 8: GOC(8, 256, true, TO); break;   \
      case 16: GOC(16, 256, true, TO); break; \
      default: GOC(32, 256, true, TO); break; \
    }                                    \
  } else                                 \
  switch (RT) {                          \
    case 4: BOTH(4, TO); break;          \
    case 8: BOTH(8, TO); break;          \
    case 16: BOTH(16, TO); break;        \
    case 32: BOTH(32, TO); break;        \
    case 64: BOTH(64, TO); break;        \
    default: GO(128, 256, TO); break;    \
  }
  if (out_dtype == PYLON_F32) {
    PICK(float);
  } else {
    PICK(bf16_t);
  }
#undef PICK
#undef BOTH
#undef GOC
#undef GO
  if (raw != nullptr && tokens > 0) {
    const long long items = static_cast<long long>(tokens) * heads;
    dim3 fgrid(static_cast<unsigned>((items + 3) / 4)), fblock(256);
    if (out_dtype == PYLON_F32)
      hipLaunchKernelGGL(delta_rule_finish_kernel<float>, fgrid, fblock, 0, stream, (float*)out, out_stride, raw, proj,
                         proj_stride, g_off, norm_w, items, heads, vdim, eps);
    else
      hipLaunchKernelGGL(delta_rule_finish_kernel<bf16_t>, fgrid, fblock, 0, stream, (bf16_t*)out, out_stride, raw, proj,
                         proj_stride, g_off, norm_w, items, heads, vdim, eps);
  }
  PYLON_LAUNCHED("delta_rule");
}
