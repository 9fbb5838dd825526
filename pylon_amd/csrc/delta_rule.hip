// The gated delta rule, a linear-attention recurrence with a state S of dim x vdim floats per
// request and head:
//
//   S <- g_t S;  u = beta_t (v_t - S^T k_t);  S <- S + k_t u^T;  o_t = S^T q_t
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
// vectors, beta, decay and the values into LDS), then every thread walks the piece token by token
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

#define DR_PAD 4  // floats between two slices of q or k in LDS (keeps the slices' reads off one bank)

template <int RT, int MAXT, typename TO>
__global__ void __launch_bounds__(MAXT)
delta_rule_kernel(TO* __restrict__ out, long long out_stride, const float* __restrict__ qkv, long long qkv_stride,
                  int q_off, int k_off, int v_off, const float* __restrict__ proj, long long proj_stride, int g_off,
                  int b_off, int a_off, const float* __restrict__ a_log, const float* __restrict__ dt_bias,
                  const float* __restrict__ norm_w, float* __restrict__ state, const int* __restrict__ row_start,
                  const int* __restrict__ row_slots, int heads, int kv_heads, int dim, int vdim, int P, int R, int CT,
                  float eps, float unit_eps, float q_scale, int col_groups, float* __restrict__ raw) {
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
  float* decays = betas + CT;       // [CT]

  float S[RT];
  float* st = state + ((static_cast<size_t>(row_slots[row]) * heads + h) * vdim + j0 + (owner ? j : 0)) * dim + p * R;
#pragma unroll
  for (int r = 0; r < RT; ++r) S[r] = (owner && r < R && p * R + r < dim) ? st[r] : 0.f;

  const float rate = expf(a_log[h]), shift = dt_bias[h];
  for (int c0 = begin; c0 < end; c0 += CT) {
    const int n = end - c0 < CT ? end - c0 : CT;
    // a wave a token: unit q and k in the slices' layout (zeros where a slice has no element)
    for (int i = wave; i < n; i += nwaves) {
      const size_t t = static_cast<size_t>(c0 + i);
      const float* qrow = qkv + t * qkv_stride + q_off + hk * dim;
      const float* krow = qkv + t * qkv_stride + k_off + hk * dim;
      const float* vrow = qkv + t * qkv_stride + v_off + h * vdim + j0;
      float sq = 0.f, sk = 0.f;
      for (int d = lane; d < dim; d += PYLON_WAVE) {
        sq = fmaf(qrow[d], qrow[d], sq);
        sk = fmaf(krow[d], krow[d], sk);
      }
      const float iq = q_scale / sqrtf(wave_sum(sq) + unit_eps);
      const float ik = 1.0f / sqrtf(wave_sum(sk) + unit_eps);
      for (int e = lane; e < KS; e += PYLON_WAVE) {
        const int pp = e / (RT + DR_PAD), r = e - pp * (RT + DR_PAD);
        const int d = pp * R + r;
        const bool there = r < R && d < dim;
        qs[i * KS + e] = there ? qrow[d] * iq : 0.f;
        ks[i * KS + e] = there ? krow[d] * ik : 0.f;
      }
      for (int d = lane; d < vg; d += PYLON_WAVE) vs[i * vg + d] = vrow[d];
      if (lane == 0) {
        const float* pr = proj + t * proj_stride;
        betas[i] = 1.0f / (1.0f + expf(-pr[b_off + h]));
        const float a = pr[a_off + h] + shift;
        const float soft = a > 20.f ? a : log1pf(expf(a));
        decays[i] = expf(-rate * soft);
      }
    }
    __syncthreads();
    if (owner) {  // the P threads of a column are all here or all away
      for (int i = 0; i < n; ++i) {
        const float4* k4 = reinterpret_cast<const float4*>(ks + i * KS + p * (RT + DR_PAD));
        const float4* q4 = reinterpret_cast<const float4*>(qs + i * KS + p * (RT + DR_PAD));
        float a = 0.f;
#pragma unroll
        for (int r = 0; r < RT / 4; ++r) {
          const float4 v = k4[r];
          a = fmaf(S[4 * r], v.x, a);
          a = fmaf(S[4 * r + 1], v.y, a);
          a = fmaf(S[4 * r + 2], v.z, a);
          a = fmaf(S[4 * r + 3], v.w, a);
        }
        for (int off = P >> 1; off > 0; off >>= 1) a += __shfl_xor(a, off, PYLON_WAVE);
        const float g = decays[i];
        const float u = betas[i] * (vs[i * vg + j] - g * a);
        float o = 0.f;
#pragma unroll
        for (int r = 0; r < RT / 4; ++r) {
          const float4 v = q4[r], w = k4[r];  // the keys once more from LDS: cheaper than holding them
          const float qq[4] = {v.x, v.y, v.z, v.w}, kk[4] = {w.x, w.y, w.z, w.w};
#pragma unroll
          for (int c = 0; c < 4; ++c) {
            S[4 * r + c] = fmaf(kk[c], u, g * S[4 * r + c]);
            o = fmaf(S[4 * r + c], qq[c], o);
          }
        }
        for (int off = P >> 1; off > 0; off >>= 1) o += __shfl_xor(o, off, PYLON_WAVE);
        if (p == 0) os[i * vg + j] = o;
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
static int delta_rule_layout(int dim, int vdim, int* P_out, int* R_out) {
  int P = 1;
  while (P * 2 <= 64 && P * 2 <= dim && vdim * P * 2 <= 256) P *= 2;
  int R = (dim + P - 1) / P;
  while (R > 64 && P * 2 <= 64 && vdim * P * 2 <= 1024) {
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
// vdim]) takes o before its norm; tokens: the rows of out.
extern "C" int pylon_delta_rule(void* out, int out_dtype, long long out_stride, const float* qkv, long long qkv_stride,
                                int q_off, int k_off, int v_off, const float* proj, long long proj_stride, int g_off,
                                int b_off, int a_off, const float* a_log, const float* dt_bias, const float* norm_w,
                                float* state, const int* row_start, const int* row_slots, int rows, int heads,
                                int kv_heads, int dim, int vdim, float eps, float unit_eps, float q_scale,
                                int col_groups, float* raw, int tokens, hipStream_t stream) {
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
  int P = 0, R = 0;
  PYLON_REQUIRE(delta_rule_layout(dim, vg, &P, &R), "delta_rule: heads of %d x %d do not fit a workgroup", dim, vg);
  if (rows == 0) return 0;
  int RT = 4;
  while (RT < R) RT *= 2;
  const int KS = P * (RT + DR_PAD);
  const int per_token = 2 * KS + 2 * vg + 2;
  int CT = 12000 / per_token;
  if (CT > 16) CT = 16;
  if (CT < 1) CT = 1;
  const size_t lds = sizeof(float) * static_cast<size_t>(CT) * per_token;
  PYLON_REQUIRE(lds <= 64 * 1024, "delta_rule: a token of %d x %d does not fit LDS", dim, vdim);
  const int threads = (vg * P + PYLON_WAVE - 1) / PYLON_WAVE * PYLON_WAVE;
  PYLON_REQUIRE(static_cast<long long>(rows) * heads * col_groups < (1ll << 31), "delta_rule: too many rows");
  dim3 grid(static_cast<unsigned>(rows * heads * col_groups)), block(threads);
#define GO(RTV, MAXT, TO)                                                                                     \
  hipLaunchKernelGGL((delta_rule_kernel<RTV, MAXT, TO>), grid, block, lds, stream, (TO*)out, out_stride, qkv,   \
                     qkv_stride, q_off, k_off, v_off, proj, proj_stride, g_off, b_off, a_off, a_log, dt_bias,   \
                     norm_w, state, row_start, row_slots, heads, kv_heads, dim, vdim, P, R, CT, eps, unit_eps,  \
                     q_scale, col_groups, raw)
  // up to 256 threads a workgroup may use all registers of a lane; more threads share them
#define BOTH(RTV, TO)                     \
  if (threads <= 256) GO(RTV, 256, TO);   \
  else GO(RTV, 1024, TO)
#define PICK(TO)                         \
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
