// A mixture of gated feed-forward experts, token by token.
//
// route_top: from float router logits (a product computed elsewhere) plus a bias, the `top`
//   experts with the largest logits (the lower index among equals) and the softmax over those
//   logits alone (scoring 0), or every chosen expert's own sigmoid(logit) as it is (scoring 1: the
//   order of the sigmoids is the order of the logits); optionally sigmoid of one more logit per
//   token, the gate of a shared expert.  One wavefront per token, everything in float.
// expert_gate_up: hidden[(t, s)] = silu(W_gate[e] x_t) * (W_up[e] x_t) for every token t and each of
//   its chosen experts e = experts[t, s]; a workgroup takes one (token, choice) and some hidden
//   units, the token's input in LDS, a wave a hidden unit at a time with the lanes along the row.
// expert_down: out[t] = sum_s weight[t, s] W_down[e_s] hidden[(t, s)] (+ gate[t] * shared[t]), float.
// route_scored: the other way to choose: scores are the softmax over all router outputs; a
//   correction is added to them for the choice only; the outputs form equal groups of neighbours of
//   which only the best few (by their largest corrected score) may be chosen from; the weights are the
//   chosen scores times a constant, not renormalised.  The last router outputs may be identity
//   experts, whose output is the token's input itself: their weights are summed into one number per
//   token, and the expert kernels pass over them.
// Experts may also be plain, W_down act(W_up x) with act the square of relu (`act` 1).
// Every sum runs over its row in one fixed order, so a token's result does not depend on what
// else is in the batch.
#include "common.h"

#define MX_MAX_TOP 32

__global__ void __launch_bounds__(256)
route_top_kernel(int* __restrict__ experts, float* __restrict__ weights, float* __restrict__ shared_gate,
                 const float* __restrict__ logits, long long row_stride, const float* __restrict__ bias,
                 int tokens, int n_experts, int top, int scoring) {
  __shared__ float chosen[4][MX_MAX_TOP];
  const int lane = threadIdx.x & (PYLON_WAVE - 1), wave = threadIdx.x / PYLON_WAVE;
  const int t = blockIdx.x * 4 + wave;
  if (t >= tokens) return;  // whole waves leave; no barrier follows
  const float* row = logits + static_cast<size_t>(t) * row_stride;
  // lane l keeps experts l, l + 64, ... (at most 8 of them)
  float z[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    const int e = lane + PYLON_WAVE * i;
    z[i] = e < n_experts ? row[e] + (bias != nullptr ? bias[e] : 0.f) : -INFINITY;
  }
  for (int k = 0; k < top; ++k) {
    float best = -INFINITY;
    int best_e = 0x7fffffff;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const int e = lane + PYLON_WAVE * i;
      if (e < n_experts && (z[i] > best || (z[i] == best && e < best_e)) && !(z[i] != z[i])) {
        best = z[i];
        best_e = e;
      }
    }
#pragma unroll
    for (int off = PYLON_WAVE / 2; off > 0; off >>= 1) {
      const float other = __shfl_xor(best, off, PYLON_WAVE);
      const int other_e = __shfl_xor(best_e, off, PYLON_WAVE);
      if (other > best || (other == best && other_e < best_e)) {
        best = other;
        best_e = other_e;
      }
    }
    if (best_e == 0x7fffffff) best_e = 0;  // nothing comparable left (NaN logits): expert 0
#pragma unroll
    for (int i = 0; i < 8; ++i)
      if (lane + PYLON_WAVE * i == best_e) z[i] = -INFINITY;  // taken; -inf also marks it for later rounds
    if (lane == 0) {
      experts[static_cast<size_t>(t) * top + k] = best_e;
      chosen[wave][k] = best;
    }
    // an expert whose logit is -inf can be taken twice only if fewer than `top` finite logits exist
  }
  __builtin_amdgcn_wave_barrier();
  if (lane == 0) {
    if (scoring == 1) {
      for (int k = 0; k < top; ++k)
        weights[static_cast<size_t>(t) * top + k] = 1.0f / (1.0f + expf(-chosen[wave][k]));
    } else {
      const float m = chosen[wave][0];  // the largest: they were taken in falling order
      float sum = 0.f;
      for (int k = 0; k < top; ++k) {
        const float p = expf(chosen[wave][k] - m);
        chosen[wave][k] = p;
        sum += p;
      }
      for (int k = 0; k < top; ++k) weights[static_cast<size_t>(t) * top + k] = chosen[wave][k] / sum;
    }
    if (shared_gate != nullptr) shared_gate[t] = 1.0f / (1.0f + expf(-row[n_experts]));
  }
}

// logits: float [tokens, n_experts (+ 1 with shared_gate)], rows row_stride apart; bias: null or
// float [n_experts]; experts int [tokens, top], weights float [tokens, top], shared_gate null or float [tokens].
extern "C" int pylon_route_top(int* experts, float* weights, float* shared_gate, const float* logits,
                               long long row_stride, const float* bias, int tokens, int n_experts, int top,
                               int scoring, hipStream_t stream) {
  PYLON_REQUIRE(scoring == 0 || scoring == 1, "route_top: unknown scoring %d", scoring);
  PYLON_REQUIRE(tokens >= 0 && n_experts >= 1 && n_experts <= 8 * PYLON_WAVE,
                "route_top: 1 to %d experts, got %d", 8 * PYLON_WAVE, n_experts);
  PYLON_REQUIRE(top >= 1 && top <= n_experts && top <= MX_MAX_TOP, "route_top: top %d of %d experts (at most %d)",
                top, n_experts, MX_MAX_TOP);
  PYLON_REQUIRE(row_stride >= n_experts + (shared_gate != nullptr ? 1 : 0), "route_top: rows of logits overlap");
  if (tokens == 0) return 0;
  hipLaunchKernelGGL(route_top_kernel, dim3((tokens + 3) / 4), dim3(256), 0, stream, experts, weights, shared_gate,
                     logits, row_stride, bias, tokens, n_experts, top, scoring);
  PYLON_LAUNCHED("route_top");
}

#define MX_MAX_OUTPUTS (8 * PYLON_WAVE)

__global__ void __launch_bounds__(256)
route_scored_kernel(int* __restrict__ experts, float* __restrict__ weights, float* __restrict__ identity_weight,
                    const float* __restrict__ logits, long long row_stride, const float* __restrict__ correction,
                    int tokens, int n_outputs, int n_experts, int top, int groups, int keep, float scale) {
  __shared__ float choice[4][MX_MAX_OUTPUTS];  // corrected scores, then -inf outside the kept groups
  __shared__ float best_of[4][MX_MAX_OUTPUTS];  // every group's largest corrected score
  const int lane = threadIdx.x & (PYLON_WAVE - 1), wave = threadIdx.x / PYLON_WAVE;
  const int t = blockIdx.x * 4 + wave;
  if (t >= tokens) return;  // whole waves leave; only wave-level barriers follow
  const float* row = logits + static_cast<size_t>(t) * row_stride;
  float z[8], s[8];
  float top_z = -INFINITY;
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    const int e = lane + PYLON_WAVE * i;
    z[i] = e < n_outputs ? row[e] : -INFINITY;
    top_z = fmaxf(top_z, z[i]);
  }
  top_z = wave_max(top_z);
  float sum = 0.f;
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    const int e = lane + PYLON_WAVE * i;
    s[i] = e < n_outputs ? expf(z[i] - top_z) : 0.f;
    sum += s[i];
  }
  const float inv = 1.0f / wave_sum(sum);
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    const int e = lane + PYLON_WAVE * i;
    s[i] *= inv;
    if (e < n_outputs) choice[wave][e] = s[i] + (correction != nullptr ? correction[e] : 0.f);
  }
  __builtin_amdgcn_wave_barrier();
  const int per_group = n_outputs / groups;
  if (keep < groups) {
    for (int g = lane; g < groups; g += PYLON_WAVE) {
      float m = -INFINITY;
      for (int k = 0; k < per_group; ++k) m = fmaxf(m, choice[wave][g * per_group + k]);
      best_of[wave][g] = m;
    }
    __builtin_amdgcn_wave_barrier();
    // a group is kept if fewer than `keep` groups come before it (a larger score, or an equal one
    // at a lower index)
    for (int g = lane; g < groups; g += PYLON_WAVE) {
      const float mine = best_of[wave][g];
      int before = 0;
      for (int o = 0; o < groups; ++o) {
        const float other = best_of[wave][o];
        before += (other > mine || (other == mine && o < g)) ? 1 : 0;
      }
      if (before >= keep)
        for (int k = 0; k < per_group; ++k) choice[wave][g * per_group + k] = -INFINITY;
    }
    __builtin_amdgcn_wave_barrier();
  }
  float c[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    const int e = lane + PYLON_WAVE * i;
    c[i] = e < n_outputs ? choice[wave][e] : -INFINITY;
  }
  float ident = 0.f;  // lane 0 adds up the identity experts' weights, in the order of the choices
  for (int k = 0; k < top; ++k) {
    float best = -INFINITY, best_s = 0.f;
    int best_e = 0x7fffffff;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const int e = lane + PYLON_WAVE * i;
      if (e < n_outputs && c[i] != -INFINITY && (c[i] > best || (c[i] == best && e < best_e)) && !(c[i] != c[i])) {
        best = c[i];
        best_e = e;
        best_s = s[i];
      }
    }
#pragma unroll
    for (int off = PYLON_WAVE / 2; off > 0; off >>= 1) {
      const float other = __shfl_xor(best, off, PYLON_WAVE);
      const int other_e = __shfl_xor(best_e, off, PYLON_WAVE);
      const float other_s = __shfl_xor(best_s, off, PYLON_WAVE);
      if (other_e != 0x7fffffff && (best_e == 0x7fffffff || other > best || (other == best && other_e < best_e))) {
        best = other;
        best_e = other_e;
        best_s = other_s;
      }
    }
    const bool none = best_e == 0x7fffffff;  // nothing comparable left: an identity of weight nothing
#pragma unroll
    for (int i = 0; i < 8; ++i)
      if (lane + PYLON_WAVE * i == best_e) c[i] = -INFINITY;
    if (lane == 0) {
      const float w = none ? 0.f : best_s * scale;
      const bool identity = none || best_e >= n_experts;
      experts[static_cast<size_t>(t) * top + k] = none ? n_outputs : best_e;
      weights[static_cast<size_t>(t) * top + k] = identity ? 0.f : w;
      if (identity) ident += w;
    }
  }
  if (lane == 0 && identity_weight != nullptr) identity_weight[t] = ident;
}

// logits: float [tokens, n_outputs], rows row_stride apart; correction: null or float [n_outputs];
// the first n_experts outputs are experts, the others identities.  experts int [tokens, top] (an
// identity keeps its index, >= n_experts), weights float [tokens, top] (nothing for an identity),
// identity_weight float [tokens] (null only if n_outputs == n_experts).
extern "C" int pylon_route_scored(int* experts, float* weights, float* identity_weight, const float* logits,
                                  long long row_stride, const float* correction, int tokens, int n_outputs,
                                  int n_experts, int top, int groups, int keep, float scale, hipStream_t stream) {
  PYLON_REQUIRE(tokens >= 0 && n_outputs >= 1 && n_outputs <= MX_MAX_OUTPUTS,
                "route_scored: 1 to %d router outputs, got %d", MX_MAX_OUTPUTS, n_outputs);
  PYLON_REQUIRE(n_experts >= 0 && n_experts <= n_outputs, "route_scored: %d experts among %d outputs", n_experts, n_outputs);
  PYLON_REQUIRE(top >= 1 && top <= n_outputs && top <= MX_MAX_TOP, "route_scored: top %d of %d outputs (at most %d)",
                top, n_outputs, MX_MAX_TOP);
  PYLON_REQUIRE(groups >= 1 && n_outputs % groups == 0 && keep >= 1 && keep <= groups,
                "route_scored: %d outputs do not form %d equal groups of which %d are kept", n_outputs, groups, keep);
  PYLON_REQUIRE(row_stride >= n_outputs, "route_scored: rows of logits overlap");
  PYLON_REQUIRE(identity_weight != nullptr || n_outputs == n_experts, "route_scored: identities need their weight's place");
  if (tokens == 0) return 0;
  hipLaunchKernelGGL(route_scored_kernel, dim3((tokens + 3) / 4), dim3(256), 0, stream, experts, weights,
                     identity_weight, logits, row_stride, correction, tokens, n_outputs, n_experts, top, groups, keep,
                     scale);
  PYLON_LAUNCHED("route_scored");
}

// The dot product of a weight row with a vector in LDS, the lanes of a wave along the row: every
// lane returns its share (the caller adds the lanes up).  Rows of a multiple of 8 elements at
// 16-byte aligned addresses are read 8 elements a lane and trip.
template <typename T>
__device__ __forceinline__ float row_dot_share(const T* __restrict__ row, const float* __restrict__ xs, int n,
                                               int lane, bool wide);

template <>
__device__ __forceinline__ float row_dot_share<float>(const float* __restrict__ row, const float* __restrict__ xs,
                                                      int n, int lane, bool wide) {
  float acc = 0.f;
  if (wide) {
    for (int i = lane * 4; i < n; i += PYLON_WAVE * 4) {
      const float4 w = *reinterpret_cast<const float4*>(row + i);
      acc = fmaf(xs[i], w.x, acc);
      acc = fmaf(xs[i + 1], w.y, acc);
      acc = fmaf(xs[i + 2], w.z, acc);
      acc = fmaf(xs[i + 3], w.w, acc);
    }
  } else {
    for (int i = lane; i < n; i += PYLON_WAVE) acc = fmaf(xs[i], row[i], acc);
  }
  return acc;
}

template <>
__device__ __forceinline__ float row_dot_share<bf16_t>(const bf16_t* __restrict__ row, const float* __restrict__ xs,
                                                       int n, int lane, bool wide) {
  float acc = 0.f;
  if (wide) {
    for (int i = lane * 8; i < n; i += PYLON_WAVE * 8) {
      const uint4 raw = *reinterpret_cast<const uint4*>(row + i);
      const uint32_t w[4] = {raw.x, raw.y, raw.z, raw.w};
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        acc = fmaf(xs[i + 2 * j], __uint_as_float(w[j] << 16), acc);
        acc = fmaf(xs[i + 2 * j + 1], __uint_as_float(w[j] & 0xffff0000u), acc);
      }
    }
  } else {
    for (int i = lane; i < n; i += PYLON_WAVE) acc = fmaf(xs[i], to_float(row[i]), acc);
  }
  return acc;
}

// The lanes' shares of the dot products of ROWS bfloat16 rows with one vector in LDS, rows of a
// multiple of 8 elements: every trip fetches PIECES 16-byte pieces of every row before it multiplies
// any, so that PIECES x ROWS loads of a wave are in flight together (one load at a time, a wave waits a
// memory latency per kilobyte; with four pieces of four rows the registers cost more than the loads
// gain: 8 requests' gate/up 130 us one at a time, 87 with two pieces of four rows, 106 with four).  Every share is added up in the order of the row, as
// row_dot_share adds it.
template <int ROWS, int PIECES>
__device__ __forceinline__ void rows_dot_share(const bf16_t* const (&rows)[ROWS], const float* __restrict__ xs, int n,
                                               int lane, float (&acc)[ROWS]) {
  constexpr int STEP = PYLON_WAVE * 8;
  for (int i = lane * 8; i < n; i += PIECES * STEP) {
    uint4 raw[ROWS][PIECES];
#pragma unroll
    for (int q = 0; q < ROWS; ++q)
#pragma unroll
      for (int p = 0; p < PIECES; ++p)
        raw[q][p] = i + p * STEP < n ? *reinterpret_cast<const uint4*>(rows[q] + i + p * STEP) : uint4{0u, 0u, 0u, 0u};
#pragma unroll
    for (int q = 0; q < ROWS; ++q)
#pragma unroll
      for (int p = 0; p < PIECES; ++p) {
        if (i + p * STEP >= n) continue;
        const float* xv = xs + i + p * STEP;
        const uint32_t w[4] = {raw[q][p].x, raw[q][p].y, raw[q][p].z, raw[q][p].w};
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          acc[q] = fmaf(xv[2 * j], __uint_as_float(w[j] << 16), acc[q]);
          acc[q] = fmaf(xv[2 * j + 1], __uint_as_float(w[j] & 0xffff0000u), acc[q]);
        }
      }
  }
}

// The same two with the vector in LDS as bfloat16 as well (half the room, so more workgroups share a
// unit's LDS, and one LDS read per eight elements): products and order of additions are those of the
// float versions, so the results are the same to the bit.
__device__ __forceinline__ float row_dot_share_packed(const bf16_t* __restrict__ row, const bf16_t* __restrict__ xs, int n,
                                                      int lane, bool wide) {
  float acc = 0.f;
  if (wide) {
    for (int i = lane * 8; i < n; i += PYLON_WAVE * 8) {
      const uint4 raw = *reinterpret_cast<const uint4*>(row + i);
      const uint4 xr = *reinterpret_cast<const uint4*>(xs + i);
      const uint32_t w[4] = {raw.x, raw.y, raw.z, raw.w};
      const uint32_t x[4] = {xr.x, xr.y, xr.z, xr.w};
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        acc = fmaf(__uint_as_float(x[j] << 16), __uint_as_float(w[j] << 16), acc);
        acc = fmaf(__uint_as_float(x[j] & 0xffff0000u), __uint_as_float(w[j] & 0xffff0000u), acc);
      }
    }
  } else {
    for (int i = lane; i < n; i += PYLON_WAVE) acc = fmaf(to_float(xs[i]), to_float(row[i]), acc);
  }
  return acc;
}

template <int ROWS, int PIECES>
__device__ __forceinline__ void rows_dot_share_packed(const bf16_t* const (&rows)[ROWS], const bf16_t* __restrict__ xs,
                                                      int n, int lane, float (&acc)[ROWS]) {
  constexpr int STEP = PYLON_WAVE * 8;
  for (int i = lane * 8; i < n; i += PIECES * STEP) {
    uint4 raw[ROWS][PIECES];
#pragma unroll
    for (int q = 0; q < ROWS; ++q)
#pragma unroll
      for (int p = 0; p < PIECES; ++p)
        raw[q][p] = i + p * STEP < n ? *reinterpret_cast<const uint4*>(rows[q] + i + p * STEP) : uint4{0u, 0u, 0u, 0u};
#pragma unroll
    for (int p = 0; p < PIECES; ++p) {
      if (i + p * STEP >= n) continue;
      const uint4 xr = *reinterpret_cast<const uint4*>(xs + i + p * STEP);
      const uint32_t x[4] = {xr.x, xr.y, xr.z, xr.w};
#pragma unroll
      for (int q = 0; q < ROWS; ++q) {
        const uint32_t w[4] = {raw[q][p].x, raw[q][p].y, raw[q][p].z, raw[q][p].w};
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          acc[q] = fmaf(__uint_as_float(x[j] << 16), __uint_as_float(w[j] << 16), acc[q]);
          acc[q] = fmaf(__uint_as_float(x[j] & 0xffff0000u), __uint_as_float(w[j] & 0xffff0000u), acc[q]);
        }
      }
    }
  }
}

template <typename T>
struct is_bf16 {
  static constexpr bool value = false;
};
template <>
struct is_bf16<bf16_t> {
  static constexpr bool value = true;
};

template <typename TX, typename TW>
__global__ void __launch_bounds__(256)
expert_gate_up_kernel(TX* __restrict__ hidden, const TX* __restrict__ x, long long x_stride,
                      const TW* __restrict__ w, long long w_stride, const int* __restrict__ experts, int top,
                      int ff, int width, int units_per_block, int wide, int act, int n_experts,
                      const float* __restrict__ in_weights) {
  extern __shared__ float xs[];  // the token's input
  const int pair = blockIdx.y, t = pair / top;
  const int lane = threadIdx.x & (PYLON_WAVE - 1), wave = threadIdx.x / PYLON_WAVE;
  const int e = experts[pair];
  if (e >= n_experts) return;  // an identity: nothing to compute (the whole workgroup, before any barrier)
  // with in_weights the expert works on the token's input times the pair's weight (float in LDS)
  const float in_w = in_weights != nullptr ? in_weights[pair] : 1.f;
  for (int i = threadIdx.x; i < width; i += 256) xs[i] = to_float(x[static_cast<size_t>(t) * x_stride + i]) * in_w;
  __syncthreads();
  const int j0 = blockIdx.x * units_per_block;
  const int j1 = j0 + units_per_block < ff ? j0 + units_per_block : ff;
  if (act == 1) {
    // plain experts: hidden = relu(W_up x)^2, a wave four hidden units at a time
    const TW* up1 = w + static_cast<size_t>(e) * ff * w_stride;
    for (int j = j0 + 4 * wave; j < j1; j += 16) {
      float share[4] = {0.f, 0.f, 0.f, 0.f};
      bool done = false;
      if constexpr (is_bf16<TW>::value) {
        if (wide) {
          const bf16_t* rows[4];
#pragma unroll
          for (int q = 0; q < 4; ++q) rows[q] = up1 + static_cast<size_t>(j + q < j1 ? j + q : j1 - 1) * w_stride;
          rows_dot_share<4, 2>(rows, xs, width, lane, share);
          done = true;
        }
      }
      if (!done) {
#pragma unroll
        for (int q = 0; q < 4; ++q)
          if (j + q < j1) share[q] = row_dot_share<TW>(up1 + static_cast<size_t>(j + q) * w_stride, xs, width, lane, wide);
      }
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const float u = fmaxf(wave_sum(share[q]), 0.f);
        if (lane == 0 && j + q < j1) hidden[static_cast<size_t>(pair) * ff + j + q] = from_float<TX>(u * u);
      }
    }
    return;
  }
  const TW* gate = w + static_cast<size_t>(e) * 2 * ff * w_stride;
  const TW* up = gate + static_cast<size_t>(ff) * w_stride;
  // a wave takes two hidden units at a time: the lanes' shares of all four rows first (their loads
  // are in flight together), then the four sums over the lanes
  for (int j = j0 + 2 * wave; j < j1; j += 8) {
    const bool two = j + 1 < j1;
    float gs0, us0, gs1, us1;
    bool done = false;
    if constexpr (is_bf16<TW>::value) {
      if (wide) {  // all four rows together (a lone last unit twice: its second result is dropped)
        const int k = two ? j + 1 : j;
        const bf16_t* const rows[4] = {gate + static_cast<size_t>(j) * w_stride, up + static_cast<size_t>(j) * w_stride,
                                       gate + static_cast<size_t>(k) * w_stride, up + static_cast<size_t>(k) * w_stride};
        float acc[4] = {0.f, 0.f, 0.f, 0.f};
        rows_dot_share<4, 2>(rows, xs, width, lane, acc);
        gs0 = acc[0], us0 = acc[1], gs1 = acc[2], us1 = acc[3];
        done = true;
      }
    }
    if (!done) {
      gs0 = row_dot_share<TW>(gate + static_cast<size_t>(j) * w_stride, xs, width, lane, wide);
      us0 = row_dot_share<TW>(up + static_cast<size_t>(j) * w_stride, xs, width, lane, wide);
      gs1 = two ? row_dot_share<TW>(gate + static_cast<size_t>(j + 1) * w_stride, xs, width, lane, wide) : 0.f;
      us1 = two ? row_dot_share<TW>(up + static_cast<size_t>(j + 1) * w_stride, xs, width, lane, wide) : 0.f;
    }
    const float g0 = wave_sum(gs0), u0 = wave_sum(us0), g1 = wave_sum(gs1), u1 = wave_sum(us1);
    if (lane == 0) {
      hidden[static_cast<size_t>(pair) * ff + j] = from_float<TX>(g0 / (1.0f + expf(-g0)) * u0);
      if (two) hidden[static_cast<size_t>(pair) * ff + j + 1] = from_float<TX>(g1 / (1.0f + expf(-g1)) * u1);
    }
  }
}

// x: [tokens, width] (rows x_stride apart); w: [n_experts, 2 ff, width] (rows w_stride apart), an
// expert's gate rows then its up rows; experts: int [tokens, top]; hidden: [tokens * top, ff].
// act 1: plain experts, w [n_experts, ff, width], hidden = relu(W_up x)^2.  A pair whose expert is
// n_experts or more (an identity) is passed over: its rows of hidden stay as they are.
// in_weights: null, or float [tokens, top]: a pair's expert works on x times the pair's weight.
extern "C" int pylon_expert_gate_up(void* hidden, const void* x, int x_dtype, long long x_stride, const void* w,
                                    int w_dtype, long long w_stride, const int* experts, int tokens, int top, int ff,
                                    int width, int act, int n_experts, const float* in_weights,
                                    hipStream_t stream) {
  PYLON_REQUIRE(act == 0 || act == 1, "expert_gate_up: unknown activation %d", act);
  PYLON_REQUIRE(pylon_valid_dtype(x_dtype) && pylon_valid_dtype(w_dtype), "expert_gate_up: unknown dtype");
  PYLON_REQUIRE(!(x_dtype == PYLON_F32 && w_dtype == PYLON_BF16), "expert_gate_up: float inputs take float weights");
  PYLON_REQUIRE(tokens >= 0 && top >= 1 && ff >= 1 && width >= 1, "expert_gate_up: sizes must be positive");
  PYLON_REQUIRE(x_stride >= width && w_stride >= width, "expert_gate_up: rows overlap");
  PYLON_REQUIRE(top <= MX_MAX_TOP, "expert_gate_up: at most %d experts a token", MX_MAX_TOP);
  const size_t lds = sizeof(float) * width;
  PYLON_REQUIRE(lds <= 64 * 1024, "expert_gate_up: a row of %d elements does not fit LDS", width);
  if (tokens == 0) return 0;
  const int per = w_dtype == PYLON_F32 ? 4 : 8;
  const int wide = (width % per == 0 && w_stride % per == 0 && reinterpret_cast<uintptr_t>(w) % 16 == 0) ? 1 : 0;
  const int units = 32;
  // grid.y is limited to 65535: more pairs go in several launches of whole tokens
  const long long pairs = static_cast<long long>(tokens) * top;
  const long long per_launch = static_cast<long long>(65535 / top) * top;
  for (long long first = 0; first < pairs; first += per_launch) {
    const int n = static_cast<int>(pairs - first < per_launch ? pairs - first : per_launch);
    dim3 grid((ff + units - 1) / units, n), block(256);
    const size_t off = static_cast<size_t>(first);
#define GO(TX, TW)                                                                                               \
  hipLaunchKernelGGL((expert_gate_up_kernel<TX, TW>), grid, block, lds, stream, (TX*)hidden + off * ff,          \
                     (const TX*)x + (off / top) * x_stride, x_stride, (const TW*)w, w_stride, experts + off, top, \
                     ff, width, units, wide, act, n_experts, in_weights != nullptr ? in_weights + off : nullptr)
    if (x_dtype == PYLON_F32) GO(float, float);
    else if (w_dtype == PYLON_F32) GO(bf16_t, float);
    else GO(bf16_t, bf16_t);
#undef GO
  }
  PYLON_LAUNCHED("expert_gate_up");
}

template <typename TH, typename TW>
__global__ void __launch_bounds__(256)
expert_down_kernel(float* __restrict__ out, const TH* __restrict__ hidden, const TW* __restrict__ w,
                   long long w_stride, const int* __restrict__ experts, const float* __restrict__ weights,
                   const float* __restrict__ shared, const float* __restrict__ shared_gate, int top, int ff,
                   int width, int cols_per_block, int wide, int n_experts, const TH* __restrict__ ident_x,
                   long long ident_stride, const float* __restrict__ ident_w) {
  // [top, ff]: the token's hidden activations of its chosen experts; bfloat16 activations for
  // bfloat16 weights stay packed (half the room: twice the workgroups a unit holds), else float
  constexpr bool PACKED = is_bf16<TH>::value && is_bf16<TW>::value;
  extern __shared__ __attribute__((aligned(16))) unsigned char hs_raw[];
  float* hs = reinterpret_cast<float*>(hs_raw);
  bf16_t* hp = reinterpret_cast<bf16_t*>(hs_raw);
  const int t = blockIdx.y;
  const int lane = threadIdx.x & (PYLON_WAVE - 1), wave = threadIdx.x / PYLON_WAVE;
  for (int i = threadIdx.x; i < top * ff; i += 256) {
    // an identity's rows of hidden were never written
    const bool real = experts[static_cast<size_t>(t) * top + i / ff] < n_experts;
    if constexpr (PACKED) {
      bf16_t v;
      v.bits = real ? reinterpret_cast<const bf16_t*>(hidden)[static_cast<size_t>(t) * top * ff + i].bits : uint16_t(0);
      hp[i] = v;
    } else {
      hs[i] = real ? to_float(hidden[static_cast<size_t>(t) * top * ff + i]) : 0.f;
    }
  }
  __syncthreads();
  // identity experts: the token's input itself, times the sum of their weights
  const float iw = ident_w != nullptr ? ident_w[t] : 0.f;
  const TH* ix = ident_x != nullptr ? ident_x + static_cast<size_t>(t) * ident_stride : nullptr;
  const int c0 = blockIdx.x * cols_per_block;
  const int c1 = c0 + cols_per_block < width ? c0 + cols_per_block : width;
  if constexpr (is_bf16<TW>::value) {
    if (wide && cols_per_block == 16) {
      // a wave takes four neighbouring columns: per chosen expert the lanes' shares of its four rows
      // with all their loads in flight together, weighed in the order of the token's choices; one sum
      // over the lanes per column at the end
      const int c = c0 + 4 * wave;
      if (c >= c1) return;
      float share[4] = {0.f, 0.f, 0.f, 0.f};
      for (int s = 0; s < top; ++s) {
        const int e = experts[static_cast<size_t>(t) * top + s];
        if (e >= n_experts) continue;
        const bf16_t* base = w + static_cast<size_t>(e) * width * w_stride;
        const bf16_t* rows[4];
#pragma unroll
        for (int q = 0; q < 4; ++q) rows[q] = base + static_cast<size_t>(c + q < c1 ? c + q : c1 - 1) * w_stride;
        float part[4] = {0.f, 0.f, 0.f, 0.f};
        if constexpr (PACKED) rows_dot_share_packed<4, 2>(rows, hp + s * ff, ff, lane, part);
        else rows_dot_share<4, 2>(rows, hs + s * ff, ff, lane, part);
        const float weight = weights[static_cast<size_t>(t) * top + s];
#pragma unroll
        for (int q = 0; q < 4; ++q) share[q] = fmaf(weight, part[q], share[q]);
      }
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        float acc = wave_sum(share[q]);
        if (lane == 0 && c + q < c1) {
          if (shared != nullptr) {
            const float g = shared_gate != nullptr ? shared_gate[t] : 1.f;
            acc = fmaf(g, shared[static_cast<size_t>(t) * width + c + q], acc);
          }
          if (ix != nullptr) acc = fmaf(iw, to_float(ix[c + q]), acc);
          out[static_cast<size_t>(t) * width + c + q] = acc;
        }
      }
      return;
    }
  }
  for (int c = c0 + wave; c < c1; c += 4) {
    // every lane weighs its shares of the chosen experts' rows, in the order of the token's choices;
    // one sum over the lanes at the end
    float share = 0.f;
    for (int s = 0; s < top; ++s) {
      const int e = experts[static_cast<size_t>(t) * top + s];
      if (e >= n_experts) continue;
      const TW* row = w + (static_cast<size_t>(e) * width + c) * w_stride;
      float part;
      if constexpr (PACKED) part = row_dot_share_packed(reinterpret_cast<const bf16_t*>(row), hp + s * ff, ff, lane, wide);
      else part = row_dot_share<TW>(row, hs + s * ff, ff, lane, wide);
      share = fmaf(weights[static_cast<size_t>(t) * top + s], part, share);
    }
    float acc = wave_sum(share);
    if (lane == 0) {
      if (shared != nullptr) {
        const float g = shared_gate != nullptr ? shared_gate[t] : 1.f;
        acc = fmaf(g, shared[static_cast<size_t>(t) * width + c], acc);
      }
      if (ix != nullptr) acc = fmaf(iw, to_float(ix[c]), acc);
      out[static_cast<size_t>(t) * width + c] = acc;
    }
  }
}

// hidden: [tokens * top, ff]; w: [n_experts, width, ff] (rows w_stride apart); experts int and
// weights float [tokens, top]; shared: null or float [tokens, width], multiplied by shared_gate[t]
// (null: by one) and added; out: float [tokens, width].  A pair whose expert is n_experts or more is
// passed over; ident_x (null, or [tokens, width] of h_dtype, rows ident_stride apart) times
// ident_w[t] is added: the identity experts' share.
extern "C" int pylon_expert_down(float* out, const void* hidden, int h_dtype, const void* w, int w_dtype,
                                 long long w_stride, const int* experts, const float* weights, const float* shared,
                                 const float* shared_gate, int tokens, int top, int ff, int width, int n_experts,
                                 const void* ident_x, long long ident_stride, const float* ident_w,
                                 hipStream_t stream) {
  PYLON_REQUIRE((ident_x == nullptr) == (ident_w == nullptr), "expert_down: identities need inputs and weights");
  PYLON_REQUIRE(pylon_valid_dtype(h_dtype) && pylon_valid_dtype(w_dtype), "expert_down: unknown dtype");
  PYLON_REQUIRE(!(h_dtype == PYLON_F32 && w_dtype == PYLON_BF16), "expert_down: float inputs take float weights");
  PYLON_REQUIRE(tokens >= 0 && top >= 1 && ff >= 1 && width >= 1, "expert_down: sizes must be positive");
  PYLON_REQUIRE(w_stride >= ff, "expert_down: rows overlap");
  const bool packed = h_dtype == PYLON_BF16 && w_dtype == PYLON_BF16;
  const size_t lds = (packed ? sizeof(uint16_t) : sizeof(float)) * top * ff;
  // a workgroup of this device may hold 160 KB; beyond 64 KB a kernel has to be told
  PYLON_REQUIRE(lds <= 160 * 1024, "expert_down: %d experts of %d hidden units do not fit LDS", top, ff);
  if (tokens == 0) return 0;
  const int per = w_dtype == PYLON_F32 ? 4 : 8;
  const int wide = (ff % per == 0 && w_stride % per == 0 && reinterpret_cast<uintptr_t>(w) % 16 == 0) ? 1 : 0;
  const int cols = 16;
  for (int first = 0; first < tokens; first += 65535) {
    const int n = tokens - first < 65535 ? tokens - first : 65535;
    dim3 grid((width + cols - 1) / cols, n), block(256);
    const size_t off = static_cast<size_t>(first);
#define GO(TH, TW)                                                                                              \
  do {                                                                                                          \
    if (lds > 64 * 1024)                                                                                        \
      (void)hipFuncSetAttribute(reinterpret_cast<const void*>(&expert_down_kernel<TH, TW>),                     \
                                hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(lds));             \
    hipLaunchKernelGGL((expert_down_kernel<TH, TW>), grid, block, lds, stream, out + off * width,               \
                       (const TH*)hidden + off * top * ff, (const TW*)w, w_stride, experts + off * top,         \
                       weights + off * top, shared != nullptr ? shared + off * width : nullptr,                 \
                       shared_gate != nullptr ? shared_gate + off : nullptr, top, ff, width, cols, wide,        \
                       n_experts, ident_x != nullptr ? (const TH*)ident_x + off * ident_stride : nullptr,       \
                       ident_stride, ident_w != nullptr ? ident_w + off : nullptr);                             \
  } while (0)
    if (h_dtype == PYLON_F32) GO(float, float);
    else if (w_dtype == PYLON_F32) GO(bf16_t, float);
    else GO(bf16_t, bf16_t);
#undef GO
  }
  PYLON_LAUNCHED("expert_down");
}

// ---- many tokens: the experts' products on the matrix cores, expert by expert ------------------
// The (token, choice) pairs are sorted by expert (on the device, by the caller); offsets[e] is the
// first sorted pair of expert e.  A workgroup takes 64 or 128 sorted pairs of one expert (128 where
// the experts have that many on average: the larger tile re-reads the weights half as often) and
// 128 output columns: four waves of 32 columns each, all rows, operands fetched in the shape the matrix
// instruction wants them (a lane: 8 neighbouring elements of one row), the next 32 elements of
// K in flight while the current ones are multiplied.  Which (expert, rows) a workgroup has it
// finds from the offsets itself; the grid is the most tiles there can be, and the workgroups
// beyond the last tile leave at once.  Every output element is one chain of additions along K,
// whatever the batch.
typedef __bf16 mx_bf16x8 __attribute__((ext_vector_type(8)));
typedef float mx_floatx4 __attribute__((ext_vector_type(4)));

#define MX_WAVE_COLS 32

template <int ACT, int MT, typename TO>
__global__ void __launch_bounds__(256)
grouped_rows_kernel(TO* __restrict__ out, long long ldo, const uint16_t* __restrict__ x, long long ldx,
                    const int* __restrict__ row_index, const uint16_t* __restrict__ w, long long ldw,
                    long long expert_rows, const int* __restrict__ offsets, int n_experts, int N, int K,
                    const float* __restrict__ row_scale) {
  constexpr bool GLU = ACT == 1;  // ACT: 0 the sums as they are, 1 silu(gate) * up, 2 the square of relu
  constexpr int MX_TM = 16 * MT;  // rows of a tile
  constexpr int J = GLU ? 4 : 2;  // weight tiles of a wave: GLU: two of gate rows, then the two of their up rows
  const int lane = threadIdx.x & (PYLON_WAVE - 1), wave = threadIdx.x / PYLON_WAVE;
  const int r = lane & 15, g = lane >> 4;
  // this workgroup's expert and rows
  int tile = blockIdx.x, e = 0, row0 = 0, rows = 0;
  for (; e < n_experts; ++e) {
    const int begin = offsets[e], count = offsets[e + 1] - begin;
    const int tiles = (count + MX_TM - 1) / MX_TM;
    if (tile < tiles) {
      row0 = begin + tile * MX_TM;
      rows = count - tile * MX_TM < MX_TM ? count - tile * MX_TM : MX_TM;
      break;
    }
    tile -= tiles;
  }
  if (e == n_experts) return;
  const int n0 = blockIdx.y * (4 * MX_WAVE_COLS) + wave * MX_WAVE_COLS;
  if (n0 >= N) return;

  const uint16_t* xp[MT];
#pragma unroll
  for (int t = 0; t < MT; ++t) {
    const int local = 16 * t + r < rows ? 16 * t + r : 0;  // rows past the tile's last repeat its first
    const int m = row0 + local;
    xp[t] = x + static_cast<size_t>(row_index != nullptr ? row_index[m] : m) * ldx + 8 * g;
  }
  const uint16_t* wp[J];
#pragma unroll
  for (int j = 0; j < J; ++j) {
    int n = n0 + 16 * (j & 1) + r;
    if (n >= N) n = N - 1;  // columns past the last repeat it; they are not stored
    const size_t row = static_cast<size_t>(e) * expert_rows + (GLU && j >= 2 ? N : 0) + n;
    wp[j] = w + row * ldw + 8 * g;
  }
  mx_floatx4 acc[J][MT];
#pragma unroll
  for (int j = 0; j < J; ++j)
#pragma unroll
    for (int t = 0; t < MT; ++t) acc[j][t] = mx_floatx4{0.f, 0.f, 0.f, 0.f};

  const mx_bf16x8 zero = __builtin_bit_cast(mx_bf16x8, uint4{0u, 0u, 0u, 0u});
  auto fetch = [&](mx_bf16x8(&xa)[MT], mx_bf16x8(&wa)[J], int k) {
    const bool ok = k + 8 * g < K;  // K is a multiple of 8: a lane's 8 elements are all inside or all outside
#pragma unroll
    for (int t = 0; t < MT; ++t) xa[t] = ok ? *reinterpret_cast<const mx_bf16x8*>(xp[t] + k) : zero;
#pragma unroll
    for (int j = 0; j < J; ++j) wa[j] = ok ? *reinterpret_cast<const mx_bf16x8*>(wp[j] + k) : zero;
  };
  auto multiply = [&](const mx_bf16x8(&xa)[MT], const mx_bf16x8(&wa)[J]) {
#pragma unroll
    for (int j = 0; j < J; ++j)
#pragma unroll
      for (int t = 0; t < MT; ++t) acc[j][t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wa[j], xa[t], acc[j][t], 0, 0, 0);
  };
  mx_bf16x8 xa[MT], wa[J], xb[MT], wb[J];
  fetch(xa, wa, 0);
  for (int k = 0; k < K; k += 64) {
    if (k + 32 < K) fetch(xb, wb, k + 32);
    multiply(xa, wa);
    if (k + 32 < K) {
      if (k + 64 < K) fetch(xa, wa, k + 64);
      multiply(xb, wb);
    }
  }
  // acc[j][t][i] is the sum for row 16 t + r and column n0 + 16 (j & 1) + 4 g + i
#pragma unroll
  for (int t = 0; t < MT; ++t) {
    if (16 * t + r >= rows) continue;
    TO* orow = out + static_cast<size_t>(row0 + 16 * t + r) * ldo;
    // a row's scale: the products are linear, so the sums of the scaled input are the scaled sums
    const float rs = row_scale != nullptr ? row_scale[row0 + 16 * t + r] : 1.f;
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int n = n0 + 16 * j + 4 * g + i;
        if (n >= N) continue;
        float v = acc[j][t][i] * rs;
        if constexpr (GLU) v = v / (1.0f + expf(-v)) * (acc[2 + j][t][i] * rs);
        if constexpr (ACT == 2) v = fmaxf(v, 0.f) * fmaxf(v, 0.f);
        orow[n] = from_float<TO>(v);
      }
  }
}

// The same product for experts with many pairs each: tiles of 128 pairs x 256 output columns
// (with the gated epilogue: 128 gate and their 128 up columns), K in pieces of 64 elements that all
// 256 threads bring into LDS together, whole 128-byte row segments at a time (a thread 16 bytes of
// one row; 32 rows further on its next load), the next piece on its way into registers while the
// matrix instructions read the current one from LDS.  Rows lie 144 bytes apart in LDS, so that
// the 16 rows of an operand fall into different banks.  A wave takes all 128 rows and a quarter of
// the columns; the 16-row pieces past a tile's last pair are not multiplied.
#define GT_ROWS 128
#define GT_COLS 128
#define GT_K 64
#define GT_PITCH 144

template <int ACT, typename TO>
__global__ void __launch_bounds__(256, 2)
grouped_tiles_kernel(TO* __restrict__ out, long long ldo, const uint16_t* __restrict__ x, long long ldx,
                     const int* __restrict__ row_index, const uint16_t* __restrict__ w, long long ldw,
                     long long expert_rows, const int* __restrict__ offsets, int n_experts, int N, int K,
                     const float* __restrict__ row_scale) {
  constexpr bool GLU = ACT == 1;
  constexpr int WROWS = 2 * GT_COLS;  // GLU: 128 gate rows and their 128 up rows; else 256 output columns
  constexpr int TILE_COLS = GLU ? GT_COLS : 2 * GT_COLS, WAVE_COLS = TILE_COLS / 4;
  constexpr int XLOADS = GT_ROWS / 32, LOADS = (GT_ROWS + WROWS) / 32;
  constexpr int J = 4, MT = GT_ROWS / 16;
  __shared__ __attribute__((aligned(16))) unsigned char lds[(GT_ROWS + WROWS) * GT_PITCH];
  const int tid = threadIdx.x, lane = tid & (PYLON_WAVE - 1), wave = tid / PYLON_WAVE;
  const int r = lane & 15, g = lane >> 4;
  int tile = blockIdx.x, e = 0, row0 = 0, rows = 0;
  for (; e < n_experts; ++e) {
    const int begin = offsets[e], count = offsets[e + 1] - begin;
    const int tiles = (count + GT_ROWS - 1) / GT_ROWS;
    if (tile < tiles) {
      row0 = begin + tile * GT_ROWS;
      rows = count - tile * GT_ROWS < GT_ROWS ? count - tile * GT_ROWS : GT_ROWS;
      break;
    }
    tile -= tiles;
  }
  if (e == n_experts) return;  // the whole workgroup: no barrier is missed
  const int n0 = blockIdx.y * TILE_COLS;

  // what this thread brings: the 16-byte piece `piece` of rows lrow, lrow + 32, ... of the tile in LDS
  const int piece = tid & 7, lrow = tid >> 3;
  unsigned src[LOADS];  // in elements, from x (the first XLOADS) or from w
#pragma unroll
  for (int i = 0; i < LOADS; ++i) {
    const int row = lrow + 32 * i;
    if (i < XLOADS) {
      const int m = row0 + (row < rows ? row : 0);  // rows past the tile's last repeat its first
      src[i] = static_cast<unsigned>((row_index != nullptr ? row_index[m] : m) * ldx + piece * 8);
    } else {
      const int c = row - GT_ROWS;
      const bool up = GLU && c >= GT_COLS;
      int n = n0 + (up ? c - GT_COLS : c);
      if (n >= N) n = N - 1;  // columns past the last repeat it; they are not stored
      src[i] = static_cast<unsigned>((e * expert_rows + (up ? N : 0) + n) * ldw + piece * 8);
    }
  }
  uint4 held[LOADS];
  auto fetch = [&](int k) {
    const bool ok = k + piece * 8 < K;  // K is a multiple of 8
#pragma unroll
    for (int i = 0; i < LOADS; ++i)
      held[i] = ok ? *reinterpret_cast<const uint4*>((i < XLOADS ? x : w) + src[i] + k) : uint4{0u, 0u, 0u, 0u};
  };
  mx_floatx4 acc[J][MT];
#pragma unroll
  for (int j = 0; j < J; ++j)
#pragma unroll
    for (int t = 0; t < MT; ++t) acc[j][t] = mx_floatx4{0.f, 0.f, 0.f, 0.f};

  fetch(0);
  for (int k = 0; k < K; k += GT_K) {
#pragma unroll
    for (int i = 0; i < LOADS; ++i) *reinterpret_cast<uint4*>(lds + (lrow + 32 * i) * GT_PITCH + piece * 16) = held[i];
    __syncthreads();
    if (k + GT_K < K) fetch(k + GT_K);
#pragma unroll
    for (int h = 0; h < GT_K / 32; ++h) {
      mx_bf16x8 wf[J];
#pragma unroll
      for (int j = 0; j < J; ++j) {
        const int row = GLU ? GT_ROWS + (j >= 2 ? GT_COLS : 0) + wave * 32 + 16 * (j & 1) + r
                            : GT_ROWS + wave * WAVE_COLS + 16 * j + r;
        wf[j] = *reinterpret_cast<const mx_bf16x8*>(lds + row * GT_PITCH + h * 64 + g * 16);
      }
#pragma unroll
      for (int t = 0; t < MT; ++t) {
        if (16 * t >= rows) continue;  // a tile's last rows: nothing to multiply (the same for the whole workgroup)
        const mx_bf16x8 xf = *reinterpret_cast<const mx_bf16x8*>(lds + (16 * t + r) * GT_PITCH + h * 64 + g * 16);
#pragma unroll
        for (int j = 0; j < J; ++j) acc[j][t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wf[j], xf, acc[j][t], 0, 0, 0);
      }
    }
    __syncthreads();
  }
  // acc[j][t][i] is the sum for row 16 t + r and, gated, column n0 + 32 wave + 16 (j & 1) + 4 g + i
  // (j < 2 the gate's, j >= 2 the up's), else column n0 + 64 wave + 16 j + 4 g + i
#pragma unroll
  for (int t = 0; t < MT; ++t) {
    if (16 * t + r >= rows) continue;
    TO* orow = out + static_cast<size_t>(row0 + 16 * t + r) * ldo;
    const float rs = row_scale != nullptr ? row_scale[row0 + 16 * t + r] : 1.f;
#pragma unroll
    for (int j = 0; j < (GLU ? 2 : J); ++j)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int n = n0 + WAVE_COLS * wave + 16 * j + 4 * g + i;
        if (n >= N) continue;
        float v = acc[j][t][i] * rs;
        if constexpr (GLU) v = v / (1.0f + expf(-v)) * (acc[2 + j][t][i] * rs);
        if constexpr (ACT == 2) v = fmaxf(v, 0.f) * fmaxf(v, 0.f);
        orow[n] = from_float<TO>(v);
      }
  }
}

// Tiles of 128 pairs through LDS pay once the experts have that many pairs on average; their
// 32-bit offsets must span both operands.
static bool grouped_large(int pairs, int n_experts, long long x_elements, long long w_elements) {
  return pairs / n_experts >= GT_ROWS && x_elements < (1ll << 32) && w_elements < (1ll << 32);
}

static int grouped_checks(const char* name, const void* x, long long ldx, const void* w, long long ldw, int K, int N,
                          int pairs, int n_experts) {
  PYLON_REQUIRE(pairs >= 0 && n_experts >= 1 && N >= 1 && K >= 8 && K % 8 == 0,
                "%s: rows of a multiple of 8 elements, got %d", name, K);
  PYLON_REQUIRE(ldx % 8 == 0 && ldw % 8 == 0 && reinterpret_cast<uintptr_t>(x) % 16 == 0 &&
                    reinterpret_cast<uintptr_t>(w) % 16 == 0,
                "%s: rows must start at 16-byte aligned addresses", name);
  PYLON_REQUIRE(ldx >= K && ldw >= K, "%s: rows overlap", name);
  return 0;
}

// hidden[p] = silu(W_gate[e] x[row_index[p]]) * (W_up[e] x[row_index[p]]) for the sorted pairs p of
// every expert e (offsets: int [n_experts + 1]); x bfloat16 [tokens, width]; w bfloat16
// [n_experts * 2 ff, width]; hidden bfloat16 [pairs, ff]; tokens_bound: the rows of x.  act 1: plain
// experts, hidden[p] = relu(W_up[e] x)^2 with w [n_experts * ff, width].  pairs counts the sorted
// pairs of these n_experts experts only (identities' pairs lie behind them).  row_scale: null, or
// float [pairs]: sorted pair p's expert works on its input times row_scale[p] (gated experts).
extern "C" int pylon_grouped_gate_up(void* hidden, const void* x, long long ldx, const int* row_index, const void* w,
                                     long long ldw, const int* offsets, int pairs, int n_experts, int ff, int width,
                                     int tokens_bound, int act, const float* row_scale, hipStream_t stream) {
  PYLON_REQUIRE(row_scale == nullptr || act == 0, "grouped_gate_up: a scale per pair goes with gated experts");
  if (grouped_checks("grouped_gate_up", x, ldx, w, ldw, width, ff, pairs, n_experts)) return 1;
  PYLON_REQUIRE(act == 0 || act == 1, "grouped_gate_up: unknown activation %d", act);
  if (pairs == 0) return 0;
  if (act == 1) {
    // plain experts: w [n_experts * ff, width], hidden = relu(W_up x)^2; tiles of 256 columns where large
    const bool large1 = grouped_large(pairs, n_experts, tokens_bound * ldx, 1ll * n_experts * ff * ldw);
    const int tile1 = large1 ? GT_ROWS : 64, cols1 = large1 ? 2 * GT_COLS : 4 * MX_WAVE_COLS;
    dim3 grid1(pairs / tile1 + n_experts, (ff + cols1 - 1) / cols1), block1(256);
    PYLON_REQUIRE(grid1.y <= 65535, "grouped_gate_up: too many columns for one launch");
    if (large1)
      hipLaunchKernelGGL((grouped_tiles_kernel<2, bf16_t>), grid1, block1, 0, stream, (bf16_t*)hidden, (long long)ff,
                         (const uint16_t*)x, ldx, row_index, (const uint16_t*)w, ldw, (long long)ff, offsets, n_experts,
                         ff, width, nullptr);
    else
      hipLaunchKernelGGL((grouped_rows_kernel<2, 4, bf16_t>), grid1, block1, 0, stream, (bf16_t*)hidden, (long long)ff,
                         (const uint16_t*)x, ldx, row_index, (const uint16_t*)w, ldw, (long long)ff, offsets, n_experts,
                         ff, width, nullptr);
    PYLON_LAUNCHED("grouped_gate_up");
  }
  const bool large = grouped_large(pairs, n_experts, tokens_bound * ldx, 2ll * n_experts * ff * ldw);
  const int tile = large ? GT_ROWS : 64;
  dim3 grid(pairs / tile + n_experts, (ff + 4 * MX_WAVE_COLS - 1) / (4 * MX_WAVE_COLS)), block(256);
  PYLON_REQUIRE(grid.y <= 65535, "grouped_gate_up: too many columns for one launch");
  if (large)
    hipLaunchKernelGGL((grouped_tiles_kernel<1, bf16_t>), grid, block, 0, stream, (bf16_t*)hidden, (long long)ff,
                       (const uint16_t*)x, ldx, row_index, (const uint16_t*)w, ldw, 2ll * ff, offsets, n_experts, ff,
                       width, row_scale);
  else
    hipLaunchKernelGGL((grouped_rows_kernel<1, 4, bf16_t>), grid, block, 0, stream, (bf16_t*)hidden,
                       (long long)ff, (const uint16_t*)x, ldx, row_index, (const uint16_t*)w, ldw, 2ll * ff, offsets,
                       n_experts, ff, width, row_scale);
  PYLON_LAUNCHED("grouped_gate_up");
}

// y[p] = W_down[e] hidden[p] for the sorted pairs p of every expert e: hidden bfloat16 [pairs, ff],
// w bfloat16 [n_experts * width, ff], y float [pairs, width].
extern "C" int pylon_grouped_down(float* y, const void* hidden, long long ldh, const void* w, long long ldw,
                                  const int* offsets, int pairs, int n_experts, int ff, int width,
                                  hipStream_t stream) {
  if (grouped_checks("grouped_down", hidden, ldh, w, ldw, ff, width, pairs, n_experts)) return 1;
  if (pairs == 0) return 0;
  const bool large = grouped_large(pairs, n_experts, pairs * ldh, 1ll * n_experts * width * ldw);
  const int tile = large ? GT_ROWS : 64, cols = large ? 2 * GT_COLS : 4 * MX_WAVE_COLS;
  dim3 grid(pairs / tile + n_experts, (width + cols - 1) / cols), block(256);
  PYLON_REQUIRE(grid.y <= 65535, "grouped_down: too many columns for one launch");
  if (large)
    hipLaunchKernelGGL((grouped_tiles_kernel<0, float>), grid, block, 0, stream, y, (long long)width,
                       (const uint16_t*)hidden, ldh, nullptr, (const uint16_t*)w, ldw, (long long)width, offsets,
                       n_experts, width, ff, nullptr);
  else
    hipLaunchKernelGGL((grouped_rows_kernel<0, 4, float>), grid, block, 0, stream, y, (long long)width,
                       (const uint16_t*)hidden, ldh, nullptr, (const uint16_t*)w, ldw, (long long)width, offsets,
                       n_experts, width, ff, nullptr);
  PYLON_LAUNCHED("grouped_down");
}

__global__ void __launch_bounds__(256)
expert_combine_kernel(float* __restrict__ out, const float* __restrict__ y, const int* __restrict__ place,
                      const float* __restrict__ weights, const float* __restrict__ shared,
                      const float* __restrict__ shared_gate, int top, int width, const int* __restrict__ real_end,
                      const uint16_t* __restrict__ ident_x, long long ident_stride, const float* __restrict__ ident_w) {
  const int t = blockIdx.y;
  const int c = blockIdx.x * 256 + threadIdx.x;
  if (c >= width) return;
  float acc = 0.f;
  const int real_pairs = real_end != nullptr ? real_end[0] : 0x7fffffff;
  for (int s = 0; s < top; ++s) {
    const int p = place[static_cast<size_t>(t) * top + s];
    if (p >= real_pairs) continue;  // an identity's pair: no expert has written its row of y
    acc = fmaf(weights[static_cast<size_t>(t) * top + s], y[static_cast<size_t>(p) * width + c], acc);
  }
  if (shared != nullptr) acc = fmaf(shared_gate != nullptr ? shared_gate[t] : 1.f, shared[static_cast<size_t>(t) * width + c], acc);
  if (ident_x != nullptr)
    acc = fmaf(ident_w[t], bf16_bits_to_float(ident_x[static_cast<size_t>(t) * ident_stride + c]), acc);
  out[static_cast<size_t>(t) * width + c] = acc;
}

// out[t] = sum_s weights[t, s] y[place[t, s]] (+ shared_gate[t] * shared[t]): the experts' outputs of
// the sorted pairs brought back to their tokens, in the order of the token's choices.
// Sorted pairs from real_end[0] on (null: none) belong to identity experts: ident_x (null, or bfloat16 [tokens, width],
// rows ident_stride apart) times ident_w[t] stands for them.
extern "C" int pylon_expert_combine(float* out, const float* y, const int* place, const float* weights,
                                    const float* shared, const float* shared_gate, int tokens, int top, int width,
                                    const int* real_end, const void* ident_x, long long ident_stride, const float* ident_w,
                                    hipStream_t stream) {
  PYLON_REQUIRE(tokens >= 0 && top >= 1 && width >= 1, "expert_combine: sizes must be positive");
  PYLON_REQUIRE((ident_x == nullptr) == (ident_w == nullptr), "expert_combine: identities need inputs and weights");
  if (tokens == 0) return 0;
  for (int first = 0; first < tokens; first += 65535) {
    const int n = tokens - first < 65535 ? tokens - first : 65535;
    const size_t off = static_cast<size_t>(first);
    hipLaunchKernelGGL(expert_combine_kernel, dim3((width + 255) / 256, n), dim3(256), 0, stream, out + off * width, y,
                       place + off * top, weights + off * top, shared != nullptr ? shared + off * width : nullptr,
                       shared_gate != nullptr ? shared_gate + off : nullptr, top, width, real_end,
                       ident_x != nullptr ? (const uint16_t*)ident_x + off * ident_stride : nullptr, ident_stride,
                       ident_w != nullptr ? ident_w + off : nullptr);
  }
  PYLON_LAUNCHED("expert_combine");
}
