// The residual sum of a layer whose sublayers are normed on both sides, fused with the norm
// that follows it:
//
//   d = sum_p delta[p]                      (the sublayer's output, maybe as partial sums)
//   x = resid + post_gain * d / rms(d)      (rms(v) = sqrt(mean(v^2) + eps); without post_gain: x = resid + d)
//   or, with a bias and a scale per element (a projection's bias that was left for here, a layer's
//   learned scale of its sublayers' outputs): x = resid + scale * (d + bias)
//   out = gain * x / rms(x)                 (gain: one number, or one per element)
//
// All of it in float; `out` is rounded once on the store.  One workgroup per output row, the
// row held in registers between the passes, so that a row costs one trip to memory.  The order
// of every sum depends on the row's length and the workgroup's size only.
#include "common.h"

// ND: the number of partial sums when it is one of the usual counts (all their loads are then sent for
// before the first addition; a loop over a count only known at run time would wait for memory once
// per partial sum), 0 for any other count.  The order of the additions is the same either way.
template <typename TD, typename TO, int PER, int ND>
__global__ void add_normed_rmsnorm_kernel(TO* __restrict__ out, float* resid, const TD* __restrict__ delta,
                                          int n_delta, long long delta_stride, const float* __restrict__ post_gain,
                                          float post_eps, const float* __restrict__ gain, int gain_stride,
                                          const int* __restrict__ row_idx, int dim, float eps, int write_resid,
                                          const float* __restrict__ delta_scale, const float* __restrict__ delta_bias) {
  __shared__ float scratch[16];
  const int r_out = blockIdx.x;
  const int r_in = row_idx ? row_idx[r_out] : r_out;
  float* xr = resid + static_cast<size_t>(r_in) * dim;
  const TD* dr = delta ? delta + static_cast<size_t>(r_in) * dim : nullptr;
  TO* yr = out + static_cast<size_t>(r_out) * dim;
  float x[PER];
  if (dr) {
    float d[PER];
    float ss = 0.f;
    if (ND > 0) {
      float e[PER][ND > 0 ? ND : 1];
#pragma unroll
      for (int n = 0; n < PER; ++n) {
        const int i = threadIdx.x + n * blockDim.x;
#pragma unroll
        for (int p = 0; p < ND; ++p) e[n][p] = (i < dim) ? to_float(dr[i + p * delta_stride]) : 0.f;
      }
#pragma unroll
      for (int n = 0; n < PER; ++n) {
        float v = e[n][0];
#pragma unroll
        for (int p = 1; p < ND; ++p) v += e[n][p];
        d[n] = v;
        ss += v * v;
      }
    } else {
#pragma unroll
      for (int n = 0; n < PER; ++n) {
        const int i = threadIdx.x + n * blockDim.x;
        d[n] = 0.f;
        if (i < dim) {
          float v = to_float(dr[i]);
          for (int p = 1; p < n_delta; ++p) v += to_float(dr[i + p * delta_stride]);
          d[n] = v;
          ss += v * v;
        }
      }
    }
    if (delta_bias) {  // before the sum of squares is used: a biased output is normed as a whole
      ss = 0.f;
#pragma unroll
      for (int n = 0; n < PER; ++n) {
        const int i = threadIdx.x + n * blockDim.x;
        if (i < dim) {
          d[n] += delta_bias[i];
          ss += d[n] * d[n];
        }
      }
    }
    float mult = 1.0f;
    if (post_gain) {
      const float total = block_sum(ss, scratch);
      mult = 1.0f / sqrtf(total / static_cast<float>(dim) + post_eps);
    }
    const float pg = post_gain ? post_gain[0] : 1.0f;
#pragma unroll
    for (int n = 0; n < PER; ++n) {
      const int i = threadIdx.x + n * blockDim.x;
      x[n] = 0.f;
      if (i < dim) {
        x[n] = delta_scale ? fmaf(delta_scale[i], d[n], xr[i]) : xr[i] + (d[n] * mult) * pg;
        if (write_resid) xr[i] = x[n];
      }
    }
  } else {
#pragma unroll
    for (int n = 0; n < PER; ++n) {
      const int i = threadIdx.x + n * blockDim.x;
      x[n] = i < dim ? xr[i] : 0.f;
    }
  }
  if (out == nullptr) return;
  float ss = 0.f;
#pragma unroll
  for (int n = 0; n < PER; ++n) ss += x[n] * x[n];
  const float total = block_sum(ss, scratch);
  const float inv = 1.0f / sqrtf(total / static_cast<float>(dim) + eps);
#pragma unroll
  for (int n = 0; n < PER; ++n) {
    const int i = threadIdx.x + n * blockDim.x;
    if (i < dim) yr[i] = from_float<TO>((x[n] * inv) * gain[static_cast<size_t>(i) * gain_stride]);
  }
}

// resid: float [tokens, dim], updated in place unless row_idx picks rows.  delta: null (nothing
// is added), [tokens, dim], or n_delta such tensors delta_stride elements apart.  post_gain: null
// (delta is added as it is) or one float.  gain: one float (gain_stride 0) or dim floats
// (gain_stride 1).  out: [rows, dim] of out_dtype, or null (only the sum is formed).
// delta_scale, delta_bias: null or dim floats each (the scale not together with post_gain).
extern "C" int pylon_add_normed_rmsnorm(void* out, int out_dtype, float* resid, const void* delta, int delta_dtype,
                                        int n_delta, long long delta_stride, const float* post_gain, float post_eps,
                                        const float* gain, int gain_stride, const int* row_idx, int rows, int dim,
                                        float eps, const float* delta_scale, const float* delta_bias,
                                        hipStream_t stream) {
  PYLON_REQUIRE(pylon_valid_dtype(out_dtype) && pylon_valid_dtype(delta_dtype), "add_normed_rmsnorm: unknown dtype");
  PYLON_REQUIRE(rows >= 0 && dim > 0 && dim <= 16384, "add_normed_rmsnorm: rows of 1 to 16384 elements, got %d", dim);
  PYLON_REQUIRE(n_delta >= 1 && (gain_stride == 0 || gain_stride == 1), "add_normed_rmsnorm: bad delta count or gain stride");
  PYLON_REQUIRE(out == nullptr || gain != nullptr, "add_normed_rmsnorm: a norm needs its gain");
  PYLON_REQUIRE(out != nullptr || (delta != nullptr && row_idx == nullptr), "add_normed_rmsnorm: nothing to do");
  PYLON_REQUIRE(delta_scale == nullptr || post_gain == nullptr,
                "add_normed_rmsnorm: a scale per element or a norm of the output, not both");
  PYLON_REQUIRE((delta_scale == nullptr && delta_bias == nullptr) || delta != nullptr,
                "add_normed_rmsnorm: a scale or a bias needs the output they belong to");
  if (rows == 0) return 0;
  const int write_resid = row_idx == nullptr ? 1 : 0;
  const int threads = dim <= 256 ? 64 : (dim <= 2048 ? 256 : (dim <= 8192 ? 512 : 1024));
  const int per = (dim + threads - 1) / threads;
  dim3 grid(rows), block(threads);
#define GO(TD, TO, PER, ND)                                                                                     \
  hipLaunchKernelGGL((add_normed_rmsnorm_kernel<TD, TO, PER, ND>), grid, block, 0, stream, (TO*)out, resid,     \
                     (const TD*)delta, n_delta, delta_stride, post_gain, post_eps, gain, gain_stride, row_idx,  \
                     dim, eps, write_resid, delta_scale, delta_bias)
#define PICK(TD, TO, ND)              \
  do {                                \
    if (per <= 4) GO(TD, TO, 4, ND);      \
    else if (per <= 8) GO(TD, TO, 8, ND); \
    else GO(TD, TO, 16, ND);          \
  } while (0)
#define PARTS(TO)                                              \
  do {                                                         \
    if (n_delta == 1 || delta == nullptr) PICK(float, TO, 1);  \
    else if (n_delta == 2) PICK(float, TO, 2);                 \
    else if (n_delta == 4 && per <= 8) PICK(float, TO, 4);     \
    else if (n_delta == 8 && per <= 8) PICK(float, TO, 8);     \
    else PICK(float, TO, 0);                                   \
  } while (0)
  if (delta_dtype == PYLON_F32 && out_dtype == PYLON_F32) PARTS(float);
  else if (delta_dtype == PYLON_F32) PARTS(bf16_t);
  else if (out_dtype == PYLON_F32) PICK(bf16_t, float, 0);
  else PICK(bf16_t, bf16_t, 0);
#undef PARTS
#undef PICK
#undef GO
  PYLON_LAUNCHED("add_normed_rmsnorm");
}

// ---- a residual stream that is a learned mix of all earlier layers' results -----------------------
//
//   X = resid + scale * (d + bias)                  (d = sum_p delta[p]; scale and bias optional)
//   streams[index] = X                              (the layer's result, kept for the layers after it)
//   resid = sum_{j <= index} coeff[j] * streams[j]  (what the next layer, or the output, reads)
//   out = gain * resid / rms(resid)                 (optional: the norm that follows)
//
// streams[0] holds the embedded tokens, streams[j] the result of layer j - 1.  All float; one
// workgroup a row, the row in registers; the streams' loads are all sent for before the first
// multiplication, and added in the order of j.
template <typename TD, typename TO, int PER>
__global__ void depth_mix_kernel(TO* __restrict__ out, float* resid, const TD* __restrict__ delta, int n_delta,
                                 long long delta_stride, const float* __restrict__ delta_scale,
                                 const float* __restrict__ delta_bias, float* streams, long long stream_stride,
                                 int index, const float* __restrict__ coeff, const float* __restrict__ gain, int dim,
                                 float eps) {
  __shared__ float scratch[16];
  const size_t row = blockIdx.x;
  float* xr = resid + row * dim;
  const TD* dr = delta ? delta + row * dim : nullptr;
  float* sr = streams + row * dim;
  float x[PER];
#pragma unroll
  for (int n = 0; n < PER; ++n) {
    const int i = threadIdx.x + n * blockDim.x;
    x[n] = 0.f;
    if (i < dim) {
      float v = xr[i];
      if (dr) {
        float d = to_float(dr[i]);
        for (int p = 1; p < n_delta; ++p) d += to_float(dr[i + p * delta_stride]);
        if (delta_bias) d += delta_bias[i];
        v = delta_scale ? fmaf(delta_scale[i], d, v) : v + d;
      }
      sr[static_cast<size_t>(index) * stream_stride + i] = v;
      float acc = 0.f;
#pragma unroll 4
      for (int j = 0; j < index; ++j) acc = fmaf(coeff[j], sr[static_cast<size_t>(j) * stream_stride + i], acc);
      x[n] = fmaf(coeff[index], v, acc);
      xr[i] = x[n];
    }
  }
  if (out == nullptr) return;
  float ss = 0.f;
#pragma unroll
  for (int n = 0; n < PER; ++n) ss += x[n] * x[n];
  const float total = block_sum(ss, scratch);
  const float inv = 1.0f / sqrtf(total / static_cast<float>(dim) + eps);
#pragma unroll
  for (int n = 0; n < PER; ++n) {
    const int i = threadIdx.x + n * blockDim.x;
    if (i < dim) out[row * dim + i] = from_float<TO>((x[n] * inv) * gain[i]);
  }
}

// resid: float [rows, dim], replaced by the mix.  delta: null, [rows, dim], or n_delta such tensors
// delta_stride elements apart; delta_scale, delta_bias: null or dim floats.  streams: float
// [>= index + 1, stream_stride / dim >= rows, dim]; coeff: index + 1 floats.  out: null, or [rows, dim]
// of out_dtype with gain: dim floats.
extern "C" int pylon_depth_mix(void* out, int out_dtype, float* resid, const void* delta, int delta_dtype, int n_delta,
                               long long delta_stride, const float* delta_scale, const float* delta_bias,
                               float* streams, long long stream_stride, int index, const float* coeff,
                               const float* gain, int rows, int dim, float eps, hipStream_t stream) {
  PYLON_REQUIRE(pylon_valid_dtype(out_dtype) && pylon_valid_dtype(delta_dtype), "depth_mix: unknown dtype");
  PYLON_REQUIRE(rows >= 0 && dim > 0 && dim <= 16384, "depth_mix: rows of 1 to 16384 elements, got %d", dim);
  PYLON_REQUIRE(n_delta >= 1 && index >= 0 && streams != nullptr && coeff != nullptr, "depth_mix: bad arguments");
  PYLON_REQUIRE(stream_stride >= static_cast<long long>(rows) * dim, "depth_mix: the streams overlap");
  PYLON_REQUIRE(out == nullptr || gain != nullptr, "depth_mix: a norm needs its weight");
  PYLON_REQUIRE((delta_scale == nullptr && delta_bias == nullptr) || delta != nullptr,
                "depth_mix: a scale or a bias needs the output they belong to");
  if (rows == 0) return 0;
  const int threads = dim <= 256 ? 64 : (dim <= 2048 ? 256 : (dim <= 8192 ? 512 : 1024));
  const int per = (dim + threads - 1) / threads;
  dim3 grid(rows), block(threads);
#define GO(TD, TO, PER)                                                                                          \
  hipLaunchKernelGGL((depth_mix_kernel<TD, TO, PER>), grid, block, 0, stream, (TO*)out, resid, (const TD*)delta, \
                     n_delta, delta_stride, delta_scale, delta_bias, streams, stream_stride, index, coeff, gain, \
                     dim, eps)
#define PICK(TD, TO)                  \
  do {                                \
    if (per <= 4) GO(TD, TO, 4);      \
    else if (per <= 8) GO(TD, TO, 8); \
    else GO(TD, TO, 16);              \
  } while (0)
  if (delta_dtype == PYLON_F32 && out_dtype == PYLON_F32) PICK(float, float);
  else if (delta_dtype == PYLON_F32) PICK(float, bf16_t);
  else if (out_dtype == PYLON_F32) PICK(bf16_t, float);
  else PICK(bf16_t, bf16_t);
#undef PICK
#undef GO
  PYLON_LAUNCHED("depth_mix");
}
