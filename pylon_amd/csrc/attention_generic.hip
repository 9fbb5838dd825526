// Paged causal grouped-query attention, the exact and general form: any element type,
// any head size up to 512 (multiples of 8 with 16-byte loads), any number of heads and groups,
// any page size, optional sliding window or chunks (first_visible in common.h).  One wavefront owns one (token, query head):
// it walks that token's visible keys 64 at a time (one key per lane), keeps a running
// maximum and sum in float, and accumulates the weighted values with one lane per
// output element.  The walk starts at the first visible key of the token, so the order
// of every sum depends only on the token's position and never on how the batch was cut.
// Options: values of another size than keys; q rows that lie q_stride elements apart (a slice
// of a fused projection); a learned bias by distance added to the scaled score,
// rel[bucket[min(i - j, bucket_len - 1)] * n_heads + head], or without a table of buckets a bias
// that grows with the logarithm of the distance and is taken off, rel[head] * log(1 + rel[n_heads +
// head] * (i - j)); and a sink, a key of score 0 without a value, which adds one to the softmax's
// denominator, or with sink_logit a learned score per head in its place (exp(sink_logit[head]) is
// added; it is neither scaled nor capped).  softcap > 0: the scaled score s becomes softcap *
// tanh(s / softcap) before anything is added to it.
#include "common.h"

#define ATT_WAVES 4

template <typename T>
struct Vec8;  // eight consecutive elements, loaded as wide as the type allows

template <>
struct Vec8<float> {
  static __device__ __forceinline__ float dot(const float* __restrict__ q, const float* __restrict__ k, float acc) {
    const float4 a = *reinterpret_cast<const float4*>(k);
    const float4 b = *reinterpret_cast<const float4*>(k + 4);
    acc = fmaf(q[0], a.x, acc);
    acc = fmaf(q[1], a.y, acc);
    acc = fmaf(q[2], a.z, acc);
    acc = fmaf(q[3], a.w, acc);
    acc = fmaf(q[4], b.x, acc);
    acc = fmaf(q[5], b.y, acc);
    acc = fmaf(q[6], b.z, acc);
    acc = fmaf(q[7], b.w, acc);
    return acc;
  }
};

template <>
struct Vec8<bf16_t> {
  static __device__ __forceinline__ float dot(const float* __restrict__ q, const bf16_t* __restrict__ k, float acc) {
    const uint4 raw = *reinterpret_cast<const uint4*>(k);
    const uint32_t w[4] = {raw.x, raw.y, raw.z, raw.w};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      acc = fmaf(q[2 * i], __uint_as_float(w[i] << 16), acc);
      acc = fmaf(q[2 * i + 1], __uint_as_float(w[i] & 0xffff0000u), acc);
    }
    return acc;
  }
};

template <typename T, int DIMS_PER_LANE>
__global__ void paged_attention_kernel(T* __restrict__ out, const T* __restrict__ q,
                                       const T* __restrict__ k_cache, const T* __restrict__ v_cache,
                                       const int* __restrict__ block_table, int table_width,
                                       const int* __restrict__ tok_row, const int* __restrict__ positions,
                                       long long items, int n_heads, int n_kv_heads, int head_dim,
                                       int page_size, int window, float scale, int v_dim, long long q_stride,
                                       const float* __restrict__ rel, const int* __restrict__ bucket,
                                       int bucket_len, int sink, int v_transposed, float softcap,
                                       const float* __restrict__ sink_logit) {
  extern __shared__ float lds[];
  const int lane = threadIdx.x & (PYLON_WAVE - 1);
  const int wave = threadIdx.x / PYLON_WAVE;
  float* qbuf = lds + wave * head_dim;
  const long long item = static_cast<long long>(blockIdx.x) * ATT_WAVES + wave;
  const bool active = item < items;
  int t = 0, h = 0;
  if (active) {
    t = static_cast<int>(item / n_heads);
    h = static_cast<int>(item - static_cast<long long>(t) * n_heads);
    const T* qr = q + static_cast<size_t>(t) * q_stride + static_cast<size_t>(h) * head_dim;
    for (int i = lane; i < head_dim; i += PYLON_WAVE) qbuf[i] = to_float(qr[i]);
  }
  __syncthreads();
  if (!active) return;

  const int kvh = h / (n_heads / n_kv_heads);
  const int pos = positions[t];
  const int* table = block_table + static_cast<size_t>(tok_row[t]) * table_width;
  const int first = first_visible(pos, window);

  float m = -INFINITY, l = 0.f;
  float acc[DIMS_PER_LANE];
#pragma unroll
  for (int i = 0; i < DIMS_PER_LANE; ++i) acc[i] = 0.f;

  for (int base = first; base <= pos; base += PYLON_WAVE) {
    const int j = base + lane;
    const bool valid = j <= pos;
    int phys = 0;
    float s = -INFINITY;
    if (valid) {
      phys = table[j / page_size] * page_size + (j % page_size);
      const T* kr = k_cache + (static_cast<size_t>(phys) * n_kv_heads + kvh) * head_dim;
      float dot = 0.f;
      if (head_dim & 7) {  // a head that is no whole number of 16-byte pieces: element by element
        for (int d = 0; d < head_dim; ++d) dot = fmaf(qbuf[d], to_float(kr[d]), dot);
      } else {
        for (int d = 0; d < head_dim; d += 8) dot = Vec8<T>::dot(qbuf + d, kr + d, dot);
      }
      s = dot * scale;
      if (softcap > 0.f) s = softcap * tanhf(s / softcap);
      if (rel != nullptr) {
        const int far = pos - j;
        if (bucket != nullptr)
          s += rel[static_cast<size_t>(bucket[far < bucket_len ? far : bucket_len - 1]) * n_heads + h];
        else
          s -= rel[h] * logf(1.0f + rel[n_heads + h] * static_cast<float>(far));
      }
    }
    const float m_new = fmaxf(m, wave_max(s));
    const float p = valid ? expf(s - m_new) : 0.f;
    const float corr = expf(m - m_new);
    l = l * corr + wave_sum(p);
#pragma unroll
    for (int i = 0; i < DIMS_PER_LANE; ++i) acc[i] *= corr;
    const int count = (pos - base + 1 < PYLON_WAVE) ? pos - base + 1 : PYLON_WAVE;
    for (int kk = 0; kk < count; ++kk) {
      const float pk = __shfl(p, kk, PYLON_WAVE);
      const int physk = __shfl(phys, kk, PYLON_WAVE);
      // values transposed inside their page: [page, kv head, element, slot in page]
      const T* vr = v_transposed
                        ? v_cache + (static_cast<size_t>(physk / page_size) * n_kv_heads + kvh) * v_dim * page_size +
                              physk % page_size
                        : v_cache + (static_cast<size_t>(physk) * n_kv_heads + kvh) * v_dim;
      const size_t vstep = v_transposed ? page_size : 1;
#pragma unroll
      for (int i = 0; i < DIMS_PER_LANE; ++i) {
        const int d = lane + PYLON_WAVE * i;
        if (d < v_dim) acc[i] = fmaf(pk, to_float(vr[d * vstep]), acc[i]);
      }
    }
    m = m_new;
  }
  T* orow = out + (static_cast<size_t>(t) * n_heads + h) * v_dim;
  if (sink_logit != nullptr) {
    // the sink joins as one more score: the larger of it and the maximum so far is the new scale
    const float z = sink_logit[h];
    const float m_fin = fmaxf(m, z);
    const float corr = expf(m - m_fin);
    l = l * corr + expf(z - m_fin);
#pragma unroll
    for (int i = 0; i < DIMS_PER_LANE; ++i) acc[i] *= corr;
  } else if (sink) {
    l += expf(-m);  // the sink's weight on the scale of the running maximum
  }
  const float inv = 1.0f / l;
#pragma unroll
  for (int i = 0; i < DIMS_PER_LANE; ++i) {
    const int d = lane + PYLON_WAVE * i;
    if (d < v_dim) orow[d] = from_float<T>(acc[i] * inv);
  }
}

template <typename T>
static int launch_paged_attention(T* out, const T* q, const T* k_cache, const T* v_cache,
                                  const int* block_table, int table_width, const int* tok_row,
                                  const int* positions, int tokens, int n_heads, int n_kv_heads,
                                  int head_dim, int page_size, int window, float scale, int v_dim,
                                  long long q_stride, const float* rel, const int* bucket, int bucket_len,
                                  int sink, int v_transposed, float softcap, const float* sink_logit,
                                  hipStream_t stream) {
  const long long items = static_cast<long long>(tokens) * n_heads;
  const long long blocks = (items + ATT_WAVES - 1) / ATT_WAVES;
  dim3 grid((unsigned)blocks), block(ATT_WAVES * PYLON_WAVE);
  const size_t lds = sizeof(float) * ATT_WAVES * head_dim;
#define LAUNCH(DPL)                                                                                  \
  hipLaunchKernelGGL((paged_attention_kernel<T, DPL>), grid, block, lds, stream, out, q, k_cache,    \
                     v_cache, block_table, table_width, tok_row, positions, items, n_heads,          \
                     n_kv_heads, head_dim, page_size, window, scale, v_dim, q_stride, rel, bucket,   \
                     bucket_len, sink, v_transposed, softcap, sink_logit)
  if (v_dim <= 64)
    LAUNCH(1);
  else if (v_dim <= 128)
    LAUNCH(2);
  else if (v_dim <= 256)
    LAUNCH(4);
  else
    LAUNCH(8);
#undef LAUNCH
  return 0;
}

// q: [tokens, n_heads, head_dim], rows q_stride elements apart; out: [tokens, n_heads, v_dim].
// Caches: keys [pages*page_size, n_kv_heads, head_dim], values [pages*page_size, n_kv_heads, v_dim].
// With v_transposed the values lie as [pages, n_kv_heads, v_dim, page_size].
// rel: null, or float [rows, n_heads] with bucket: int [bucket_len], every entry a row of rel; or,
// with bucket null, float [2, n_heads]: per head the factor and the slope of a logarithmic bias.
// block_table: [rows, table_width] page ids; tok_row[t] names the table row of token t;
// positions[t] is the token's index in its request; keys first(t)..positions[t] are read,
// first(t) = max(0, positions[t] - window + 1) when window > 0; the start of the token's chunk of
// -window positions when window < 0; else 0.
extern "C" int pylon_paged_attention(void* out, const void* q, const void* k_cache, const void* v_cache,
                                     int dtype, const int* block_table, int table_width,
                                     const int* tok_row, const int* positions, int tokens, int n_heads,
                                     int n_kv_heads, int head_dim, int page_size, int window,
                                     float scale, int v_dim, long long q_stride, const float* rel,
                                     const int* bucket, int bucket_len, int sink, int v_transposed,
                                     float softcap, const float* sink_logit, hipStream_t stream) {
  PYLON_REQUIRE(pylon_valid_dtype(dtype), "paged_attention: unknown dtype");
  PYLON_REQUIRE(tokens >= 0 && n_heads > 0 && n_kv_heads > 0 && n_heads % n_kv_heads == 0,
                "paged_attention: %d query heads cannot be grouped over %d key/value heads", n_heads,
                n_kv_heads);
  PYLON_REQUIRE(head_dim >= 1 && head_dim <= 512, "paged_attention: head_dim %d must be between 1 and 512", head_dim);
  PYLON_REQUIRE(page_size > 0 && table_width > 0, "paged_attention: bad page size or table width");
  PYLON_REQUIRE(v_dim >= 1 && v_dim <= 512, "paged_attention: values of 1 to 512 elements, got %d", v_dim);
  PYLON_REQUIRE(q_stride >= static_cast<long long>(n_heads) * head_dim, "paged_attention: q rows overlap");
  PYLON_REQUIRE(rel == nullptr || bucket == nullptr || bucket_len >= 1,
                "paged_attention: a table of buckets holds at least one entry");
  if (tokens == 0) return 0;
  PYLON_REQUIRE(static_cast<long long>(tokens) * n_heads / ATT_WAVES < (1ll << 31),
                "paged_attention: too many (token, head) pairs for one launch");
  if (dtype == PYLON_F32)
    launch_paged_attention<float>((float*)out, (const float*)q, (const float*)k_cache,
                                  (const float*)v_cache, block_table, table_width, tok_row, positions,
                                  tokens, n_heads, n_kv_heads, head_dim, page_size, window, scale, v_dim,
                                  q_stride, rel, bucket, bucket_len, sink, v_transposed, softcap, sink_logit,
                                  stream);
  else
    launch_paged_attention<bf16_t>((bf16_t*)out, (const bf16_t*)q, (const bf16_t*)k_cache,
                                   (const bf16_t*)v_cache, block_table, table_width, tok_row, positions,
                                   tokens, n_heads, n_kv_heads, head_dim, page_size, window, scale, v_dim,
                                   q_stride, rel, bucket, bucket_len, sink, v_transposed, softcap, sink_logit,
                                  stream);
  PYLON_LAUNCHED("paged_attention");
}
