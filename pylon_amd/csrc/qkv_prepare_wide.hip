// q/k/v preparation for attention whose norm runs over a whole projection: one norm over all
// heads of q at once and one over all heads of k (each divided by the root mean square of the
// whole row and multiplied by a weight of the row's size; either may be absent), then a rotation
// of the first rot_dim elements of every head of q and k by position * inv_freq[i], pairing
// either neighbours (2i, 2i + 1) or halves (i, i + rot_dim/2); q goes to q_out, k and v into the
// token's cache slot.  Values may have another size than keys.  One workgroup per token; sums,
// angles and rotation in float, one rounding at the end.
// With per_head the norms run head by head instead (weights of head_dim elements shared by the
// heads).  rot_scale multiplies every cosine and sine (a rotation that also stretches, as
// frequency-scaled encodings for long contexts ask).  The values are read v_offset elements into
// the row: behind the keys, or at the keys themselves as projected (values that are the keys
// before norm and rotation).
#include "common.h"

#define QW_THREADS 256

template <typename T>
__global__ void __launch_bounds__(QW_THREADS)
qkv_prepare_wide_kernel(T* __restrict__ q_out, T* __restrict__ k_cache, T* __restrict__ v_cache,
                        const T* __restrict__ qkv, long long row_stride, const float* __restrict__ q_weight,
                        const float* __restrict__ k_weight, float eps, const float* __restrict__ inv_freq,
                        int rot_dim, int interleaved, const int* __restrict__ positions,
                        const int* __restrict__ slot_map, int n_heads, int n_kv_heads, int head_dim, int v_dim,
                        int store, int per_head, float rot_scale, int v_offset, int v_page) {
  extern __shared__ float turn[];  // cos then sin of the token's rot_dim/2 angles, then per head 1/rms
  float* head_inv = turn + (rot_dim > 0 ? rot_dim : 1);
  __shared__ float scratch[16];
  const int t = blockIdx.x, tid = threadIdx.x;
  const T* row = qkv + static_cast<size_t>(t) * row_stride;
  const int q_size = n_heads * head_dim, k_size = n_kv_heads * head_dim, v_size = n_kv_heads * v_dim;
  const int half = rot_dim / 2;
  if (rot_dim > 0) {
    const float pos = static_cast<float>(positions[t]);
    for (int i = tid; i < half; i += QW_THREADS) {
      float s, c;
      sincosf(pos * inv_freq[i], &s, &c);
      turn[i] = c * rot_scale;
      turn[half + i] = s * rot_scale;
    }
  }
  float inv_q = 1.f, inv_k = 1.f;
  if (per_head) {
    // a wave a head at a time: heads of q first, then those of k
    const int lane = tid & (PYLON_WAVE - 1), wave = tid / PYLON_WAVE;
    const int heads = n_heads + (store ? n_kv_heads : 0);
    for (int hh = wave; hh < heads; hh += QW_THREADS / PYLON_WAVE) {
      const bool has = hh < n_heads ? q_weight != nullptr : k_weight != nullptr;
      float sq = 0.f;
      if (has)
        for (int d = lane; d < head_dim; d += PYLON_WAVE) {
          const float v = to_float(row[static_cast<size_t>(hh) * head_dim + d]);
          sq = fmaf(v, v, sq);
        }
      sq = wave_sum(sq);
      if (lane == 0) head_inv[hh] = has ? 1.0f / sqrtf(sq / static_cast<float>(head_dim) + eps) : 1.f;
    }
  } else if (q_weight != nullptr) {
    float sq = 0.f;
    for (int e = tid; e < q_size; e += QW_THREADS) {
      const float v = to_float(row[e]);
      sq = fmaf(v, v, sq);
    }
    inv_q = 1.0f / sqrtf(block_sum(sq, scratch) / static_cast<float>(q_size) + eps);
  }
  if (!per_head && store && k_weight != nullptr) {
    float sq = 0.f;
    for (int e = tid; e < k_size; e += QW_THREADS) {
      const float v = to_float(row[q_size + e]);
      sq = fmaf(v, v, sq);
    }
    inv_k = 1.0f / sqrtf(block_sum(sq, scratch) / static_cast<float>(k_size) + eps);
  }
  __syncthreads();  // the angles are in LDS

  // one projection (q: part 0, k: part 1): norm, rotation, store
  for (int part = 0; part < (store ? 2 : 1); ++part) {
    const int size = part == 0 ? q_size : k_size;
    const T* src = row + (part == 0 ? 0 : q_size);
    const float* weight = part == 0 ? q_weight : k_weight;
    const float inv_all = part == 0 ? inv_q : inv_k;
    const float* inv_of = head_inv + (part == 0 ? 0 : n_heads);
    T* dst = part == 0 ? q_out + static_cast<size_t>(t) * q_size
                       : k_cache + static_cast<size_t>(slot_map[t]) * k_size;
    for (int e = tid; e < size; e += QW_THREADS) {
      const int d = e % head_dim;
      const float inv = per_head ? inv_of[e / head_dim] : inv_all;
      const int wd = per_head ? head_dim : size;  // the weight's length: a head's or the projection's
      float x = to_float(src[e]) * inv * (weight != nullptr ? weight[e % wd] : 1.f);
      if (d < rot_dim) {
        int i, other;
        bool first;
        if (interleaved) {
          i = d >> 1;
          first = (d & 1) == 0;
          other = e - d + (d ^ 1);
        } else {
          first = d < half;
          i = first ? d : d - half;
          other = first ? e + half : e - half;
        }
        const float y = to_float(src[other]) * inv * (weight != nullptr ? weight[other % wd] : 1.f);
        const float c = turn[i], s = turn[half + i];
        // the pair (u, v) becomes (u cos - v sin, v cos + u sin)
        x = first ? x * c - y * s : x * c + y * s;
      }
      dst[e] = from_float<T>(x);
    }
  }
  if (store) {
    const T* src = row + v_offset;
    if (v_page > 0) {
      // values transposed inside their page: [page, kv head, element, slot in page]
      const int slot = slot_map[t];
      T* dst = v_cache + static_cast<size_t>(slot / v_page) * v_size * v_page + slot % v_page;
      for (int e = tid; e < v_size; e += QW_THREADS) dst[static_cast<size_t>(e) * v_page] = src[e];
    } else {
      T* dst = v_cache + static_cast<size_t>(slot_map[t]) * v_size;
      for (int e = tid; e < v_size; e += QW_THREADS) dst[e] = src[e];
    }
  }
}

// qkv: [tokens, n_heads*head_dim (+ n_kv_heads*head_dim + n_kv_heads*v_dim with store)], rows
// row_stride elements apart.  q_out: [tokens, n_heads, head_dim].  k_cache: [slots, n_kv_heads,
// head_dim], v_cache: [slots, n_kv_heads, v_dim], slot_map[t] the token's slot.  q_weight
// [n_heads*head_dim] and k_weight [n_kv_heads*head_dim] float, or null for no norm.  inv_freq:
// rot_dim/2 floats (rot_dim 0: no rotation); interleaved 1 pairs neighbours, 0 halves.
// per_head 1: q_weight and k_weight hold head_dim floats and every head is normed by itself.
// v_offset: where in a row the values start (with store).  v_page > 0: the values' cache is
// [pages, n_kv_heads, v_dim, v_page] (transposed inside pages of v_page slots).
extern "C" int pylon_qkv_prepare_wide(void* q_out, void* k_cache, void* v_cache, const void* qkv, int dtype,
                                      long long row_stride, const float* q_weight, const float* k_weight, float eps,
                                      const float* inv_freq, int rot_dim, int interleaved, const int* positions,
                                      const int* slot_map, int tokens, int n_heads, int n_kv_heads, int head_dim,
                                      int v_dim, int store, int per_head, float rot_scale, int v_offset, int v_page,
                                      hipStream_t stream) {
  PYLON_REQUIRE(pylon_valid_dtype(dtype), "qkv_prepare_wide: unknown dtype");
  PYLON_REQUIRE(tokens >= 0 && n_heads > 0 && n_kv_heads > 0 && head_dim > 0 && v_dim > 0,
                "qkv_prepare_wide: sizes must be positive");
  PYLON_REQUIRE(rot_dim >= 0 && rot_dim % 2 == 0 && rot_dim <= head_dim,
                "qkv_prepare_wide: rot_dim %d must be even and at most the head size %d", rot_dim, head_dim);
  PYLON_REQUIRE(rot_dim == 0 || (inv_freq != nullptr && positions != nullptr),
                "qkv_prepare_wide: a rotation needs frequencies and positions");
  PYLON_REQUIRE(!store || (k_cache != nullptr && v_cache != nullptr && slot_map != nullptr),
                "qkv_prepare_wide: storing needs the caches and the slot map");
  long long width = static_cast<long long>(n_heads) * head_dim + (store ? static_cast<long long>(n_kv_heads) * head_dim : 0);
  if (store) {
    PYLON_REQUIRE(v_offset >= 0, "qkv_prepare_wide: the values cannot start before the row");
    const long long v_end = static_cast<long long>(v_offset) + static_cast<long long>(n_kv_heads) * v_dim;
    if (v_end > width) width = v_end;
  }
  PYLON_REQUIRE(row_stride >= width, "qkv_prepare_wide: rows of %lld elements lie %lld apart", width, row_stride);
  PYLON_REQUIRE(rot_dim * sizeof(float) <= 48 * 1024, "qkv_prepare_wide: rot_dim %d is too large", rot_dim);
  if (tokens == 0) return 0;
  const size_t lds = sizeof(float) * ((rot_dim > 0 ? rot_dim : 1) + n_heads + n_kv_heads);
  PYLON_REQUIRE(lds <= 60 * 1024, "qkv_prepare_wide: too many heads");
  if (dtype == PYLON_F32)
    hipLaunchKernelGGL((qkv_prepare_wide_kernel<float>), dim3(tokens), dim3(QW_THREADS), lds, stream, (float*)q_out,
                       (float*)k_cache, (float*)v_cache, (const float*)qkv, row_stride, q_weight, k_weight, eps,
                       inv_freq, rot_dim, interleaved, positions, slot_map, n_heads, n_kv_heads, head_dim, v_dim,
                       store, per_head, rot_scale, v_offset, v_page);
  else
    hipLaunchKernelGGL((qkv_prepare_wide_kernel<bf16_t>), dim3(tokens), dim3(QW_THREADS), lds, stream,
                       (bf16_t*)q_out, (bf16_t*)k_cache, (bf16_t*)v_cache, (const bf16_t*)qkv, row_stride, q_weight,
                       k_weight, eps, inv_freq, rot_dim, interleaved, positions, slot_map, n_heads, n_kv_heads,
                       head_dim, v_dim, store, per_head, rot_scale, v_offset, v_page);
  PYLON_LAUNCHED("qkv_prepare_wide");
}
