// Keys and values of a step's tokens, copied from the rows of a fused projection into their
// cache slots.  Keys and values may differ in size per head; nothing is normed or rotated.
// Values can be stored transposed inside their page, [page, element of all heads, slot in page]
// (page_size > 0), for attention kernels that feed runs of neighbouring keys to a matrix unit.
#include "common.h"

template <typename T>
__global__ void kv_store_kernel(T* __restrict__ k_cache, T* __restrict__ v_cache, const T* __restrict__ proj,
                                long long ld, int k_off, int v_off, const int* __restrict__ slot_map, int k_row,
                                int v_row, int page_size) {
  const int t = blockIdx.x;
  const size_t slot = static_cast<size_t>(slot_map[t]);
  const T* pr = proj + static_cast<size_t>(t) * ld;
  T* kd = k_cache + slot * k_row;
  T* vd = v_cache + slot * v_row;
  for (int i = threadIdx.x; i < k_row; i += blockDim.x) kd[i] = pr[k_off + i];
  if (page_size > 0) {
    T* page = v_cache + (slot / page_size) * page_size * v_row + slot % page_size;
    for (int i = threadIdx.x; i < v_row; i += blockDim.x) page[static_cast<size_t>(i) * page_size] = pr[v_off + i];
  } else {
    for (int i = threadIdx.x; i < v_row; i += blockDim.x) vd[i] = pr[v_off + i];
  }
}

// proj: [tokens, ld]; k_cache: [slots, k_row]; v_cache: [slots, v_row], all of dtype; k_row and
// v_row are the elements of all key/value heads of one token; page_size > 0: v_cache is
// [pages, v_row, page_size] instead.  The host guarantees that every
// slot_map[t] is a slot of the caches.
extern "C" int pylon_kv_store(void* k_cache, void* v_cache, const void* proj, int dtype, long long ld, int k_off,
                              int v_off, const int* slot_map, int tokens, int k_row, int v_row, int page_size,
                              hipStream_t stream) {
  PYLON_REQUIRE(pylon_valid_dtype(dtype), "kv_store: unknown dtype");
  PYLON_REQUIRE(tokens >= 0 && k_row > 0 && v_row > 0 && k_off >= 0 && v_off >= 0, "kv_store: bad sizes");
  PYLON_REQUIRE(ld >= k_off + k_row && ld >= v_off + v_row, "kv_store: the projection's rows are too short");
  if (tokens == 0) return 0;
  dim3 grid(tokens), block(256);
  if (dtype == PYLON_F32)
    hipLaunchKernelGGL(kv_store_kernel<float>, grid, block, 0, stream, (float*)k_cache, (float*)v_cache,
                       (const float*)proj, ld, k_off, v_off, slot_map, k_row, v_row, page_size);
  else
    hipLaunchKernelGGL(kv_store_kernel<bf16_t>, grid, block, 0, stream, (bf16_t*)k_cache, (bf16_t*)v_cache,
                       (const bf16_t*)proj, ld, k_off, v_off, slot_map, k_row, v_row, page_size);
  PYLON_LAUNCHED("kv_store");
}

// The same with the projection's bias, and the queries too: q, k and v of a fused projection
// (its float sums, or rounded already) get their bias, are rounded once to the caches' type, and go
// where the attention kernels read them: q to a tensor of its own, k and v to the tokens' cache slots.
template <typename TI, typename TO>
__global__ void qkv_bias_store_kernel(TO* __restrict__ q_out, TO* __restrict__ k_cache, TO* __restrict__ v_cache,
                                      const TI* __restrict__ proj, long long ld, const float* __restrict__ bias,
                                      const int* __restrict__ slot_map, int q_row, int k_row, int v_row,
                                      int page_size, int store) {
  const int t = blockIdx.x;
  const TI* pr = proj + static_cast<size_t>(t) * ld;
  TO* qd = q_out + static_cast<size_t>(t) * q_row;
  for (int i = threadIdx.x; i < q_row; i += blockDim.x)
    qd[i] = from_float<TO>(to_float(pr[i]) + (bias ? bias[i] : 0.f));
  if (!store) return;
  const size_t slot = static_cast<size_t>(slot_map[t]);
  TO* kd = k_cache + slot * k_row;
  for (int i = threadIdx.x; i < k_row; i += blockDim.x)
    kd[i] = from_float<TO>(to_float(pr[q_row + i]) + (bias ? bias[q_row + i] : 0.f));
  const int v_off = q_row + k_row;
  if (page_size > 0) {
    TO* page = v_cache + (slot / page_size) * page_size * v_row + slot % page_size;
    for (int i = threadIdx.x; i < v_row; i += blockDim.x)
      page[static_cast<size_t>(i) * page_size] = from_float<TO>(to_float(pr[v_off + i]) + (bias ? bias[v_off + i] : 0.f));
  } else {
    TO* vd = v_cache + slot * v_row;
    for (int i = threadIdx.x; i < v_row; i += blockDim.x)
      vd[i] = from_float<TO>(to_float(pr[v_off + i]) + (bias ? bias[v_off + i] : 0.f));
  }
}

// proj: [tokens, ld] of in_dtype, a row q_row + k_row + v_row elements (q_row alone without store);
// bias: null or float of a row's length; q_out: [tokens, q_row]; caches as for kv_store, of out_dtype.
extern "C" int pylon_qkv_bias_store(void* q_out, void* k_cache, void* v_cache, int out_dtype, const void* proj,
                                    int in_dtype, long long ld, const float* bias, const int* slot_map, int tokens,
                                    int q_row, int k_row, int v_row, int page_size, int store, hipStream_t stream) {
  PYLON_REQUIRE(pylon_valid_dtype(out_dtype) && pylon_valid_dtype(in_dtype), "qkv_bias_store: unknown dtype");
  PYLON_REQUIRE(tokens >= 0 && q_row > 0 && k_row > 0 && v_row > 0, "qkv_bias_store: bad sizes");
  PYLON_REQUIRE(ld >= q_row + (store ? k_row + v_row : 0), "qkv_bias_store: the projection's rows are too short");
  PYLON_REQUIRE(!store || (slot_map != nullptr && k_cache != nullptr && v_cache != nullptr),
                "qkv_bias_store: storing needs the caches and the tokens' slots");
  PYLON_REQUIRE(!(in_dtype == PYLON_BF16 && out_dtype == PYLON_F32), "qkv_bias_store: a float cache takes float sums");
  if (tokens == 0) return 0;
  dim3 grid(tokens), block(256);
#define GO(TI, TO)                                                                                               \
  hipLaunchKernelGGL((qkv_bias_store_kernel<TI, TO>), grid, block, 0, stream, (TO*)q_out, (TO*)k_cache,          \
                     (TO*)v_cache, (const TI*)proj, ld, bias, slot_map, q_row, k_row, v_row, page_size, store)
  if (in_dtype == PYLON_F32 && out_dtype == PYLON_F32) GO(float, float);
  else if (in_dtype == PYLON_F32) GO(float, bf16_t);
  else GO(bf16_t, bf16_t);
#undef GO
  PYLON_LAUNCHED("qkv_bias_store");
}
