// Paged causal attention with a learned bias by distance and a sink, on the matrix cores, for
// bfloat16 prompt portions and single tokens alike:
//
//   s_ij = scale * q_i.k_j + bias[head, min(i - j, bucket_len - 1)],   j <= i
//   out_i = sum_j exp(s_ij) v_j / (1 + sum_j exp(s_ij))
//
// (the learned table's rows already looked up by distance).  Keys have `dim` elements, values `vdim`.  Keys lie in the cache as [slot, kv head, dim];
// values lie transposed inside every page, [page, kv head, vdim, slot in page], so that the
// eight keys a lane feeds to a matrix instruction are neighbours in memory.
//
// A workgroup owns up to 32 consecutive tokens of one request and the (up to four) query heads of
// one key/value head; each of its eight wavefronts one head and 16 of the tokens (one tile of query columns).  It walks the keys in blocks of 32 (which never cross a page: pages are
// multiples of 32).  Scores are computed transposed, S^T = K Q^T (16x16x32 instructions: rows are
// keys, columns are queries), so that everything that belongs to a query (its running maximum,
// its sum, its output) lives in the lanes of that query's column, and the exponentials are
// already laid out as the operand of O^T = V^T P^T.  Scores, bias, maximum, exponentials and
// sums are float; the weights enter the value product as two bfloat16 terms, p = hi + lo, so
// that they carry sixteen bits of mantissa.  The sink is where the walk starts: maximum 0,
// sum 1, output 0.  The waves of a workgroup take heads of one key/value head at the same
// tokens: a block's keys and values are fetched once, with 16-byte loads of whole rows, into LDS
// (two buffers in turns: one barrier a block) and read from there by every wave as operands
// (rows padded against bank conflicts).  Keys
// may be cut over `cuts` workgroups, which then leave float partial results (maximum, sum,
// unnormalised output) for a second small kernel to merge in order; the sink belongs to the
// first cut.  The order of a query's sums depends on its position and the number of cuts only.
#include "common.h"

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float floatx4 __attribute__((ext_vector_type(4)));
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
typedef unsigned int u32x2 __attribute__((ext_vector_type(2)));

#define AS_BLOCK 32   // keys per step of the walk
#define AS_QT 1       // query tiles of 16 per wave
#define AS_MAX_BIAS 4096

__device__ __forceinline__ uint32_t as_pack(float a, float b) {
  return static_cast<uint32_t>(float_to_bf16_bits(a)) | (static_cast<uint32_t>(float_to_bf16_bits(b)) << 16);
}

// KS: steps of 32 key elements (dim <= 32 KS); NV: tiles of 16 value elements (vdim <= 16 NV).
// scale * s, or with a cap c > 0: c * tanh(scale * s / c), the tangent as 1 - 2 / (e^(2x) + 1)
// (it ends at 1 and -1 where the exponential overflows or vanishes).
__device__ __forceinline__ float capped_score(float s, float scale, float cap) {
  const float v = s * scale;
  if (!(cap > 0.f)) return v;
  const float e = __expf(2.0f * v / cap);
  return cap * (1.0f - 2.0f / (e + 1.0f));
}

template <int KS, int NV>
__global__ __launch_bounds__(512) void attention_sink_kernel(
    bf16_t* __restrict__ out, const bf16_t* __restrict__ q, long long q_stride, const bf16_t* __restrict__ k_cache,
    const bf16_t* __restrict__ v_cache, const int* __restrict__ block_table, int table_width,
    const int* __restrict__ tiles, const int* __restrict__ positions, int n_heads, int n_kv_heads, int dim, int vdim, int page_size, float scale,
    const float* __restrict__ bias, int bucket_len, int sink, int cuts, float* __restrict__ partial, int window,
    float softcap, const float* __restrict__ sink_logit) {
  // eight waves: wave & 3 names the head of the group, wave >> 2 which 16 of the tile's 32 tokens, so
  // that every SIMD holds two waves that fill each other's waits
  constexpr int waves_per_group = 4;
  constexpr int KL = (KS + 3) / 4, VL = (NV + 7) / 8;  // 16-byte pieces of a block a thread fetches
  extern __shared__ float bias_lds[];  // [heads of the workgroup][bucket_len], then the block's keys and values
  const int lane = threadIdx.x & 63, wave = (threadIdx.x >> 6) & 3, qsel = threadIdx.x >> 8;
  const int col = lane & 15, grp = lane >> 4;
  const int group = n_heads / n_kv_heads;
  const int chunks = (group + waves_per_group - 1) / waves_per_group;
  int b = blockIdx.x;
  const int cut = b % cuts;
  b /= cuts;
  const int chunk = b % chunks;
  b /= chunks;
  const int kvh = b % n_kv_heads;
  const int tile = b / n_kv_heads;
  const int in_group = chunk * waves_per_group + wave;
  const bool idle = in_group >= group;  // a wave beyond the group's heads helps to fetch and stores nothing
  const int head = kvh * group + (idle ? group - 1 : in_group);
  // without a table of tiles every token is a tile of its own and row t of the block table is token t's
  const int tok0 = tiles ? tiles[4 * tile] : tile, count = tiles ? tiles[4 * tile + 1] : 1;
  const int row = tiles ? tiles[4 * tile + 2] : tile, pos0 = tiles ? tiles[4 * tile + 3] : positions[tile];
  const int kv_last = pos0 + count - 1;
  const int n_qt = (qsel == 0 || count > 16) ? 1 : 0;  // a tile of up to 16 tokens leaves the second half's waves idle
  const int* table = block_table + static_cast<size_t>(row) * table_width;

  const int tstride = (bucket_len + 3) & ~3;  // keeps what follows the tables 16-byte aligned
  float* tbl = bias_lds + wave * tstride;
  const int kstr = dim + 8, vstr = AS_BLOCK + 4;  // LDS rows, padded
  // two buffers of a block's keys and values, used in turns
  bf16_t* kv_lds = reinterpret_cast<bf16_t*>(bias_lds + waves_per_group * tstride);
  const int buf_elems = AS_BLOCK * kstr + ((vdim + 15) & ~15) * vstr;
  constexpr int threads = 2 * waves_per_group * 64;
  const float* bias_row = bias ? bias + static_cast<size_t>(head) * bucket_len : nullptr;
  if (bias != nullptr) {
#pragma unroll 8
    for (int d = lane; d < bucket_len; d += 64) tbl[d] = bias_row[d];
  }
  const float far_bias = bias != nullptr ? bias_row[bucket_len - 1] : 0.f;

  // Q^T operands: column = query, eight key elements per lane and step
  bf16x8 qf[AS_QT][KS];
  int qpos[AS_QT], qfirst[AS_QT];  // a query's position and the first key it sees (a window, a chunk)
#pragma unroll
  for (int qt = 0; qt < AS_QT; ++qt) {
    const int qi = (qt + qsel) * 16 + col;
    qpos[qt] = pos0 + qi;
    qfirst[qt] = first_visible(qpos[qt], window);
    const int t = tok0 + (qi < count ? qi : count - 1);
    const bf16_t* qr = q + static_cast<size_t>(t) * q_stride + static_cast<size_t>(head) * dim;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      const int d = ks * 32 + grp * 8;
      u32x4 raw = {0u, 0u, 0u, 0u};
      if (d < dim) raw = *reinterpret_cast<const u32x4*>(qr + d);
      qf[qt][ks] = __builtin_bit_cast(bf16x8, raw);
    }
  }

  floatx4 o[AS_QT][NV];
  float m_run[AS_QT], l_run[AS_QT];
#pragma unroll
  for (int qt = 0; qt < AS_QT; ++qt) {
    // the sink: a key without a value (one lane of a query's four carries its one) whose score is 0,
    // or the head's learned number
    m_run[qt] = (sink && cut == 0) ? (sink_logit != nullptr ? sink_logit[head] : 0.f) : -INFINITY;
    l_run[qt] = (sink && cut == 0 && grp == 0) ? 1.f : 0.f;
#pragma unroll
    for (int dt = 0; dt < NV; ++dt) o[qt][dt] = floatx4{0.f, 0.f, 0.f, 0.f};
  }

  // the walk starts at the block of the first key that the tile's first query sees
  const int kb_first = first_visible(pos0, window) / AS_BLOCK * AS_BLOCK;
  const int n_blocks = (kv_last - kb_first) / AS_BLOCK + 1;
  const int per_cut = (n_blocks + cuts - 1) / cuts;
  const int kb_begin = kb_first + cut * per_cut * AS_BLOCK;
  const int kb_end = kb_first + ((cut + 1) * per_cut < n_blocks ? (cut + 1) * per_cut : n_blocks) * AS_BLOCK;
  // A block's keys and values travel global -> registers -> LDS; the registers of block b + 1
  // are filled while block b is computed.
  u32x4 kreg[KL], vreg[VL];
  const int kchunks = dim >> 3;  // 16-byte pieces of a key row
  auto fetch = [&](int kb) {
    const int page = table[kb / page_size];
    const int in_page = kb % page_size;
    const bf16_t* kbase = k_cache + ((static_cast<size_t>(page) * page_size + in_page) * n_kv_heads + kvh) * dim;
#pragma unroll
    for (int n = 0; n < KL; ++n) {
      const int c = threadIdx.x + n * threads;
      if (c < AS_BLOCK * kchunks) {
        const int r = c / kchunks, e = (c - r * kchunks) * 8;
        kreg[n] = *reinterpret_cast<const u32x4*>(kbase + static_cast<size_t>(r) * n_kv_heads * dim + e);
      }
    }
    const bf16_t* vbase = v_cache + (static_cast<size_t>(page) * n_kv_heads + kvh) * vdim * page_size + in_page;
#pragma unroll
    for (int n = 0; n < VL; ++n) {
      const int c = threadIdx.x + n * threads;
      if (c < vdim * (AS_BLOCK / 8)) {
        const int r = c / (AS_BLOCK / 8), e = (c - r * (AS_BLOCK / 8)) * 8;
        vreg[n] = *reinterpret_cast<const u32x4*>(vbase + static_cast<size_t>(r) * page_size + e);
      }
    }
  };
  auto stage = [&](int turn) {
    bf16_t* k_lds = kv_lds + turn * buf_elems;
    bf16_t* v_lds = k_lds + AS_BLOCK * kstr;
#pragma unroll
    for (int n = 0; n < KL; ++n) {
      const int c = threadIdx.x + n * threads;
      if (c < AS_BLOCK * kchunks) {
        const int r = c / kchunks, e = (c - r * kchunks) * 8;
        *reinterpret_cast<u32x4*>(k_lds + r * kstr + e) = kreg[n];
      }
    }
#pragma unroll
    for (int n = 0; n < VL; ++n) {
      const int c = threadIdx.x + n * threads;
      if (c < vdim * (AS_BLOCK / 8)) {
        const int r = c / (AS_BLOCK / 8), e = (c - r * (AS_BLOCK / 8)) * 8;
        *reinterpret_cast<u32x2*>(v_lds + r * vstr + e) = u32x2{vreg[n][0], vreg[n][1]};
        *reinterpret_cast<u32x2*>(v_lds + r * vstr + e + 4) = u32x2{vreg[n][2], vreg[n][3]};
      }
    }
  };
  // Block b is computed from one buffer while block b + 1, fetched during block b - 1's math, is
  // written to the other and block b + 2 is sent for: one barrier a block.
  if (kb_begin < kb_end) {
    fetch(kb_begin);
    stage(0);
    if (kb_begin + AS_BLOCK < kb_end) fetch(kb_begin + AS_BLOCK);
  }
  __syncthreads();
  int turn = 0;
  for (int kb = kb_begin; kb < kb_end; kb += AS_BLOCK, turn ^= 1) {
    const bf16_t* k_lds = kv_lds + turn * buf_elems;
    const bf16_t* v_lds = k_lds + AS_BLOCK * kstr;
    // K operands: row = key, eight elements per lane and step
    floatx4 s[AS_QT][2];
#pragma unroll
    for (int t = 0; t < 2; ++t) {
      const bf16_t* kr = k_lds + (t * 16 + col) * kstr;
#pragma unroll
      for (int qt = 0; qt < AS_QT; ++qt) s[qt][t] = floatx4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) {
        const int d = ks * 32 + grp * 8;
        u32x4 raw = {0u, 0u, 0u, 0u};
        if (d < dim) raw = *reinterpret_cast<const u32x4*>(kr + d);
        const bf16x8 kf = __builtin_bit_cast(bf16x8, raw);
#pragma unroll
        for (int qt = 0; qt < AS_QT; ++qt)
          if (qt < n_qt) s[qt][t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf, qf[qt][ks], s[qt][t], 0, 0, 0);
      }
    }
    // V^T operands: row = value element, keys kb + 4 grp + {0..3} and kb + 16 + 4 grp + {0..3}
    bf16x8 vf[NV];
    const bool ragged = kb + AS_BLOCK - 1 > kv_last;  // slots past the request's end hold anything
#pragma unroll
    for (int dt = 0; dt < NV; ++dt) {
      const int d = dt * 16 + col;
      u32x4 raw = {0u, 0u, 0u, 0u};
      if (d < vdim) {
        const bf16_t* vr = v_lds + d * vstr + 4 * grp;
        const u32x2 first = *reinterpret_cast<const u32x2*>(vr);
        const u32x2 second = *reinterpret_cast<const u32x2*>(vr + 16);
        raw = u32x4{first[0], first[1], second[0], second[1]};
        if (ragged) {
#pragma unroll
          for (int e = 0; e < 8; ++e) {
            const int key = kb + (e >> 2) * 16 + 4 * grp + (e & 3);
            if (key > kv_last) raw[e >> 1] &= (e & 1) ? 0x0000ffffu : 0xffff0000u;
          }
        }
      }
      vf[dt] = __builtin_bit_cast(bf16x8, raw);
    }

#pragma unroll
    for (int qt = 0; qt < AS_QT; ++qt) {
      if (qt >= n_qt) continue;
      // scores of this lane: keys kb + 16 t + 4 grp + i for query qpos[qt]
      float sc[8];
      const int near = qpos[qt] - (kb + AS_BLOCK - 1);  // the smallest distance of the block for this query
      const bool all_far = bias == nullptr || near >= bucket_len - 1;
      float top = m_run[qt];
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const int key = kb + (e >> 2) * 16 + 4 * grp + (e & 3);
        const int dist = qpos[qt] - key;
        float bias = far_bias;
        if (!all_far) {
          int idx = dist < 0 ? 0 : dist;
          idx = idx < bucket_len - 1 ? idx : bucket_len - 1;
          bias = tbl[idx];
        }
        const float v = capped_score(s[qt][e >> 2][e & 3], scale, softcap) + bias;
        sc[e] = (dist >= 0 && key >= qfirst[qt]) ? v : -INFINITY;
        top = fmaxf(top, sc[e]);
      }
      top = fmaxf(top, __shfl_xor(top, 16, 64));
      top = fmaxf(top, __shfl_xor(top, 32, 64));
      // a query past the tile's end, or one whose every key so far is hidden, keeps -inf: no NaN from inf - inf
      const float m_new = top;
      const float corr = (m_new == -INFINITY) ? 1.f : __expf(m_run[qt] - m_new);
      float p[8], sum = 0.f;
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        p[e] = (sc[e] == -INFINITY) ? 0.f : __expf(sc[e] - m_new);
        sum += p[e];
      }
      l_run[qt] = l_run[qt] * corr + sum;
      m_run[qt] = m_new;
      u32x4 hi, lo;
#pragma unroll
      for (int e = 0; e < 8; e += 2) {
        // hi: the upper sixteen bits of p as they are; lo: those of the rest (p - hi is exact)
        const uint32_t a = __float_as_uint(p[e]), c = __float_as_uint(p[e + 1]);
        hi[e >> 1] = __builtin_amdgcn_perm(c, a, 0x07060302u);
        const float ra = p[e] - __uint_as_float(a & 0xffff0000u), rc = p[e + 1] - __uint_as_float(c & 0xffff0000u);
        lo[e >> 1] = __builtin_amdgcn_perm(__float_as_uint(rc), __float_as_uint(ra), 0x07060302u);
      }
      const bf16x8 p_hi = __builtin_bit_cast(bf16x8, hi), p_lo = __builtin_bit_cast(bf16x8, lo);
      const bool rescale = __any(corr != 1.f);  // no query of the wave raised its maximum: nothing to scale
#pragma unroll
      for (int dt = 0; dt < NV; ++dt) {
        floatx4 acc = o[qt][dt];
        if (rescale) {
          acc[0] *= corr; acc[1] *= corr; acc[2] *= corr; acc[3] *= corr;
        }
        acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf[dt], p_hi, acc, 0, 0, 0);
        o[qt][dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf[dt], p_lo, acc, 0, 0, 0);
      }
    }
    if (kb + AS_BLOCK < kb_end) {
      stage(turn ^ 1);  // nobody reads that buffer: the block before this one is done everywhere
      if (kb + 2 * AS_BLOCK < kb_end) fetch(kb + 2 * AS_BLOCK);
    }
    __syncthreads();
  }

#pragma unroll
  for (int qt = 0; qt < AS_QT; ++qt) {
    float l = l_run[qt];
    l += __shfl_xor(l, 16, 64);
    l += __shfl_xor(l, 32, 64);
    const int qi = (qt + qsel) * 16 + col;
    if (qi >= count || idle) continue;
    if (cuts > 1) {
      // [token, head, cut, 2 + vdim]: maximum, sum, unnormalised output
      float* dst = partial + ((static_cast<size_t>(tok0 + qi) * n_heads + head) * cuts + cut) * (2 + vdim);
      if (grp == 0) {
        dst[0] = m_run[qt];
        dst[1] = l;
      }
#pragma unroll
      for (int dt = 0; dt < NV; ++dt)
#pragma unroll
        for (int i = 0; i < 4; ++i)
          if (dt * 16 + 4 * grp + i < vdim) dst[2 + dt * 16 + 4 * grp + i] = o[qt][dt][i];
      continue;
    }
    const float inv = 1.0f / l;
    bf16_t* orow = out + (static_cast<size_t>(tok0 + qi) * n_heads + head) * vdim;
#pragma unroll
    for (int dt = 0; dt < NV; ++dt) {
      const int d = dt * 16 + 4 * grp;
      if (d + 3 < vdim) {
        u32x2 packed = {as_pack(o[qt][dt][0] * inv, o[qt][dt][1] * inv), as_pack(o[qt][dt][2] * inv, o[qt][dt][3] * inv)};
        *reinterpret_cast<u32x2*>(orow + d) = packed;
      } else {
#pragma unroll
        for (int i = 0; i < 4; ++i)
          if (d + i < vdim) orow[d + i].bits = float_to_bf16_bits(o[qt][dt][i] * inv);
      }
    }
  }
}

// A step of single tokens: one workgroup per (token, key/value head, cut of the keys).  The heads of
// the group (at most 16) sit side by side in the query columns of one tile, all at the token's
// position, so a block's scores for the whole group cost what one head's cost; the four waves take
// every fourth block of the cut and fetch their operands themselves (no wave reads what another
// fetched, so nothing is staged and nothing waits at a barrier); at the end the four waves' partial
// results (maximum, sum, unnormalised output, all float) meet in LDS and are merged in the order of
// the waves: into the output if the keys are not cut, else into the cut's partial result for the
// merge kernel.
template <int KS, int NV>
__global__ __launch_bounds__(256) void attention_sink_decode_kernel(
    bf16_t* __restrict__ out, const bf16_t* __restrict__ q, long long q_stride, const bf16_t* __restrict__ k_cache,
    const bf16_t* __restrict__ v_cache, const int* __restrict__ block_table, int table_width,
    const int* __restrict__ positions, int n_heads, int n_kv_heads, int dim, int vdim, int page_size, float scale,
    const float* __restrict__ bias, int bucket_len, int sink, int cuts, float* __restrict__ partial, int window,
    float softcap, const float* __restrict__ sink_logit) {
  extern __shared__ float bias_lds[];  // [group][bucket_len]
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int col = lane & 15, grp = lane >> 4;
  const int group = n_heads / n_kv_heads;
  int b = blockIdx.x;
  const int cut = b % cuts;
  b /= cuts;
  const int kvh = b % n_kv_heads;
  const int tok = b / n_kv_heads;
  const int pos = positions[tok];
  const int* table = block_table + static_cast<size_t>(tok) * table_width;
  const int my_head = kvh * group + (col < group ? col : group - 1);  // columns past the group repeat its last head
  if (bias != nullptr) {
    for (int i = threadIdx.x; i < group * bucket_len; i += 256) {
      const int h = i / bucket_len;
      bias_lds[i] = bias[static_cast<size_t>(kvh * group + h) * bucket_len + (i - h * bucket_len)];
    }
  }
  __syncthreads();
  const float* tbl = bias_lds + (col < group ? col : group - 1) * bucket_len;
  const float far_bias = bias != nullptr ? tbl[bucket_len - 1] : 0.f;

  bf16x8 qf[KS];
  {
    const bf16_t* qr = q + static_cast<size_t>(tok) * q_stride + static_cast<size_t>(my_head) * dim;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      const int d = ks * 32 + grp * 8;
      u32x4 raw = {0u, 0u, 0u, 0u};
      if (d < dim) raw = *reinterpret_cast<const u32x4*>(qr + d);
      qf[ks] = __builtin_bit_cast(bf16x8, raw);
    }
  }
  floatx4 o[NV];
#pragma unroll
  for (int dt = 0; dt < NV; ++dt) o[dt] = floatx4{0.f, 0.f, 0.f, 0.f};
  const bool first = sink && cut == 0 && wave == 0;  // the sink belongs to one partial result
  float m_run = first ? (sink_logit != nullptr ? sink_logit[my_head] : 0.f) : -INFINITY;
  float l_run = (first && grp == 0) ? 1.f : 0.f;

  const int first_key = first_visible(pos, window);  // a window, a chunk: the walk starts at its block
  const int kb_first = first_key / AS_BLOCK * AS_BLOCK;
  const int n_blocks = (pos - kb_first) / AS_BLOCK + 1;
  const int per_cut = (n_blocks + cuts - 1) / cuts;
  const int kb_begin = kb_first + cut * per_cut * AS_BLOCK;
  const int kb_end = kb_first + ((cut + 1) * per_cut < n_blocks ? (cut + 1) * per_cut : n_blocks) * AS_BLOCK;
  for (int kb = kb_begin + wave * AS_BLOCK; kb < kb_end; kb += 4 * AS_BLOCK) {
    const int page = table[kb / page_size];
    const int in_page = kb % page_size;
    floatx4 s[2];
#pragma unroll
    for (int t = 0; t < 2; ++t) {
      const size_t slot = static_cast<size_t>(page) * page_size + in_page + t * 16 + col;
      const bf16_t* kr = k_cache + (slot * n_kv_heads + kvh) * dim;
      s[t] = floatx4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) {
        const int d = ks * 32 + grp * 8;
        u32x4 raw = {0u, 0u, 0u, 0u};
        if (d < dim) raw = *reinterpret_cast<const u32x4*>(kr + d);
        s[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, raw), qf[ks], s[t], 0, 0, 0);
      }
    }
    bf16x8 vf[NV];
    const bool ragged = kb + AS_BLOCK - 1 > pos;
#pragma unroll
    for (int dt = 0; dt < NV; ++dt) {
      const int d = dt * 16 + col;
      u32x4 raw = {0u, 0u, 0u, 0u};
      if (d < vdim) {
        const bf16_t* vr = v_cache + ((static_cast<size_t>(page) * n_kv_heads + kvh) * vdim + d) * page_size +
                           in_page + 4 * grp;
        const u32x2 a0 = *reinterpret_cast<const u32x2*>(vr);
        const u32x2 a1 = *reinterpret_cast<const u32x2*>(vr + 16);
        raw = u32x4{a0[0], a0[1], a1[0], a1[1]};
        if (ragged) {
#pragma unroll
          for (int e = 0; e < 8; ++e) {
            const int key = kb + (e >> 2) * 16 + 4 * grp + (e & 3);
            if (key > pos) raw[e >> 1] &= (e & 1) ? 0x0000ffffu : 0xffff0000u;
          }
        }
      }
      vf[dt] = __builtin_bit_cast(bf16x8, raw);
    }
    float sc[8];
    const bool all_far = bias == nullptr || pos - (kb + AS_BLOCK - 1) >= bucket_len - 1;
    float top = m_run;
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const int key = kb + (e >> 2) * 16 + 4 * grp + (e & 3);
      const int dist = pos - key;
      float add = far_bias;
      if (!all_far) {
        int idx = dist < 0 ? 0 : dist;
        idx = idx < bucket_len - 1 ? idx : bucket_len - 1;
        add = tbl[idx];
      }
      const float v = capped_score(s[e >> 2][e & 3], scale, softcap) + add;
      sc[e] = (dist >= 0 && key >= first_key) ? v : -INFINITY;
      top = fmaxf(top, sc[e]);
    }
    top = fmaxf(top, __shfl_xor(top, 16, 64));
    top = fmaxf(top, __shfl_xor(top, 32, 64));
    const float corr = (top == -INFINITY || m_run == -INFINITY) ? (m_run == -INFINITY ? 0.f : 1.f) : __expf(m_run - top);
    float p[8], sum = 0.f;
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      p[e] = (sc[e] == -INFINITY) ? 0.f : __expf(sc[e] - top);
      sum += p[e];
    }
    l_run = l_run * corr + sum;
    m_run = top;
    u32x4 hi, lo;
#pragma unroll
    for (int e = 0; e < 8; e += 2) {
      const uint32_t a = __float_as_uint(p[e]), c = __float_as_uint(p[e + 1]);
      hi[e >> 1] = __builtin_amdgcn_perm(c, a, 0x07060302u);
      const float ra = p[e] - __uint_as_float(a & 0xffff0000u), rc = p[e + 1] - __uint_as_float(c & 0xffff0000u);
      lo[e >> 1] = __builtin_amdgcn_perm(__float_as_uint(rc), __float_as_uint(ra), 0x07060302u);
    }
    const bf16x8 p_hi = __builtin_bit_cast(bf16x8, hi), p_lo = __builtin_bit_cast(bf16x8, lo);
#pragma unroll
    for (int dt = 0; dt < NV; ++dt) {
      floatx4 acc = o[dt];
      acc[0] *= corr; acc[1] *= corr; acc[2] *= corr; acc[3] *= corr;
      acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf[dt], p_hi, acc, 0, 0, 0);
      o[dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf[dt], p_lo, acc, 0, 0, 0);
    }
  }
  float l = l_run;
  l += __shfl_xor(l, 16, 64);
  l += __shfl_xor(l, 32, 64);
  float* mrg = bias_lds + (bias != nullptr ? group * bucket_len : 4);  // [4 waves][group][2 + vdim]
  if (col < group) {
    float* mine = mrg + (wave * group + col) * (2 + vdim);
    if (grp == 0) {
      mine[0] = m_run;
      mine[1] = l;
    }
#pragma unroll
    for (int dt = 0; dt < NV; ++dt)
#pragma unroll
      for (int i = 0; i < 4; ++i)
        if (dt * 16 + 4 * grp + i < vdim) mine[2 + dt * 16 + 4 * grp + i] = o[dt][i];
  }
  __syncthreads();
  for (int idx = threadIdx.x; idx < group * vdim; idx += 256) {
    const int h = idx / vdim, d = idx - h * vdim;
    const float* src = mrg + h * (2 + vdim);
    const int stride = group * (2 + vdim);
    float m = -INFINITY;
#pragma unroll
    for (int w = 0; w < 4; ++w) m = fmaxf(m, src[w * stride]);
    float total = 0.f, acc = 0.f;
#pragma unroll
    for (int w = 0; w < 4; ++w) {
      const float mw = src[w * stride];
      const float f = (mw == -INFINITY) ? 0.f : __expf(mw - m);
      total = fmaf(src[w * stride + 1], f, total);
      acc = fmaf(src[w * stride + 2 + d], f, acc);
    }
    const size_t item = static_cast<size_t>(tok) * n_heads + kvh * group + h;
    if (cuts == 1) {
      out[item * vdim + d].bits = float_to_bf16_bits(acc / total);
    } else {
      float* dst = partial + (item * cuts + cut) * (2 + vdim);
      if (d == 0) {
        dst[0] = m;
        dst[1] = total;
      }
      dst[2 + d] = acc;
    }
  }
}

// One wave per (token, head): out = sum_c o_c e^(m_c - m) / sum_c l_c e^(m_c - m), cuts in order.
__global__ void attention_sink_merge_kernel(bf16_t* __restrict__ out, const float* __restrict__ partial, int items,
                                            int cuts, int vdim) {
  const int item = blockIdx.x * (blockDim.x / 64) + (threadIdx.x >> 6);
  const int lane = threadIdx.x & 63;
  if (item >= items) return;
  const float* src = partial + static_cast<size_t>(item) * cuts * (2 + vdim);
  // lane c takes cut c's maximum and sum (at most 64 cuts); the values come in a loop whose loads
  // do not wait for one another
  const float mc = lane < cuts ? src[lane * (2 + vdim)] : -INFINITY;
  const float lc = lane < cuts ? src[lane * (2 + vdim) + 1] : 0.f;
  const float m = wave_max(mc);
  const float w = (mc == -INFINITY) ? 0.f : __expf(mc - m);
  const float inv = 1.0f / wave_sum(lc * w);
  for (int d0 = 0; d0 < vdim; d0 += 64) {  // every lane stays in the loop: its weight is read by the others
    const int d = d0 + lane;
    const bool mine = d < vdim;
    float acc = 0.f;
#pragma unroll 8
    for (int c = 0; c < cuts; ++c) acc = fmaf(mine ? src[c * (2 + vdim) + 2 + d] : 0.f, __shfl(w, c, 64), acc);
    if (mine) out[static_cast<size_t>(item) * vdim + d].bits = float_to_bf16_bits(acc * inv);
  }
}

// q: bf16 [tokens, n_heads, dim], rows q_stride elements apart; out: bf16 [tokens, n_heads, vdim].
// k_cache: bf16 [pages * page_size, n_kv_heads, dim]; v_cache: bf16 [pages, n_kv_heads, vdim, page_size].
// tiles: int [n_tiles, 4] = (first token, count <= 32, block-table row, first position) of runs of
// consecutive tokens of one request; or null, and then positions: int [n_tiles], one token per tile,
// token t on row t of the block table (a step of single tokens).  bias: null or float [n_heads, bucket_len
// <= 4096], a head's bias by distance, the last entry for every distance from bucket_len - 1 on.  dim a multiple of 8 up to 256, vdim a multiple of 4
// up to 256, page_size a multiple of 32.  window: the mask as one integer (first_visible in common.h).
// The host guarantees that the tiles lie inside q and the table.
extern "C" int pylon_attention_sink(void* out, const void* q, long long q_stride, const void* k_cache,
                                    const void* v_cache, const int* block_table, int table_width, const int* tiles,
                                    const int* positions, int n_tiles, int n_heads, int n_kv_heads, int dim, int vdim, int page_size,
                                    float scale, const float* bias, int bucket_len, int sink,
                                    int cuts, float* partial, long long partial_floats, int tokens, int window,
                                    float softcap, const float* sink_logit, hipStream_t stream) {
  PYLON_REQUIRE(sink_logit == nullptr || sink, "attention_sink: a learned sink is a sink");
  PYLON_REQUIRE(n_tiles >= 0 && n_heads > 0 && n_kv_heads > 0 && n_heads % n_kv_heads == 0,
                "attention_sink: %d query heads cannot be grouped over %d key/value heads", n_heads, n_kv_heads);
  PYLON_REQUIRE(dim >= 8 && dim % 8 == 0 && dim <= 256, "attention_sink: keys of a multiple of 8 up to 256 elements, got %d", dim);
  PYLON_REQUIRE(vdim >= 4 && vdim % 4 == 0 && vdim <= 256, "attention_sink: values of a multiple of 4 up to 256 elements, got %d", vdim);
  PYLON_REQUIRE(page_size > 0 && page_size % AS_BLOCK == 0, "attention_sink: pages of a multiple of %d tokens, got %d", AS_BLOCK, page_size);
  PYLON_REQUIRE(table_width > 0 && q_stride >= static_cast<long long>(n_heads) * dim && q_stride % 8 == 0,
                "attention_sink: bad table width or q stride");
  PYLON_REQUIRE((reinterpret_cast<uintptr_t>(q) & 15) == 0 && (reinterpret_cast<uintptr_t>(k_cache) & 15) == 0 &&
                (reinterpret_cast<uintptr_t>(v_cache) & 7) == 0 && (reinterpret_cast<uintptr_t>(out) & 7) == 0,
                "attention_sink: operands must be 16-byte aligned");
  PYLON_REQUIRE(tiles != nullptr || positions != nullptr, "attention_sink: tiles or positions are required");
  PYLON_REQUIRE(bias == nullptr || (bucket_len >= 1 && bucket_len <= AS_MAX_BIAS),
                "attention_sink: a bias by distance is a table of 1 to %d entries a head", AS_MAX_BIAS);
  PYLON_REQUIRE(cuts >= 1 && cuts <= 64, "attention_sink: 1 to 64 cuts, got %d", cuts);
  const int group = n_heads / n_kv_heads;
  // single tokens whose group of heads fits a tile's columns and whose bias tables fit LDS: the
  // kernel with the heads side by side, four partial results a cut
  const bool side_by_side = tiles == nullptr && group <= 16 &&
                            (bias == nullptr || static_cast<long long>(group) * bucket_len * 4 <= 64 * 1024) &&
                            (cuts == 1 || (partial != nullptr &&
                                           partial_floats >= static_cast<long long>(tokens) * n_heads * cuts * (2 + vdim)));
  PYLON_REQUIRE(side_by_side || cuts == 1 ||
                    (partial != nullptr && partial_floats >= static_cast<long long>(tokens) * n_heads * cuts * (2 + vdim)),
                "attention_sink: cut keys need room for their partial results");
  if (n_tiles == 0) return 0;
  if (side_by_side) {
    const long long wgs = static_cast<long long>(tokens) * n_kv_heads * cuts;
    PYLON_REQUIRE(wgs < (1ll << 31), "attention_sink: too many workgroups for one launch");
    const size_t lds_d = sizeof(float) * ((bias != nullptr ? group * bucket_len : 4) + 4 * group * (2 + vdim));
    const int ks_d = (dim + 31) / 32, nv_d = (vdim + 15) / 16;
#define GO_D(KS, NV)                                                                                                \
  do {                                                                                                              \
    if (lds_d > 48 * 1024)                                                                                          \
      (void)hipFuncSetAttribute(reinterpret_cast<const void*>(&attention_sink_decode_kernel<KS, NV>),                \
                                hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(lds_d));                \
    hipLaunchKernelGGL((attention_sink_decode_kernel<KS, NV>), dim3(static_cast<unsigned>(wgs)), dim3(256), lds_d,    \
                       stream, (bf16_t*)out, (const bf16_t*)q, q_stride, (const bf16_t*)k_cache, (const bf16_t*)v_cache,           \
                       block_table, table_width, positions, n_heads, n_kv_heads, dim, vdim, page_size, scale, bias,  \
                       bias != nullptr ? bucket_len : 1, sink, cuts, partial, window, softcap, sink_logit);          \
  } while (0)
#define PICK_D(KS)                  \
  do {                              \
    if (nv_d <= 2) GO_D(KS, 2);     \
    else if (nv_d <= 4) GO_D(KS, 4);\
    else if (nv_d <= 8) GO_D(KS, 8);\
    else GO_D(KS, 16);              \
  } while (0)
    if (ks_d <= 1) PICK_D(1);
    else if (ks_d <= 2) PICK_D(2);
    else if (ks_d <= 4) PICK_D(4);
    else PICK_D(8);
#undef PICK_D
#undef GO_D
    if (cuts > 1) {
      const int items = tokens * n_heads;
      hipLaunchKernelGGL(attention_sink_merge_kernel, dim3((items + 3) / 4), dim3(256), 0, stream, (bf16_t*)out,
                         partial, items, cuts, vdim);
    }
    PYLON_LAUNCHED("attention_sink");
  }
  const int waves = 4;
  const int chunks = (group + waves - 1) / waves;
  const long long blocks = static_cast<long long>(n_tiles) * n_kv_heads * chunks * cuts;
  PYLON_REQUIRE(blocks < (1ll << 31), "attention_sink: too many tiles for one launch");
  dim3 grid(static_cast<unsigned>(blocks)), block(2 * 64 * waves);
  const int table_len = bias != nullptr ? bucket_len : 1;
  const size_t lds = sizeof(float) * waves * ((table_len + 3) & ~3) +
                     2 * 2 * (static_cast<size_t>(AS_BLOCK) * (dim + 8) +
                              static_cast<size_t>((vdim + 15) / 16 * 16) * (AS_BLOCK + 4));  // two buffers of bfloat16
  PYLON_REQUIRE(lds <= 160 * 1024, "attention_sink: the bias table and a block do not fit LDS");
  const int ks = (dim + 31) / 32, nv = (vdim + 15) / 16;
#define GO(KS, NV) \
  do { \
  if (lds > 48 * 1024) \
    (void)hipFuncSetAttribute(reinterpret_cast<const void*>(&attention_sink_kernel<KS, NV>), \
                              hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(lds)); \
  hipLaunchKernelGGL((attention_sink_kernel<KS, NV>), grid, block, lds, stream, (bf16_t*)out, (const bf16_t*)q, \
                     q_stride, (const bf16_t*)k_cache, (const bf16_t*)v_cache, block_table, table_width, tiles, \
                     positions, n_heads, n_kv_heads, dim, vdim, page_size, scale, bias, table_len, sink, cuts, partial, window, \
                     softcap, sink_logit); \
  } while (0)
#define PICK_NV(KS)                 \
  do {                              \
    if (nv <= 2) GO(KS, 2);         \
    else if (nv <= 4) GO(KS, 4);    \
    else if (nv <= 8) GO(KS, 8);    \
    else GO(KS, 16);                \
  } while (0)
  if (ks <= 1) PICK_NV(1);
  else if (ks <= 2) PICK_NV(2);
  else if (ks <= 4) PICK_NV(4);
  else PICK_NV(8);
#undef PICK_NV
#undef GO
  if (cuts > 1) {
    const int items = tokens * n_heads;
    hipLaunchKernelGGL(attention_sink_merge_kernel, dim3((items + 3) / 4), dim3(256), 0, stream, (bf16_t*)out, partial,
                       items, cuts, vdim);
  }
  PYLON_LAUNCHED("attention_sink");
}
