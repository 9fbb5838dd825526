// A short causal convolution over time on every channel, added to its input:
//
//   out[t, c] = h[t, c] + sum_{j < taps} w[c, j] * h[t - taps + 1 + j, c]
//
// with zeros before a request's first token; or, with mode 1, the convolution alone through an
// activation, out[t, c] = silu(sum_j w[c, j] * h[t - taps + 1 + j, c]).  The rows of h may lie
// further apart than width (a slice of a wider projection).  The last taps - 1 inputs of every request are
// kept in its state slot, float [taps - 1, width] (oldest first), so that a request may come
// in portions: a portion's first tokens read what the portion before left there.
//
// A workgroup takes up to CONV_TILE consecutive tokens of one row of the step and 256 channels;
// a thread walks its channel through the tile with the window in registers.  The thread that
// has a row's first tile is the only one that reads that row's old state, and it writes the
// new one after it has read the old: no other thread touches that (row, channel).
#include "common.h"

#define CONV_TILE 16
#define CONV_MAX_TAPS 8

template <typename TI, typename TW, typename TO>
__global__ void short_conv_kernel(TO* __restrict__ out, const TI* __restrict__ h, const TW* __restrict__ w,
                                  float* state, const int* __restrict__ row_start,
                                  const int* __restrict__ row_slots, int tiles_per_row, int width, int taps,
                                  long long h_stride, int mode) {
  const int row = blockIdx.x / tiles_per_row;
  const int tile = blockIdx.x - row * tiles_per_row;
  const int begin = row_start[row], end = row_start[row + 1];
  const int a = begin + tile * CONV_TILE;
  if (a >= end) return;
  const int b = a + CONV_TILE < end ? a + CONV_TILE : end;
  const int c = blockIdx.y * blockDim.x + threadIdx.x;
  if (c >= width) return;
  const int keep = taps - 1;
  float* st = state + (static_cast<size_t>(row_slots[row]) * keep) * width + c;
  float wt[CONV_MAX_TAPS], win[CONV_MAX_TAPS], old[CONV_MAX_TAPS];
#pragma unroll
  for (int j = 0; j < CONV_MAX_TAPS; ++j) {
    wt[j] = j < taps ? to_float(w[static_cast<size_t>(c) * taps + j]) : 0.f;
    win[j] = 0.f;
    old[j] = 0.f;
  }
  const bool first_tile = tile == 0;
  if (first_tile) {
#pragma unroll
    for (int i = 0; i < CONV_MAX_TAPS - 1; ++i)
      if (i < keep) old[i] = st[static_cast<size_t>(i) * width];
  }
  // win[j] holds the input taps - 1 - j steps before the token in hand; win[taps - 1] is its own.
#pragma unroll
  for (int j = 0; j < CONV_MAX_TAPS - 1; ++j) {
    if (j < keep) {
      const int src = a - keep + j;  // token index of the step
      if (src >= begin) win[j + 1] = to_float(h[static_cast<size_t>(src) * h_stride + c]);
      else if (first_tile) win[j + 1] = old[keep - (begin - src)];
    }
  }
  // a tile's inputs are fetched before the first sum, so that their trips to memory overlap
  float xs[CONV_TILE];
#pragma unroll
  for (int n = 0; n < CONV_TILE; ++n) xs[n] = (a + n < b) ? to_float(h[static_cast<size_t>(a + n) * h_stride + c]) : 0.f;
#pragma unroll
  for (int n = 0; n < CONV_TILE; ++n) {
    const int t = a + n;
    if (t >= b) break;
#pragma unroll
    for (int j = 0; j < CONV_MAX_TAPS - 1; ++j) win[j] = win[j + 1];
    const float x = xs[n];
#pragma unroll
    for (int j = 0; j < CONV_MAX_TAPS; ++j)
      if (j == taps - 1) win[j] = x;
    float acc = 0.f;
#pragma unroll
    for (int j = 0; j < CONV_MAX_TAPS; ++j)
      if (j < taps) acc = fmaf(wt[j], win[j], acc);
    out[static_cast<size_t>(t) * width + c] = from_float<TO>(mode == 1 ? acc / (1.0f + expf(-acc)) : x + acc);
  }
  if (first_tile) {
#pragma unroll
    for (int i = 0; i < CONV_MAX_TAPS - 1; ++i) {
      if (i < keep) {
        const int src = end - keep + i;
        float v;
        if (src >= begin) v = to_float(h[static_cast<size_t>(src) * h_stride + c]);
        else v = old[keep - (begin - src)];
        st[static_cast<size_t>(i) * width] = v;
      }
    }
  }
}

// h: [tokens, width] of in_dtype, rows h_stride elements apart; w: [width, taps] of w_dtype; out:
// [tokens, width] of out_dtype; mode 0: input plus convolution, 1: silu of the convolution;
// state: float [slots, taps - 1, width]; row_start: [rows + 1] prefix sums of the rows' token
// counts; row_slots: [rows] state slot of each row; max_count: the most tokens any row brings
// (an upper bound will do).  The host guarantees row_slots < slots and row_start[rows] <= tokens.
extern "C" int pylon_short_conv(void* out, int out_dtype, const void* h, int in_dtype, const void* w, int w_dtype,
                                float* state, const int* row_start, const int* row_slots, int rows, int max_count,
                                int width, int taps, long long h_stride, int mode, hipStream_t stream) {
  PYLON_REQUIRE(pylon_valid_dtype(out_dtype) && pylon_valid_dtype(in_dtype) && pylon_valid_dtype(w_dtype),
                "short_conv: unknown dtype");
  PYLON_REQUIRE(taps >= 1 && taps <= CONV_MAX_TAPS, "short_conv: 1 to %d taps, got %d", CONV_MAX_TAPS, taps);
  PYLON_REQUIRE(CONV_TILE >= CONV_MAX_TAPS, "short_conv: a tile must hold a window");
  PYLON_REQUIRE(rows >= 0 && max_count >= 0 && width > 0, "short_conv: bad sizes");
  PYLON_REQUIRE(h_stride >= width && (mode == 0 || mode == 1), "short_conv: rows overlap, or an unknown mode");
  PYLON_REQUIRE(taps == 1 || state != nullptr, "short_conv: a window over several tokens needs its state");
  if (rows == 0 || max_count == 0) return 0;
  const int tiles_per_row = (max_count + CONV_TILE - 1) / CONV_TILE;
  PYLON_REQUIRE(static_cast<long long>(rows) * tiles_per_row < (1ll << 31), "short_conv: too many tiles");
  dim3 grid(static_cast<unsigned>(rows * tiles_per_row), (width + 255) / 256), block(256);
#define GO(TI, TW, TO)                                                                                       \
  hipLaunchKernelGGL((short_conv_kernel<TI, TW, TO>), grid, block, 0, stream, (TO*)out, (const TI*)h,        \
                     (const TW*)w, state, row_start, row_slots, tiles_per_row, width, taps, h_stride, mode)
  const int key = (in_dtype == PYLON_F32 ? 4 : 0) | (w_dtype == PYLON_F32 ? 2 : 0) | (out_dtype == PYLON_F32 ? 1 : 0);
  switch (key) {
    case 0: GO(bf16_t, bf16_t, bf16_t); break;
    case 1: GO(bf16_t, bf16_t, float); break;
    case 2: GO(bf16_t, float, bf16_t); break;
    case 3: GO(bf16_t, float, float); break;
    case 4: GO(float, bf16_t, bf16_t); break;
    case 5: GO(float, bf16_t, float); break;
    case 6: GO(float, float, bf16_t); break;
    default: GO(float, float, float); break;
  }
#undef GO
  PYLON_LAUNCHED("short_conv");
}

// ---- token shift -------------------------------------------------------------------------------
//   out[t, c] = h[t, c] + (h[t - 1, c] - h[t, c]) * shift[c]
// with zeros before a request's first token; a request's last input is kept in its state slot,
// float [width].  Tiles and the ownership of the state as in the convolution above: the thread with
// a row's first tile reads the old state, and writes the new one after it has read the old.
template <typename TI, typename TO>
__global__ void token_shift_kernel(TO* __restrict__ out, const TI* __restrict__ h, const float* __restrict__ shift,
                                   float* state, const int* __restrict__ row_start,
                                   const int* __restrict__ row_slots, int tiles_per_row, int width) {
  const int row = blockIdx.x / tiles_per_row;
  const int tile = blockIdx.x - row * tiles_per_row;
  const int begin = row_start[row], end = row_start[row + 1];
  const int a = begin + tile * CONV_TILE;
  if (a >= end) return;
  const int b = a + CONV_TILE < end ? a + CONV_TILE : end;
  const int c = blockIdx.y * blockDim.x + threadIdx.x;
  if (c >= width) return;
  float* st = state + static_cast<size_t>(row_slots[row]) * width + c;
  const float s = shift[c];
  float prev = tile == 0 ? st[0] : to_float(h[static_cast<size_t>(a - 1) * width + c]);
  float xs[CONV_TILE];
#pragma unroll
  for (int n = 0; n < CONV_TILE; ++n) xs[n] = (a + n < b) ? to_float(h[static_cast<size_t>(a + n) * width + c]) : 0.f;
#pragma unroll
  for (int n = 0; n < CONV_TILE; ++n) {
    if (a + n >= b) break;
    const float x = xs[n];
    out[static_cast<size_t>(a + n) * width + c] = from_float<TO>(fmaf(prev - x, s, x));
    prev = x;
  }
  if (tile == 0) st[0] = to_float(h[static_cast<size_t>(end - 1) * width + c]);
}

// h: [tokens, width] of in_dtype; shift: float [width]; out: [tokens, width] of out_dtype; state: float
// [slots, width]; row_start, row_slots, max_count as for the convolution.
extern "C" int pylon_token_shift(void* out, int out_dtype, const void* h, int in_dtype, const float* shift,
                                 float* state, const int* row_start, const int* row_slots, int rows, int max_count,
                                 int width, hipStream_t stream) {
  PYLON_REQUIRE(pylon_valid_dtype(out_dtype) && pylon_valid_dtype(in_dtype), "token_shift: unknown dtype");
  PYLON_REQUIRE(rows >= 0 && max_count >= 0 && width > 0, "token_shift: bad sizes");
  PYLON_REQUIRE(state != nullptr && shift != nullptr, "token_shift: the state and the weights are required");
  if (rows == 0 || max_count == 0) return 0;
  const int tiles_per_row = (max_count + CONV_TILE - 1) / CONV_TILE;
  PYLON_REQUIRE(static_cast<long long>(rows) * tiles_per_row < (1ll << 31), "token_shift: too many tiles");
  dim3 grid(static_cast<unsigned>(rows * tiles_per_row), (width + 255) / 256), block(256);
#define GO(TI, TO)                                                                                        \
  hipLaunchKernelGGL((token_shift_kernel<TI, TO>), grid, block, 0, stream, (TO*)out, (const TI*)h, shift, \
                     state, row_start, row_slots, tiles_per_row, width)
  if (in_dtype == PYLON_F32 && out_dtype == PYLON_F32) GO(float, float);
  else if (in_dtype == PYLON_F32) GO(float, bf16_t);
  else if (out_dtype == PYLON_F32) GO(bf16_t, float);
  else GO(bf16_t, bf16_t);
#undef GO
  PYLON_LAUNCHED("token_shift");
}
