// A short causal convolution over time on every channel of a slice of a projected matrix, continued from step to
// step through a state that holds the last taps - 1 inputs of each sequence:
//   y[t][c] = sum_j w[c][j] * u[t - taps + 1 + j][c]  (+ bias[c])  (then silu),   zeros before a sequence starts.
//   short_conv        the rows of a step; inputs that lie before the step come from the state
//   short_conv_state  the state after the step (run it after every reader of the old state)
// State of one sequence: [taps - 1][channels] float32, the oldest input first, at `state + slot * slot_stride`.
// Sums are float32; the result is float32.
#include "common.h"

#define SC_MAX_TAPS 16

template <typename T>
__global__ __launch_bounds__(256) void short_conv_kernel(const T* __restrict__ u, int row_stride, int first,
                                                         const float* __restrict__ w, const float* __restrict__ bias,
                                                         const float* __restrict__ state, long slot_stride,
                                                         const int32_t* __restrict__ row_seq, const int32_t* __restrict__ seq_start,
                                                         const int32_t* __restrict__ seq_slot, float* __restrict__ out,
                                                         int n_rows, int channels, int taps, int silu) {
  const int c = blockIdx.x * blockDim.x + threadIdx.x;
  if (c >= channels) return;
  float wc[SC_MAX_TAPS];
#pragma unroll
  for (int j = 0; j < SC_MAX_TAPS; ++j) wc[j] = j < taps ? w[(size_t)c * taps + j] : 0.f;
  const float b = bias ? bias[c] : 0.f;
  for (int row = blockIdx.y; row < n_rows; row += gridDim.y) {
    const int seq = row_seq[row];
    const int t = row - seq_start[seq];      // the row's place among its sequence's rows of this step
    const float* old = state + (size_t)seq_slot[seq] * slot_stride;
    float acc = b;
#pragma unroll
    for (int j = 0; j < SC_MAX_TAPS; ++j) {
      if (j >= taps) break;
      const int back = taps - 1 - j;         // how many rows before this one
      float v;
      if (back <= t) v = to_f32(u[(size_t)(row - back) * row_stride + first + c]);
      else v = old[(size_t)(taps - 1 + t - back) * channels + c];
      acc = fmaf(wc[j], v, acc);
    }
    if (silu) acc = acc / (1.0f + expf(-acc));
    out[(size_t)row * channels + c] = acc;
  }
}

// The same for steps of many rows: a thread walks SC_ROWS consecutive rows of its channel with the last TAPS inputs in
// registers, so that every input is loaded once (where a sequence starts inside the stretch, the window is filled anew
// from that sequence's state).
#define SC_ROWS 32

template <typename T, int TAPS>
__global__ __launch_bounds__(256) void short_conv_walk_kernel(const T* __restrict__ u, int row_stride, int first,
                                                              const float* __restrict__ w, const float* __restrict__ bias,
                                                              const float* __restrict__ state, long slot_stride,
                                                              const int32_t* __restrict__ row_seq, const int32_t* __restrict__ seq_start,
                                                              const int32_t* __restrict__ seq_slot, float* __restrict__ out,
                                                              int n_rows, int channels, int silu) {
  const int c = blockIdx.x * blockDim.x + threadIdx.x;
  if (c >= channels) return;
  float wc[TAPS], win[TAPS];
#pragma unroll
  for (int j = 0; j < TAPS; ++j) wc[j] = w[(size_t)c * TAPS + j];
  const float b = bias ? bias[c] : 0.f;
  const int r0 = blockIdx.y * SC_ROWS, r1 = r0 + SC_ROWS < n_rows ? r0 + SC_ROWS : n_rows;
  int seq = -1;
  for (int row = r0; row < r1; ++row) {
    const int here = row_seq[row];
    if (here != seq) {      // the first row of the stretch, or of a sequence: the inputs before it
      seq = here;
      const int t = row - seq_start[seq];
      const float* old = state + (size_t)seq_slot[seq] * slot_stride;
#pragma unroll
      for (int j = 0; j < TAPS - 1; ++j) {
        const int back = TAPS - 1 - j;
        win[j] = back <= t ? to_f32(u[(size_t)(row - back) * row_stride + first + c]) : old[(size_t)(TAPS - 1 + t - back) * channels + c];
      }
    } else {
#pragma unroll
      for (int j = 0; j < TAPS - 1; ++j) win[j] = win[j + 1];
    }
    win[TAPS - 1] = to_f32(u[(size_t)row * row_stride + first + c]);
    float acc = b;
#pragma unroll
    for (int j = 0; j < TAPS; ++j) acc = fmaf(wc[j], win[j], acc);
    if (silu) acc = acc / (1.0f + expf(-acc));
    out[(size_t)row * channels + c] = acc;
  }
}

extern "C" int bh_short_conv(const void* u, int dtype, int row_stride, int first, const float* w, const float* bias,
                             const float* state, long slot_stride, const int32_t* row_seq, const int32_t* seq_start,
                             const int32_t* seq_slot, float* out, int n_rows, int channels, int taps, int silu,
                             hipStream_t stream) {
  BH_REQUIRE(n_rows > 0 && channels > 0, "short_conv: sizes must be positive");
  BH_REQUIRE(taps >= 1 && taps <= SC_MAX_TAPS, "short_conv: 1 to %d taps, got %d", SC_MAX_TAPS, taps);
  BH_REQUIRE(first >= 0 && first + channels <= row_stride, "short_conv: channels %d..%d lie outside a row of %d", first,
             first + channels, row_stride);
  BH_REQUIRE(taps == 1 || state != nullptr, "short_conv: more than one tap needs a state");
  if (n_rows >= 4 * SC_ROWS && taps >= 2 && taps <= 4 && (dtype == BH_F32 || dtype == BH_BF16)) {
    dim3 walk((channels + 255) / 256, (n_rows + SC_ROWS - 1) / SC_ROWS);
#define BH_SW(T, TAPS)                                                                                                              \
  short_conv_walk_kernel<T, TAPS><<<walk, 256, 0, stream>>>((const T*)u, row_stride, first, w, bias, state, slot_stride, row_seq, seq_start, \
                                                            seq_slot, out, n_rows, channels, silu)
    if (dtype == BH_F32) {
      if (taps == 2) BH_SW(float, 2);
      else if (taps == 3) BH_SW(float, 3);
      else BH_SW(float, 4);
    } else {
      if (taps == 2) BH_SW(bf16_t, 2);
      else if (taps == 3) BH_SW(bf16_t, 3);
      else BH_SW(bf16_t, 4);
    }
#undef BH_SW
    return bh_check_launch("short_conv");
  }
  dim3 grid((channels + 255) / 256, n_rows < 4096 ? n_rows : 4096);
  if (dtype == BH_F32)
    short_conv_kernel<float><<<grid, 256, 0, stream>>>((const float*)u, row_stride, first, w, bias, state, slot_stride, row_seq,
                                                       seq_start, seq_slot, out, n_rows, channels, taps, silu);
  else if (dtype == BH_BF16)
    short_conv_kernel<bf16_t><<<grid, 256, 0, stream>>>((const bf16_t*)u, row_stride, first, w, bias, state, slot_stride, row_seq,
                                                        seq_start, seq_slot, out, n_rows, channels, taps, silu);
  else
    return bh_fail("short_conv: unknown dtype %d", dtype);
  return bh_check_launch("short_conv");
}

// One thread a (sequence, channel): it reads what the new state takes from the old one before it writes.
template <typename T>
__global__ __launch_bounds__(256) void short_conv_state_kernel(const T* __restrict__ u, int row_stride, int first,
                                                               float* __restrict__ state, long slot_stride,
                                                               const int32_t* __restrict__ seq_start,
                                                               const int32_t* __restrict__ seq_slot, int channels, int taps) {
  const int c = blockIdx.x * blockDim.x + threadIdx.x, seq = blockIdx.y;
  if (c >= channels) return;
  const int start = seq_start[seq], n_new = seq_start[seq + 1] - start, keep = taps - 1;
  float* mine = state + (size_t)seq_slot[seq] * slot_stride;
  float next[SC_MAX_TAPS];
#pragma unroll
  for (int s = 0; s < SC_MAX_TAPS; ++s) {
    if (s >= keep) break;
    const int at = n_new + s - keep;        // index into the step's rows; negative: still an old input
    next[s] = at >= 0 ? to_f32(u[(size_t)(start + at) * row_stride + first + c]) : mine[(size_t)(n_new + s) * channels + c];
  }
#pragma unroll
  for (int s = 0; s < SC_MAX_TAPS; ++s) {
    if (s >= keep) break;
    mine[(size_t)s * channels + c] = next[s];
  }
}

extern "C" int bh_short_conv_state(const void* u, int dtype, int row_stride, int first, float* state, long slot_stride,
                                   const int32_t* seq_start, const int32_t* seq_slot, int n_seqs, int channels, int taps,
                                   hipStream_t stream) {
  BH_REQUIRE(n_seqs > 0 && channels > 0, "short_conv_state: sizes must be positive");
  BH_REQUIRE(taps >= 1 && taps <= SC_MAX_TAPS, "short_conv_state: 1 to %d taps, got %d", SC_MAX_TAPS, taps);
  BH_REQUIRE(first >= 0 && first + channels <= row_stride, "short_conv_state: channels lie outside a row");
  if (taps == 1) return 0;
  dim3 grid((channels + 255) / 256, n_seqs);
  if (dtype == BH_F32)
    short_conv_state_kernel<float><<<grid, 256, 0, stream>>>((const float*)u, row_stride, first, state, slot_stride, seq_start,
                                                             seq_slot, channels, taps);
  else if (dtype == BH_BF16)
    short_conv_state_kernel<bf16_t><<<grid, 256, 0, stream>>>((const bf16_t*)u, row_stride, first, state, slot_stride, seq_start,
                                                              seq_slot, channels, taps);
  else
    return bh_fail("short_conv_state: unknown dtype %d", dtype);
  return bh_check_launch("short_conv_state");
}
