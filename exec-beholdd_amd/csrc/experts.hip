// Routed experts: each row chooses `top` of E small gated feed-forward layers by the largest router logits and
// adds their outputs, weighted by the softmax over the chosen logits alone.
//   route_top_k        chosen [rows][top] (int32, largest first, ties to the lower index) and weights [rows][top]
//   experts_gate_up    per (row, chosen expert): inner = act(Wg_e h, Wu_e h)             (weights read per pair: the
//   experts_down       per row: h_res += sum_j weight_j * Wd_ej inner_j, j in order       form for steps of few rows)
//   clamped_glu        act over a stacked [gate | up] matrix (the shared expert, and experts run as products of rows)
//   act(g, u) = g' * sigmoid(alpha g') * (u' + 1),  g' = min(g, limit),  u' = clamp(u, -limit, limit)
// Router logits, the softmax and all sums are float32.
#include "common.h"

__device__ inline float clamped_glu(float g, float u, float limit, float alpha) {
  g = fminf(g, limit);
  u = fminf(fmaxf(u, -limit), limit);
  return g / (1.0f + expf(-alpha * g)) * (u + 1.0f);
}

#define ROUTE_MAX_TOP 32

// One thread a row.
__global__ __launch_bounds__(64) void route_top_k_kernel(const float* __restrict__ logits, const float* __restrict__ bias,
                                                        int32_t* __restrict__ chosen, float* __restrict__ weights, int n_rows,
                                                        int E, int top) {
  const int row = blockIdx.x * blockDim.x + threadIdx.x;
  if (row >= n_rows) return;
  const float* z = logits + (size_t)row * E;
  int picked[ROUTE_MAX_TOP];
  float value[ROUTE_MAX_TOP];
  for (int j = 0; j < top; ++j) {
    int best = -1;
    float best_v = 0.f;
    for (int e = 0; e < E; ++e) {
      bool taken = false;
      for (int i = 0; i < j; ++i) taken |= picked[i] == e;
      if (taken) continue;
      const float v = z[e] + (bias ? bias[e] : 0.f);
      if (best < 0 || v > best_v) {
        best = e;
        best_v = v;
      }
    }
    picked[j] = best;
    value[j] = best_v;
  }
  float sum = 0.f;
  const float largest = value[0];
  for (int j = 0; j < top; ++j) {
    value[j] = expf(value[j] - largest);
    sum += value[j];
  }
  for (int j = 0; j < top; ++j) {
    chosen[(size_t)row * top + j] = picked[j];
    weights[(size_t)row * top + j] = value[j] / sum;
  }
}

extern "C" int bh_route_top_k(const float* logits, const float* bias, int32_t* chosen, float* weights, int n_rows, int E, int top,
                              hipStream_t stream) {
  BH_REQUIRE(n_rows > 0 && E > 0, "route_top_k: sizes must be positive");
  BH_REQUIRE(top >= 1 && top <= E && top <= ROUTE_MAX_TOP, "route_top_k: 1 to min(%d, %d) experts a row, got %d", E, ROUTE_MAX_TOP, top);
  route_top_k_kernel<<<(n_rows + 63) / 64, 64, 0, stream>>>(logits, bias, chosen, weights, n_rows, E, top);
  return bh_check_launch("route_top_k");
}

// A wave's dot product of a weight row with a vector kept in LDS as float32; every lane gets the sum.
template <typename T>
__device__ inline float wave_dot(const T* __restrict__ w, const float* __restrict__ x, int K, int lane) {
  float acc = 0.f;
  if (K % 4 == 0) {
    for (int k = lane * 4; k < K; k += BH_WAVE * 4) {
      acc = fmaf(to_f32(w[k]), x[k], acc);
      acc = fmaf(to_f32(w[k + 1]), x[k + 1], acc);
      acc = fmaf(to_f32(w[k + 2]), x[k + 2], acc);
      acc = fmaf(to_f32(w[k + 3]), x[k + 3], acc);
    }
  } else {
    for (int k = lane; k < K; k += BH_WAVE) acc = fmaf(to_f32(w[k]), x[k], acc);
  }
  return wave_sum(acc);
}

#define EX_WAVES 4
#define EX_OUTS 16      // outputs a workgroup computes

// grid (pairs, ceil(ff / EX_OUTS)); w_gu [E][2 ff][K]: an expert's gate rows, then its up rows.
template <typename T>
__global__ __launch_bounds__(256) void experts_gate_up_kernel(const T* __restrict__ h, const int32_t* __restrict__ chosen,
                                                              const T* __restrict__ w_gu, T* __restrict__ inner, int top, int K, int ff,
                                                              float limit, float alpha) {
  extern __shared__ float xs[];
  const int pair = blockIdx.x, row = pair / top, e = chosen[pair];
  for (int k = threadIdx.x; k < K; k += blockDim.x) xs[k] = to_f32(h[(size_t)row * K + k]);
  __syncthreads();
  const int lane = threadIdx.x & (BH_WAVE - 1), wave = threadIdx.x / BH_WAVE;
  const T* base = w_gu + (size_t)e * 2 * ff * K;
  for (int i = wave; i < EX_OUTS; i += EX_WAVES) {
    const int o = blockIdx.y * EX_OUTS + i;
    if (o >= ff) break;
    const float g = wave_dot(base + (size_t)o * K, xs, K, lane);
    const float u = wave_dot(base + (size_t)(ff + o) * K, xs, K, lane);
    if (lane == 0) inner[(size_t)pair * ff + o] = from_f32<T>(clamped_glu(g, u, limit, alpha));
  }
}

extern "C" int bh_experts_gate_up(const void* h, int dtype, const int32_t* chosen, const void* w_gu, void* inner, int n_rows, int top,
                                  int K, int ff, float limit, float alpha, hipStream_t stream) {
  BH_REQUIRE(n_rows > 0 && top > 0 && K > 0 && ff > 0, "experts_gate_up: sizes must be positive");
  BH_REQUIRE((size_t)K * sizeof(float) <= 64 * 1024, "experts_gate_up: rows of up to 16384 inputs, got %d", K);
  dim3 grid(n_rows * top, (ff + EX_OUTS - 1) / EX_OUTS);
  const size_t lds = (size_t)K * sizeof(float);
  if (dtype == BH_F32)
    experts_gate_up_kernel<float><<<grid, 64 * EX_WAVES, lds, stream>>>((const float*)h, chosen, (const float*)w_gu, (float*)inner, top, K, ff,
                                                                       limit, alpha);
  else if (dtype == BH_BF16)
    experts_gate_up_kernel<bf16_t><<<grid, 64 * EX_WAVES, lds, stream>>>((const bf16_t*)h, chosen, (const bf16_t*)w_gu, (bf16_t*)inner, top, K,
                                                                        ff, limit, alpha);
  else
    return bh_fail("experts_gate_up: unknown dtype %d", dtype);
  return bh_check_launch("experts_gate_up");
}

// grid (rows, ceil(D / EX_OUTS)); w_d [E][D][ff].  The chosen experts' shares of an output are added in their order.
template <typename T>
__global__ __launch_bounds__(256) void experts_down_kernel(const T* __restrict__ inner, const int32_t* __restrict__ chosen,
                                                           const float* __restrict__ weights, const T* __restrict__ w_d,
                                                           float* __restrict__ hidden, int top, int ff, int D) {
  extern __shared__ float xs[];      // [top][ff]
  const int row = blockIdx.x;
  for (int k = threadIdx.x; k < top * ff; k += blockDim.x) xs[k] = to_f32(inner[(size_t)row * top * ff + k]);
  __syncthreads();
  const int lane = threadIdx.x & (BH_WAVE - 1), wave = threadIdx.x / BH_WAVE;
  for (int i = wave; i < EX_OUTS; i += EX_WAVES) {
    const int o = blockIdx.y * EX_OUTS + i;
    if (o >= D) break;
    float total = 0.f;
    for (int j = 0; j < top; ++j) {
      const int e = chosen[(size_t)row * top + j];
      total = fmaf(weights[(size_t)row * top + j], wave_dot(w_d + ((size_t)e * D + o) * ff, xs + (size_t)j * ff, ff, lane), total);
    }
    if (lane == 0) hidden[(size_t)row * D + o] += total;
  }
}

extern "C" int bh_experts_down(const void* inner, int dtype, const int32_t* chosen, const float* weights, const void* w_d, float* hidden,
                               int n_rows, int top, int ff, int D, hipStream_t stream) {
  BH_REQUIRE(n_rows > 0 && top > 0 && ff > 0 && D > 0, "experts_down: sizes must be positive");
  const size_t lds = (size_t)top * ff * sizeof(float);
  BH_REQUIRE(lds <= 64 * 1024, "experts_down: %d experts a row of %d inner values do not fit the local memory", top, ff);
  dim3 grid(n_rows, (D + EX_OUTS - 1) / EX_OUTS);
  if (dtype == BH_F32)
    experts_down_kernel<float><<<grid, 64 * EX_WAVES, lds, stream>>>((const float*)inner, chosen, weights, (const float*)w_d, hidden, top, ff, D);
  else if (dtype == BH_BF16)
    experts_down_kernel<bf16_t><<<grid, 64 * EX_WAVES, lds, stream>>>((const bf16_t*)inner, chosen, weights, (const bf16_t*)w_d, hidden, top, ff,
                                                                     D);
  else
    return bh_fail("experts_down: unknown dtype %d", dtype);
  return bh_check_launch("experts_down");
}

template <typename T>
__global__ __launch_bounds__(256) void clamped_glu_kernel(const T* __restrict__ gu, T* __restrict__ out, int n_rows, int ff, float limit,
                                                          float alpha, int out_block_rows) {
  const size_t n = (size_t)n_rows * ff;
  for (size_t e = (size_t)blockIdx.x * blockDim.x + threadIdx.x; e < n; e += (size_t)gridDim.x * blockDim.x) {
    const int r = (int)(e / ff), i = (int)(e % ff);
    const float g = to_f32(gu[(size_t)r * 2 * ff + i]), u = to_f32(gu[(size_t)r * 2 * ff + ff + i]);
    out[bh_rows_index(out_block_rows, r, i, ff)] = from_f32<T>(clamped_glu(g, u, limit, alpha));
  }
}

extern "C" int bh_clamped_glu(const void* gu, int dtype, void* out, int n_rows, int ff, float limit, float alpha, int out_block_rows,
                              hipStream_t stream) {
  BH_REQUIRE(n_rows > 0 && ff > 0, "clamped_glu: sizes must be positive");
  BH_REQUIRE(out_block_rows == 0 || ((out_block_rows == 8 || out_block_rows == 16) && ff % 32 == 0 && dtype == BH_BF16),
             "clamped_glu: rows in blocks of %d of width %d are not written", out_block_rows, ff);
  const size_t n = (size_t)n_rows * ff;
  const int blocks = (int)((n + 255) / 256 < 8192 ? (n + 255) / 256 : 8192);
  if (dtype == BH_F32)
    clamped_glu_kernel<float><<<blocks, 256, 0, stream>>>((const float*)gu, (float*)out, n_rows, ff, limit, alpha, out_block_rows);
  else if (dtype == BH_BF16)
    clamped_glu_kernel<bf16_t><<<blocks, 256, 0, stream>>>((const bf16_t*)gu, (bf16_t*)out, n_rows, ff, limit, alpha, out_block_rows);
  else
    return bh_fail("clamped_glu: unknown dtype %d", dtype);
  return bh_check_launch("clamped_glu");
}
