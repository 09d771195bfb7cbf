// Several residual streams side by side, and the small elementwise steps of layers that keep their sublayer's
// result apart from the residual: the residual of a row is x[S][D] (S streams of width D, float32); a sublayer reads
// one weighted sum of the streams through an RMSNorm and its result y[D] goes back into every stream,
//   x_t <- sum_s mix[s][t] x_s + give[t] * scale[i] * y[i]        (all streams at once, from the old ones).
// With S = 1, mix = give = 1 this is a plain residual with a per-channel scale on the sublayer's result.
// Everything here is float32 arithmetic; only a norm's output takes the activation type.
#include "common.h"

#define BH_STREAMS_MOST 16

// ---- open: every stream starts as the same row -------------------------------------------------------------
__global__ void streams_open_kernel(const float* __restrict__ src, float* __restrict__ dst, int width, int streams) {
  const int row = blockIdx.x;
  const float* from = src + (size_t)row * width;
  float* to = dst + (size_t)row * streams * width;
  for (int i = threadIdx.x; i < width; i += blockDim.x) {
    const float v = from[i];
    for (int s = 0; s < streams; ++s) to[(size_t)s * width + i] = v;
  }
}

extern "C" int bh_streams_open(const float* src, float* dst, int n_rows, int width, int streams, hipStream_t stream) {
  BH_REQUIRE(n_rows > 0 && width > 0 && streams > 0, "streams_open: rows %d, width %d and streams %d must be positive",
             n_rows, width, streams);
  streams_open_kernel<<<dim3(n_rows), dim3(256), 0, stream>>>(src, dst, width, streams);
  return bh_check_launch("streams_open");
}

// ---- read: RMSNorm of a weighted sum of the streams --------------------------------------------------------
// out[r, i] = u[i] / sqrt(mean(u^2) + eps) * w[i],  u = sum_s take[s] * x[src, s, :]  (take == null: every stream once),
// src = rows ? rows[r] : r.  PER > 0: the row fits PER elements a thread and u stays in registers; PER == 0: u is
// formed twice.
template <typename TO, int PER>
__global__ void streams_rmsnorm_kernel(const float* __restrict__ x, const int32_t* __restrict__ rows,
                                       const float* __restrict__ take, const float* __restrict__ w, TO* __restrict__ out,
                                       int width, int streams, float eps, int block_rows) {
  __shared__ float scratch[16];
  __shared__ float share[BH_STREAMS_MOST];
  const int r = blockIdx.x;
  const int src = rows ? rows[r] : r;
  const float* xr = x + (size_t)src * streams * width;
  if (threadIdx.x < streams) share[threadIdx.x] = take ? take[threadIdx.x] : 1.f;
  __syncthreads();
  auto mixed = [&](int i) {
    float u = 0.f;
    for (int s = 0; s < streams; ++s) u = fmaf(share[s], xr[(size_t)s * width + i], u);
    return u;
  };
  auto at = [&](int i) { return out + bh_rows_index(block_rows, r, i, width); };
  float ss = 0.f;
  if (PER > 0) {
    float uv[PER > 0 ? PER : 1];
#pragma unroll
    for (int j = 0; j < PER; ++j) {
      const int i = threadIdx.x + j * blockDim.x;
      uv[j] = i < width ? mixed(i) : 0.f;
      ss += uv[j] * uv[j];
    }
    ss = block_sum(ss, scratch);
    const float inv = 1.0f / sqrtf(ss / (float)width + eps);
#pragma unroll
    for (int j = 0; j < PER; ++j) {
      const int i = threadIdx.x + j * blockDim.x;
      if (i < width) *at(i) = from_f32<TO>(uv[j] * inv * (w ? w[i] : 1.f));
    }
    return;
  }
  for (int i = threadIdx.x; i < width; i += blockDim.x) {
    const float u = mixed(i);
    ss += u * u;
  }
  ss = block_sum(ss, scratch);
  const float inv = 1.0f / sqrtf(ss / (float)width + eps);
  for (int i = threadIdx.x; i < width; i += blockDim.x) *at(i) = from_f32<TO>(mixed(i) * inv * (w ? w[i] : 1.f));
}

template <typename TO>
static void launch_streams_rmsnorm(const float* x, const int32_t* rows, const float* take, const float* w, void* out,
                                   int n_rows, int width, int streams, float eps, int block_rows, hipStream_t stream) {
  const int threads = width >= 4096 ? 1024 : (width >= 1024 ? 512 : 256);
  const int per = (width + threads - 1) / threads;
  dim3 grid(n_rows), block(threads);
#define BH_SNORM(PER) \
  streams_rmsnorm_kernel<TO, PER><<<grid, block, 0, stream>>>(x, rows, take, w, (TO*)out, width, streams, eps, block_rows)
  if (per <= 4) BH_SNORM(4);
  else if (per <= 8) BH_SNORM(8);
  else BH_SNORM(0);
#undef BH_SNORM
}

extern "C" int bh_streams_rmsnorm(const float* x, const int32_t* rows, const float* take, const float* w, void* out,
                                  int out_dtype, int n_rows, int width, int streams, float eps, int out_block_rows,
                                  hipStream_t stream) {
  BH_REQUIRE(n_rows > 0 && width > 0, "streams_rmsnorm: rows %d and width %d must be positive", n_rows, width);
  BH_REQUIRE(streams >= 1 && streams <= BH_STREAMS_MOST, "streams_rmsnorm: 1 to %d streams, not %d", BH_STREAMS_MOST, streams);
  BH_REQUIRE(eps >= 0.f, "streams_rmsnorm: eps must not be negative");
  BH_REQUIRE(out_block_rows == 0 || ((out_block_rows == 8 || out_block_rows == 16) && out_dtype == BH_BF16 && width % 32 == 0),
             "streams_rmsnorm: rows in blocks of %d need bfloat16 and a width that is a multiple of 32 (got %d)",
             out_block_rows, width);
  if (out_dtype == BH_F32) launch_streams_rmsnorm<float>(x, rows, take, w, out, n_rows, width, streams, eps, out_block_rows, stream);
  else if (out_dtype == BH_BF16) launch_streams_rmsnorm<bf16_t>(x, rows, take, w, out, n_rows, width, streams, eps, out_block_rows, stream);
  else return bh_fail("streams_rmsnorm: unknown output dtype %d", out_dtype);
  return bh_check_launch("streams_rmsnorm");
}

// ---- write: a sublayer's result goes back into every stream ------------------------------------------------
__global__ __launch_bounds__(256) void streams_update_kernel(float* __restrict__ x, const float* __restrict__ y,
                                                             const float* __restrict__ mix, const float* __restrict__ give,
                                                             const float* __restrict__ scale, int width, int streams,
                                                             size_t total) {
  __shared__ float m[BH_STREAMS_MOST * BH_STREAMS_MOST];
  __shared__ float g[BH_STREAMS_MOST];
  for (int e = threadIdx.x; e < streams * streams; e += blockDim.x) m[e] = mix ? mix[e] : (e / streams == e % streams ? 1.f : 0.f);
  if (threadIdx.x < streams) g[threadIdx.x] = give ? give[threadIdx.x] : 1.f;
  __syncthreads();
  const size_t at = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (at >= total) return;
  const size_t row = at / width;
  const int i = (int)(at % width);
  float* xr = x + row * streams * width + i;
  float old[BH_STREAMS_MOST];
  for (int s = 0; s < streams; ++s) old[s] = xr[(size_t)s * width];
  const float add = (scale ? scale[i] : 1.f) * y[at];
  for (int t = 0; t < streams; ++t) {
    float v = 0.f;
    for (int s = 0; s < streams; ++s) v = fmaf(m[s * streams + t], old[s], v);
    xr[(size_t)t * width] = fmaf(g[t], add, v);
  }
}

extern "C" int bh_streams_update(float* x, const float* y, const float* mix, const float* give, const float* scale,
                                 int n_rows, int width, int streams, hipStream_t stream) {
  BH_REQUIRE(n_rows > 0 && width > 0, "streams_update: rows %d and width %d must be positive", n_rows, width);
  BH_REQUIRE(streams >= 1 && streams <= BH_STREAMS_MOST, "streams_update: 1 to %d streams, not %d", BH_STREAMS_MOST, streams);
  const size_t total = (size_t)n_rows * width;
  const size_t blocks = (total + 255) / 256;
  BH_REQUIRE(blocks <= 2147483647u, "streams_update: too many elements");
  streams_update_kernel<<<dim3((unsigned)blocks), dim3(256), 0, stream>>>(x, y, mix, give, scale, width, streams, total);
  return bh_check_launch("streams_update");
}

// ---- write, and read for the sublayer that follows, in one pass ---------------------------------------------------
// streams_update for one row, then streams_rmsnorm of the row as it has become (with the next sublayer's `take` and
// norm weight): a workgroup per row; a thread keeps the next sublayer's sum of its elements while it writes the streams.
template <typename TO, int PER>
__global__ void streams_update_rmsnorm_kernel(float* __restrict__ x, const float* __restrict__ y, const float* __restrict__ mix,
                                              const float* __restrict__ give, const float* __restrict__ scale,
                                              const float* __restrict__ take, const float* __restrict__ w, TO* __restrict__ out,
                                              int width, int streams, float eps, int block_rows) {
  __shared__ float scratch[16];
  __shared__ float m[BH_STREAMS_MOST * BH_STREAMS_MOST];
  __shared__ float g[BH_STREAMS_MOST], share[BH_STREAMS_MOST];
  const int r = blockIdx.x;
  for (int e = threadIdx.x; e < streams * streams; e += blockDim.x) m[e] = mix ? mix[e] : (e / streams == e % streams ? 1.f : 0.f);
  if (threadIdx.x < streams) {
    g[threadIdx.x] = give ? give[threadIdx.x] : 1.f;
    share[threadIdx.x] = take ? take[threadIdx.x] : 1.f;
  }
  __syncthreads();
  float* xr = x + (size_t)r * streams * width;
  const float* yr = y + (size_t)r * width;
  auto renew = [&](int i) {      // the streams' element i as it becomes, written; returns the next sublayer's sum of it
    float old[BH_STREAMS_MOST];
    for (int s = 0; s < streams; ++s) old[s] = xr[(size_t)s * width + i];
    const float add = (scale ? scale[i] : 1.f) * yr[i];
    float u = 0.f;
    for (int t = 0; t < streams; ++t) {
      float v = 0.f;
      for (int s = 0; s < streams; ++s) v = fmaf(m[s * streams + t], old[s], v);
      v = fmaf(g[t], add, v);
      xr[(size_t)t * width + i] = v;
      u = fmaf(share[t], v, u);
    }
    return u;
  };
  auto at = [&](int i) { return out + bh_rows_index(block_rows, r, i, width); };
  float ss = 0.f;
  if (PER > 0) {
    float uv[PER > 0 ? PER : 1];
#pragma unroll
    for (int j = 0; j < PER; ++j) {
      const int i = threadIdx.x + j * blockDim.x;
      uv[j] = i < width ? renew(i) : 0.f;
      ss += uv[j] * uv[j];
    }
    ss = block_sum(ss, scratch);
    const float inv = 1.0f / sqrtf(ss / (float)width + eps);
#pragma unroll
    for (int j = 0; j < PER; ++j) {
      const int i = threadIdx.x + j * blockDim.x;
      if (i < width) *at(i) = from_f32<TO>(uv[j] * inv * (w ? w[i] : 1.f));
    }
    return;
  }
  for (int i = threadIdx.x; i < width; i += blockDim.x) {
    const float u = renew(i);
    ss += u * u;
  }
  ss = block_sum(ss, scratch);
  const float inv = 1.0f / sqrtf(ss / (float)width + eps);
  for (int i = threadIdx.x; i < width; i += blockDim.x) {      // a thread reads back what it wrote itself
    float u = 0.f;
    for (int t = 0; t < streams; ++t) u = fmaf(share[t], xr[(size_t)t * width + i], u);
    *at(i) = from_f32<TO>(u * inv * (w ? w[i] : 1.f));
  }
}

extern "C" int bh_streams_update_rmsnorm(float* x, const float* y, const float* mix, const float* give, const float* scale,
                                         const float* take, const float* w, void* out, int out_dtype, int n_rows, int width,
                                         int streams, float eps, int out_block_rows, hipStream_t stream) {
  BH_REQUIRE(n_rows > 0 && width > 0, "streams_update_rmsnorm: rows %d and width %d must be positive", n_rows, width);
  BH_REQUIRE(streams >= 1 && streams <= BH_STREAMS_MOST, "streams_update_rmsnorm: 1 to %d streams, not %d", BH_STREAMS_MOST, streams);
  BH_REQUIRE(eps >= 0.f, "streams_update_rmsnorm: eps must not be negative");
  BH_REQUIRE(out_block_rows == 0 || ((out_block_rows == 8 || out_block_rows == 16) && out_dtype == BH_BF16 && width % 32 == 0),
             "streams_update_rmsnorm: rows in blocks of %d need bfloat16 and a width that is a multiple of 32 (got %d)",
             out_block_rows, width);
  const int threads = width >= 4096 ? 1024 : (width >= 1024 ? 512 : 256);
  const int per = (width + threads - 1) / threads;
  dim3 grid(n_rows), block(threads);
#define BH_SUN(TO, PER)                                                                                                  \
  streams_update_rmsnorm_kernel<TO, PER><<<grid, block, 0, stream>>>(x, y, mix, give, scale, take, w, (TO*)out, width, streams, \
                                                                     eps, out_block_rows)
#define BH_SUN_SIZES(TO)           \
  do {                             \
    if (per <= 4) BH_SUN(TO, 4);   \
    else if (per <= 8) BH_SUN(TO, 8); \
    else BH_SUN(TO, 0);            \
  } while (0)
  if (out_dtype == BH_F32) BH_SUN_SIZES(float);
  else if (out_dtype == BH_BF16) BH_SUN_SIZES(bf16_t);
  else return bh_fail("streams_update_rmsnorm: unknown output dtype %d", out_dtype);
#undef BH_SUN_SIZES
#undef BH_SUN
  return bh_check_launch("streams_update_rmsnorm");
}

// ---- small elementwise steps ---------------------------------------------------------------------------------
__global__ void scale_kernel(float* __restrict__ x, float factor, size_t total) {
  const size_t at = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (at < total) x[at] *= factor;
}

extern "C" int bh_scale(float* x, long total, float factor, hipStream_t stream) {
  BH_REQUIRE(total > 0, "scale: nothing to scale");
  const size_t blocks = ((size_t)total + 255) / 256;
  BH_REQUIRE(blocks <= 2147483647u, "scale: too many elements");
  scale_kernel<<<dim3((unsigned)blocks), dim3(256), 0, stream>>>(x, factor, (size_t)total);
  return bh_check_launch("scale");
}

// out <- max(x, 0)^2 (out may be x itself), in float32 whatever the element type; the output's rows one after the other
// or in blocks of rows (bh_rows_index)
template <typename T>
__global__ void relu_squared_kernel(const T* __restrict__ x, T* __restrict__ out, int width, size_t total, int block_rows) {
  const size_t at = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (at >= total) return;
  const float v = fmaxf(to_f32(x[at]), 0.f);
  const size_t to = block_rows ? (size_t)bh_rows_index(block_rows, (int)(at / width), (int)(at % width), width) : at;
  out[to] = from_f32<T>(v * v);
}

extern "C" int bh_relu_squared(const void* x, void* out, int dtype, int n_rows, int width, int out_block_rows, hipStream_t stream) {
  BH_REQUIRE(n_rows > 0 && width > 0, "relu_squared: nothing to do");
  BH_REQUIRE(out_block_rows == 0 || ((out_block_rows == 8 || out_block_rows == 16) && dtype == BH_BF16 && width % 32 == 0 && x != out),
             "relu_squared: rows in blocks of %d need bfloat16, a width that is a multiple of 32 (got %d) and an output of their own",
             out_block_rows, width);
  const size_t total = (size_t)n_rows * width;
  const size_t blocks = (total + 255) / 256;
  BH_REQUIRE(blocks <= 2147483647u, "relu_squared: too many elements");
  if (dtype == BH_F32)
    relu_squared_kernel<float><<<dim3((unsigned)blocks), dim3(256), 0, stream>>>((const float*)x, (float*)out, width, total, out_block_rows);
  else if (dtype == BH_BF16)
    relu_squared_kernel<bf16_t><<<dim3((unsigned)blocks), dim3(256), 0, stream>>>((const bf16_t*)x, (bf16_t*)out, width, total, out_block_rows);
  else return bh_fail("relu_squared: unknown dtype %d", dtype);
  return bh_check_launch("relu_squared");
}
