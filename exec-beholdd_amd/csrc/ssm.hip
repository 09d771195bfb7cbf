// A selective state-space recurrence with a scalar decay per head (the "state-space duality" form), kept as a
// recurrent state, and the gated norm behind it:
//   ssm_scan            per (sequence, head): dt = softplus(dt_raw + dt_bias);  S <- exp(-exp(A_log) dt) S + dt B x^T;
//                       y = S^T C + D x.   S is [N][vdim] float32 and lives in the sequence's state region.
//   gated_group_rmsnorm out = rms_g(y * silu(z)) * w, the root mean square taken in `groups` equal parts of a row
// Everything but the reading of dt_raw and z is float32.
#include "common.h"

__device__ inline float softplus_f32(float x) { return x > 20.f ? x : log1pf(expf(x)); }

// One workgroup a (sequence, head): thread (p, s) owns column p of the state for the rows n of slice s; the state
// stays in LDS over the rows of the step, a thread touching only its own elements.  A row's B, C, x and dt go
// through LDS once; the slices' shares of y are added in slice order.
template <typename T>
__global__ __launch_bounds__(256) void ssm_scan_kernel(const float* __restrict__ xbc, int xbc_stride, const T* __restrict__ proj,
                                                       int proj_stride, int dt_first, const float* __restrict__ dt_bias,
                                                       const float* __restrict__ a_log, const float* __restrict__ d_skip,
                                                       float* __restrict__ state, long slot_stride,
                                                       const int32_t* __restrict__ seq_start, const int32_t* __restrict__ seq_slot,
                                                       float* __restrict__ y, int H, int vdim, int N, int G, int slices) {
  extern __shared__ float lds[];
  float* S = lds;                          // [N][vdim]
  float* bc = S + (size_t)N * vdim;        // B [N], C [N]
  float* xs = bc + 2 * N;                  // x [vdim]
  float* part = xs + vdim;                 // [slices][vdim]
  __shared__ float step[2];                // decay, dt
  const int seq = blockIdx.x, head = blockIdx.y, group = head / (H / G);
  const int inner = H * vdim;
  const int start = seq_start[seq], stop = seq_start[seq + 1];
  float* mine = state + (size_t)seq_slot[seq] * slot_stride + (size_t)head * N * vdim;
  for (int e = threadIdx.x; e < N * vdim; e += blockDim.x) S[e] = mine[e];
  const int p = threadIdx.x % vdim, s = threadIdx.x / vdim;
  const bool works = s < slices;
  const int per = (N + slices - 1) / slices;
  const int n0 = s * per, n1 = (n0 + per < N) ? n0 + per : N;
  const float rate = expf(a_log[head]), skip = d_skip[head], bias = dt_bias[head];
  __syncthreads();
  for (int row = start; row < stop; ++row) {
    const float* in = xbc + (size_t)row * xbc_stride;
    for (int e = threadIdx.x; e < 2 * N; e += blockDim.x)
      bc[e] = in[inner + (e < N ? 0 : G * N) + group * N + (e < N ? e : e - N)];
    for (int e = threadIdx.x; e < vdim; e += blockDim.x) xs[e] = in[head * vdim + e];
    if (threadIdx.x == 0) {
      const float dt = softplus_f32(to_f32(proj[(size_t)row * proj_stride + dt_first + head]) + bias);
      step[0] = expf(-rate * dt);
      step[1] = dt;
    }
    __syncthreads();
    if (works) {
      const float decay = step[0], dtx = step[1] * xs[p];
      float acc = 0.f;
      for (int n = n0; n < n1; ++n) {
        const float v = fmaf(decay, S[n * vdim + p], bc[n] * dtx);
        S[n * vdim + p] = v;
        acc = fmaf(v, bc[N + n], acc);
      }
      part[s * vdim + p] = acc;
    }
    __syncthreads();
    if (threadIdx.x < vdim) {
      float total = skip * xs[threadIdx.x];
      for (int k = 0; k < slices; ++k) total += part[k * vdim + threadIdx.x];
      y[(size_t)row * inner + head * vdim + threadIdx.x] = total;
    }
    __syncthreads();
  }
  for (int e = threadIdx.x; e < N * vdim; e += blockDim.x) mine[e] = S[e];
}

extern "C" int bh_ssm_scan(const float* xbc, int xbc_stride, const void* proj, int dtype, int proj_stride, int dt_first,
                           const float* dt_bias, const float* a_log, const float* d_skip, float* state, long slot_stride,
                           const int32_t* seq_start, const int32_t* seq_slot, float* y, int n_seqs, int H, int vdim, int N, int G,
                           hipStream_t stream) {
  BH_REQUIRE(n_seqs > 0 && H > 0 && vdim > 0 && N > 0 && G > 0, "ssm_scan: sizes must be positive");
  BH_REQUIRE(H % G == 0, "ssm_scan: %d heads do not fall into %d groups evenly", H, G);
  BH_REQUIRE(vdim <= 256, "ssm_scan: heads of up to 256 values, got %d", vdim);
  BH_REQUIRE(xbc_stride >= H * vdim + 2 * G * N, "ssm_scan: a row of %d does not hold x, B and C", xbc_stride);
  BH_REQUIRE(dt_first >= 0 && dt_first + H <= proj_stride, "ssm_scan: the step sizes lie outside their row");
  int slices = 256 / vdim;
  if (slices > N) slices = N;
  const size_t lds_bytes = ((size_t)N * vdim + 2 * N + vdim + (size_t)slices * vdim) * sizeof(float);
  BH_REQUIRE(lds_bytes <= 160 * 1024 - 64, "ssm_scan: a state of %d x %d does not fit the local memory", N, vdim);
  dim3 grid(n_seqs, H);
  if (dtype == BH_F32) {
    if (lds_bytes > 48 * 1024)
      (void)hipFuncSetAttribute((const void*)ssm_scan_kernel<float>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_bytes);
    ssm_scan_kernel<float><<<grid, 256, lds_bytes, stream>>>(xbc, xbc_stride, (const float*)proj, proj_stride, dt_first, dt_bias, a_log,
                                                             d_skip, state, slot_stride, seq_start, seq_slot, y, H, vdim, N, G, slices);
  } else if (dtype == BH_BF16) {
    if (lds_bytes > 48 * 1024)
      (void)hipFuncSetAttribute((const void*)ssm_scan_kernel<bf16_t>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_bytes);
    ssm_scan_kernel<bf16_t><<<grid, 256, lds_bytes, stream>>>(xbc, xbc_stride, (const bf16_t*)proj, proj_stride, dt_first, dt_bias,
                                                              a_log, d_skip, state, slot_stride, seq_start, seq_slot, y, H, vdim, N, G,
                                                              slices);
  } else {
    return bh_fail("ssm_scan: unknown dtype %d", dtype);
  }
  return bh_check_launch("ssm_scan");
}

// One workgroup a (row, group).
template <typename T>
__global__ __launch_bounds__(256) void gated_group_rmsnorm_kernel(const float* __restrict__ y, const T* __restrict__ z, int z_stride,
                                                                  int z_first, const float* __restrict__ w, float eps,
                                                                  T* __restrict__ out, int width, int groups, int out_block_rows) {
  __shared__ float scratch[8];
  const int row = blockIdx.x, per = width / groups, c0 = blockIdx.y * per;
  const float* src = y + (size_t)row * width + c0;
  const T* gate = z + (size_t)row * z_stride + z_first + c0;
  float ss = 0.f;
  for (int i = threadIdx.x; i < per; i += blockDim.x) {
    const float g = to_f32(gate[i]);
    const float v = src[i] * (g / (1.0f + expf(-g)));
    ss += v * v;
  }
  const float inv = 1.0f / sqrtf(block_sum(ss, scratch) / (float)per + eps);
  for (int i = threadIdx.x; i < per; i += blockDim.x) {
    const float g = to_f32(gate[i]);
    const float v = src[i] * (g / (1.0f + expf(-g)));
    out[bh_rows_index(out_block_rows, row, c0 + i, width)] = from_f32<T>(v * inv * w[c0 + i]);
  }
}

extern "C" int bh_gated_group_rmsnorm(const float* y, const void* z, int dtype, int z_stride, int z_first, const float* w, float eps,
                                      void* out, int n_rows, int width, int groups, int out_block_rows, hipStream_t stream) {
  BH_REQUIRE(n_rows > 0 && width > 0 && groups > 0 && width % groups == 0, "gated_group_rmsnorm: %d columns in %d equal parts", width,
             groups);
  BH_REQUIRE(z_first >= 0 && z_first + width <= z_stride, "gated_group_rmsnorm: the gate lies outside its row");
  BH_REQUIRE(out_block_rows == 0 || ((out_block_rows == 8 || out_block_rows == 16) && width % 32 == 0 && dtype == BH_BF16),
             "gated_group_rmsnorm: rows in blocks of %d of width %d are not written", out_block_rows, width);
  dim3 grid(n_rows, groups);
  if (dtype == BH_F32)
    gated_group_rmsnorm_kernel<float><<<grid, 256, 0, stream>>>(y, (const float*)z, z_stride, z_first, w, eps, (float*)out, width, groups,
                                                                out_block_rows);
  else if (dtype == BH_BF16)
    gated_group_rmsnorm_kernel<bf16_t><<<grid, 256, 0, stream>>>(y, (const bf16_t*)z, z_stride, z_first, w, eps, (bf16_t*)out, width,
                                                                 groups, out_block_rows);
  else
    return bh_fail("gated_group_rmsnorm: unknown dtype %d", dtype);
  return bh_check_launch("gated_group_rmsnorm");
}
