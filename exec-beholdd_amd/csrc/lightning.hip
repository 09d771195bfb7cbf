// Linear attention with a per-head decay ("lightning attention") as a recurrence over a float32 state:
//   S_t = decay_h * S_(t-1) + k_t v_t^T        S [dim][vdim] per (sequence, head), kept between steps
//   o_t = S_t^T q_t
// with q, k, v = silu of the rows of one fused projection.  The state, the decay and both products are float32
// (plain FMA) whatever type the projection rows have.  A workgroup owns a tile of up to 64 value columns of one
// (sequence, head) and walks that sequence's rows of the step in order; a thread owns a slice of `dim` of one
// column, so the state lives in registers from the first row to the last and memory sees it once each way.
// A stage of LN_TOKENS rows goes through LDS at a time (q and k are read by all lanes of a wave at the same
// address, v by each lane at its own), the partial sums of the slices of `dim` are added up through LDS in a
// fixed order.  Steps of one row a sequence (decoding) are the same kernel: one stage of one row.
#include "common.h"

#define LN_TOKENS 16

__device__ inline float silu_f32(float x) { return x / (1.0f + expf(-x)); }

// DPT: elements of `dim` a thread owns; VT: value columns a workgroup owns (lanes j = tid % VT); blockDim = VT * parts.
template <typename T, int DPT, int VT>
__global__ void lightning_scan_kernel(const T* __restrict__ proj, int row_stride, int q_off, int k_off, int v_off,
                                      float* __restrict__ state, const float* __restrict__ decay,
                                      const int32_t* __restrict__ seq_start, const int32_t* __restrict__ seq_slot,
                                      float* __restrict__ out, int H, int dim, int vdim, int parts) {
  extern __shared__ float lds[];
  const int seq = blockIdx.x, head = blockIdx.y, tile = blockIdx.z;
  const int j = threadIdx.x % VT, part = threadIdx.x / VT;
  const int column = tile * VT + j;
  const int padded = parts * DPT;                 // dim rounded up to whole slices; the padding holds zeros
  float* qs = lds;                                // [LN_TOKENS][padded]
  float* ks = qs + LN_TOKENS * padded;            // [LN_TOKENS][padded]
  float* vs = ks + LN_TOKENS * padded;            // [LN_TOKENS][VT]
  float* sums = vs + LN_TOKENS * VT;              // [LN_TOKENS][parts][VT]
  const int lo = seq_start[seq], hi = seq_start[seq + 1];
  const int slot = seq_slot[seq];
  const float lambda = decay[head];
  float* mine = state + (((size_t)slot * H + head) * dim) * vdim;
  const bool live = column < vdim;
  float s[DPT];
#pragma unroll
  for (int e = 0; e < DPT; ++e) {
    const int i = part * DPT + e;
    s[e] = (live && i < dim) ? mine[(size_t)i * vdim + column] : 0.f;
  }
  for (int r0 = lo; r0 < hi; r0 += LN_TOKENS) {
    const int n = hi - r0 < LN_TOKENS ? hi - r0 : LN_TOKENS;
    __syncthreads();      // the stage before has been read
    for (int e = threadIdx.x; e < n * padded; e += blockDim.x) {
      const int t = e / padded, i = e % padded;
      const T* row = proj + (size_t)(r0 + t) * row_stride + (size_t)head * dim + i;
      qs[e] = i < dim ? silu_f32(to_f32(row[q_off])) : 0.f;
      ks[e] = i < dim ? silu_f32(to_f32(row[k_off])) : 0.f;
    }
    for (int e = threadIdx.x; e < n * VT; e += blockDim.x) {
      const int t = e / VT, c = tile * VT + e % VT;
      vs[e] = c < vdim ? silu_f32(to_f32(proj[(size_t)(r0 + t) * row_stride + v_off + (size_t)head * vdim + c])) : 0.f;
    }
    __syncthreads();
    for (int t = 0; t < n; ++t) {
      const float v = vs[t * VT + j];
      const float* kt = ks + t * padded + part * DPT;
      const float* qt = qs + t * padded + part * DPT;
      float acc = 0.f;
#pragma unroll
      for (int e = 0; e < DPT; ++e) {
        s[e] = fmaf(lambda, s[e], kt[e] * v);
        acc = fmaf(s[e], qt[e], acc);
      }
      sums[(t * parts + part) * VT + j] = acc;
    }
    __syncthreads();
    for (int e = threadIdx.x; e < n * VT; e += blockDim.x) {
      const int t = e / VT, c = tile * VT + e % VT;
      if (c >= vdim) continue;
      float total = 0.f;
      for (int p = 0; p < parts; ++p) total += sums[(t * parts + p) * VT + e % VT];
      out[((size_t)(r0 + t) * H + head) * vdim + c] = total;
    }
  }
  if (live) {
#pragma unroll
    for (int e = 0; e < DPT; ++e) {
      const int i = part * DPT + e;
      if (i < dim) mine[(size_t)i * vdim + column] = s[e];
    }
  }
}

template <typename T, int DPT>
static int launch_lightning(const void* proj, int row_stride, int q_off, int k_off, int v_off, float* state,
                            const float* decay, const int32_t* seq_start, const int32_t* seq_slot, float* out, int n_seqs,
                            int H, int dim, int vdim, hipStream_t stream) {
  const int parts = (dim + DPT - 1) / DPT;
  const int vt = vdim > 32 ? 64 : (vdim > 16 ? 32 : 16);
  BH_REQUIRE(parts * vt <= 1024, "lightning: heads of %d x %d need more than 1024 threads", dim, vdim);
  const int tiles = (vdim + vt - 1) / vt;
  const size_t smem = (size_t)LN_TOKENS * (2 * parts * DPT + vt + parts * vt) * sizeof(float);
  BH_REQUIRE(smem <= 64 * 1024, "lightning: heads of %d x %d need %zu bytes of LDS", dim, vdim, smem);
  dim3 grid(n_seqs, H, tiles), block(parts * vt);
#define BH_SCAN(VT)                                                                                               \
  lightning_scan_kernel<T, DPT, VT><<<grid, block, smem, stream>>>((const T*)proj, row_stride, q_off, k_off, v_off, \
                                                                   state, decay, seq_start, seq_slot, out, H, dim, vdim, parts)
  if (vt == 64) BH_SCAN(64);
  else if (vt == 32) BH_SCAN(32);
  else BH_SCAN(16);
#undef BH_SCAN
  return bh_check_launch("lightning_scan");
}

// proj [n_rows][row_stride]: a row holds q (H x dim) from q_off, k (H x dim) from k_off, v (H x vdim) from v_off, all
// before their silu.  state [slots][H][dim][vdim] float32; rows seq_start[b] .. seq_start[b + 1] - 1 belong to the
// sequence in slot seq_slot[b], in order.  out [n_rows][H * vdim] float32.
extern "C" int bh_lightning_scan(const void* proj, int dtype, int row_stride, int q_off, int k_off, int v_off, float* state,
                                 const float* decay, const int32_t* seq_start, const int32_t* seq_slot, float* out,
                                 int n_seqs, int H, int dim, int vdim, hipStream_t stream) {
  BH_REQUIRE(n_seqs > 0 && H > 0 && dim > 0 && vdim > 0, "lightning: sizes must be positive");
  BH_REQUIRE(H <= 65535 && n_seqs <= 2147483647, "lightning: too many heads");
  BH_REQUIRE(dim <= 1024, "lightning: a key size of %d is above the limit of 1024", dim);
  BH_REQUIRE(q_off >= 0 && k_off >= 0 && v_off >= 0 && q_off + H * dim <= row_stride && k_off + H * dim <= row_stride &&
                 v_off + H * vdim <= row_stride,
             "lightning: q, k and v do not lie inside a row of %d", row_stride);
  const int quarter = (dim + 3) / 4;     // four slices of dim a column where that keeps a slice short
#define BH_LN(T, DPT) \
  return launch_lightning<T, DPT>(proj, row_stride, q_off, k_off, v_off, state, decay, seq_start, seq_slot, out, n_seqs, H, dim, vdim, stream)
#define BH_LN_SIZES(T)              \
  if (quarter <= 4) BH_LN(T, 4);    \
  if (quarter <= 8) BH_LN(T, 8);    \
  if (quarter <= 16) BH_LN(T, 16);  \
  if (quarter <= 32) BH_LN(T, 32);  \
  BH_LN(T, 64)
  if (dtype == BH_F32) { BH_LN_SIZES(float); }
  if (dtype == BH_BF16) { BH_LN_SIZES(bf16_t); }
#undef BH_LN_SIZES
#undef BH_LN
  return bh_fail("lightning: unknown dtype %d", dtype);
}

// ---- the recurrence's output, normed over all heads together and gated -------------------------------------
// out[r, i] = o[r, i] / sqrt(mean_i(o[r]^2) + eps) * w[i] * sigmoid(gate[r, i]); o float32 [n][width], gate from the
// fused projection's rows (before its sigmoid), out in the activation type (rows, or blocks of rows).
template <typename T>
__global__ void gated_rmsnorm_kernel(const float* __restrict__ o, const T* __restrict__ gate, int gate_stride,
                                     const float* __restrict__ w, T* __restrict__ out, int width, float eps, int block_rows) {
  __shared__ float scratch[16];
  const int r = blockIdx.x;
  const float* row = o + (size_t)r * width;
  const T* g = gate + (size_t)r * gate_stride;
  float ss = 0.f;
  for (int i = threadIdx.x; i < width; i += blockDim.x) ss += row[i] * row[i];
  ss = block_sum(ss, scratch);
  const float inv = 1.0f / sqrtf(ss / (float)width + eps);
  for (int i = threadIdx.x; i < width; i += blockDim.x) {
    const float opened = 1.0f / (1.0f + expf(-to_f32(g[i])));
    out[bh_rows_index(block_rows, r, i, width)] = from_f32<T>(row[i] * inv * (w ? w[i] : 1.f) * opened);
  }
}

extern "C" int bh_gated_rmsnorm(const float* o, const void* gate, int dtype, int gate_stride, const float* w, void* out,
                                int n_rows, int width, float eps, int out_block_rows, hipStream_t stream) {
  BH_REQUIRE(n_rows > 0 && width > 0 && gate_stride >= width, "gated_rmsnorm: rows %d, width %d, gate stride %d", n_rows,
             width, gate_stride);
  BH_REQUIRE(out_block_rows == 0 || ((out_block_rows == 8 || out_block_rows == 16) && dtype == BH_BF16 && width % 32 == 0),
             "gated_rmsnorm: rows in blocks of %d need bfloat16 and a width that is a multiple of 32 (got %d)", out_block_rows, width);
  const int threads = width >= 2048 ? 1024 : (width >= 512 ? 512 : 256);
  if (dtype == BH_F32)
    gated_rmsnorm_kernel<float><<<dim3(n_rows), dim3(threads), 0, stream>>>(o, (const float*)gate, gate_stride, w, (float*)out, width, eps, out_block_rows);
  else if (dtype == BH_BF16)
    gated_rmsnorm_kernel<bf16_t><<<dim3(n_rows), dim3(threads), 0, stream>>>(o, (const bf16_t*)gate, gate_stride, w, (bf16_t*)out, width, eps, out_block_rows);
  else
    return bh_fail("gated_rmsnorm: unknown dtype %d", dtype);
  return bh_check_launch("gated_rmsnorm");
}
