// Linear attention with a per-head decay ("lightning attention") as a recurrence over a float32 state:
//   S_t = decay_h * S_(t-1) + k_t v_t^T        S [dim][vdim] per (sequence, head), kept between steps
//   o_t = S_t^T q_t
// with q, k, v = silu of the rows of one fused projection.  The state, the decay and both products are float32
// (plain FMA) whatever type the projection rows have.  A workgroup owns a tile of VT value columns of one
// (sequence, head) and walks that sequence's rows of the step in order; a thread owns a slice of `dim` of one
// column, so the state lives in registers from the first row to the last and memory sees it once each way.
// The tile is as narrow as it takes to give every compute unit a workgroup (a prompt of one sequence has only
// heads x vdim / VT of them), the slices as short as it takes to make the workgroup four waves.
// A stage of LN_TOKENS rows goes through LDS at a time (q and k are read by all lanes of a slice at the same
// address, v by each lane at its own) while the next stage's rows are already on their way into registers; the
// partial sums of the slices of `dim` are added up through LDS in a fixed order.
// Within a stage that starts from the state S, row t (0-based) has S_t = decay^(t+1) (S + sum_(j<=t) decay^-(j+1) k_j v_j^T):
// with k'_j = decay^-(j+1) k_j and q'_t = decay^(t+1) q_t the inner loop is S' += k'_t v_t^T, o_t = S'^T q'_t, two
// FMAs an element instead of three, and S' is scaled by decay^n once when the stage ends.  decay^-16 must stay a
// modest number for that: heads that forget faster than 0.5 a row take the recurrence as written.
// A long sequence that would leave compute units idle is cut into chunks of rows that are walked at the same time
// (bh_lightning_chunks): every chunk but a sequence's first starts from a zero state and leaves its own end state in
// scratch memory; lightning_combine_kernel then goes through a sequence's chunks in order, E_c = decay^rows_c E_(c-1) + Z_c,
// leaves every chunk the state it should have started from and the cache the last one; and lightning_carry_kernel adds
// what that state owes each row, decay^(t+1) E_(c-1)^T q_t (t counted from the chunk's first row), a small matrix product
// per chunk and head.  All of it float32 FMA; the sums are the recurrence's, in another order.
// Steps of one row a sequence (decoding) have a lean kernel of their own.
#include "common.h"

#define LN_TOKENS 16
#define LN_SCALED_FROM 0.5f

// x / (1 + exp(-x)) with the hardware's reciprocal (one ulp) in place of a division of a dozen instructions
__device__ inline float silu_f32(float x) { return x * __builtin_amdgcn_rcpf(1.0f + expf(-x)); }

// DPT: elements of `dim` a thread owns; VT: value columns a workgroup owns (lanes j = tid % VT); blockDim = VT * parts.
// (Workgroups have at most 256 threads unless a slice of 64 is not enough for `dim`: saying so gives the state, the
// prefetched stage and its places the registers they need; with the default bound of 1,024 threads they went to scratch.)
template <typename T, int DPT, int VT>
__global__ __launch_bounds__(DPT == 64 ? 1024 : 256) void lightning_scan_kernel(const T* __restrict__ proj, int row_stride, int q_off, int k_off, int v_off,
                                      float* __restrict__ state, const float* __restrict__ decay,
                                      const int32_t* __restrict__ seq_start, const int32_t* __restrict__ seq_slot,
                                      float* __restrict__ out, int H, int dim, int vdim, int parts, int n_chunks,
                                      int chunk_rows, float* __restrict__ chunk_state) {
  extern __shared__ __align__(16) float lds[];
  __shared__ float grow[LN_TOKENS], shrink[LN_TOKENS];      // decay^(t+1) and its inverse
  constexpr int PRE = (2 * LN_TOKENS * DPT + VT - 1) / VT + LN_TOKENS;      // a stage's elements a thread, at most
  const int seq = blockIdx.x / n_chunks, chunk = blockIdx.x % n_chunks, head = blockIdx.y, tile = blockIdx.z;
  const int threads = blockDim.x;
  const int j = threadIdx.x % VT, part = threadIdx.x / VT;
  const int column = tile * VT + j;
  const int padded = parts * DPT;                 // dim rounded up to whole slices; the padding holds zeros
  float* qs = lds;                                // [LN_TOKENS][padded]
  float* ks = qs + LN_TOKENS * padded;            // [LN_TOKENS][padded]
  float* vs = ks + LN_TOKENS * padded;            // [LN_TOKENS][VT]
  float* sums = vs + LN_TOKENS * VT;              // [LN_TOKENS][parts][VT]
  const int lo = seq_start[seq] + chunk * chunk_rows;
  if (lo >= seq_start[seq + 1]) return;      // the sequence has no such chunk
  const int hi = seq_start[seq + 1] < lo + chunk_rows ? seq_start[seq + 1] : lo + chunk_rows;
  const int slot = seq_slot[seq];
  const float lambda = decay[head];
  const bool scaled = lambda >= LN_SCALED_FROM;
  if (threadIdx.x < LN_TOKENS) {
    float power = lambda;
    for (int t = 0; t < (int)threadIdx.x; ++t) power *= lambda;
    grow[threadIdx.x] = scaled ? power : 1.f;
    shrink[threadIdx.x] = scaled ? 1.0f / power : 1.f;
  }
  float* mine = state + (((size_t)slot * H + head) * dim) * vdim;
  // where the end state goes: the cache, or with chunks the chunk's place in scratch memory
  float* left = n_chunks > 1 ? chunk_state + ((((size_t)seq * n_chunks + chunk) * H + head) * dim) * vdim : mine;
  const bool live = column < vdim;
  float s[DPT];
#pragma unroll
  for (int e = 0; e < DPT; ++e) {
    const int i = part * DPT + e;
    s[e] = (live && i < dim && chunk == 0) ? mine[(size_t)i * vdim + column] : 0.f;
  }
  // A stage's elements in one numbering, row after row: q [padded], k [padded], v [VT] of each row.  Where a thread's
  // elements come from (the column of a projected row, -1 for padding) and go to (the place in LDS) is worked out
  // once: the divisions are by run-time numbers.
  const int per_row = 2 * padded + VT, q_end = LN_TOKENS * padded, k_end = 2 * LN_TOKENS * padded;
  int src[PRE], dst[PRE], tok[PRE];
#pragma unroll
  for (int i = 0; i < PRE; ++i) {
    const int e = threadIdx.x + i * threads;
    const int t = e / per_row, r = e % per_row;
    tok[i] = t < LN_TOKENS ? t : LN_TOKENS;
    if (r < padded) {
      dst[i] = t * padded + r;
      src[i] = r < dim ? q_off + head * dim + r : -1;
    } else if (r < 2 * padded) {
      dst[i] = q_end + t * padded + (r - padded);
      src[i] = r - padded < dim ? k_off + head * dim + (r - padded) : -1;
    } else {
      dst[i] = k_end + t * VT + (r - 2 * padded);
      src[i] = tile * VT + (r - 2 * padded) < vdim ? v_off + head * vdim + tile * VT + (r - 2 * padded) : -1;
    }
  }
  // (`src` becomes the element's offset from the stage's first row.)  Every load is issued whether its element exists or
  // not, from a place that does, and masked afterwards: loads under a branch each waited for the one before.
  const int pre = (LN_TOKENS * per_row + threads - 1) / threads;      // elements a thread really has (<= PRE)
  __syncthreads();      // the powers are written
  float mul[PRE];       // what an element is multiplied by on its way into LDS: decay^(t+1) for q, its inverse for k
#pragma unroll
  for (int i = 0; i < PRE; ++i) {
    src[i] = src[i] >= 0 ? tok[i] * row_stride + src[i] : -1;
    const int t = tok[i] < LN_TOKENS ? tok[i] : 0;
    mul[i] = dst[i] < q_end ? grow[t] : (dst[i] < k_end ? shrink[t] : 1.f);
  }
  // What a load brings stays as it came until the stage is written into LDS: nothing in `fetch` reads a loaded value
  // (its widening to float32 and its mask come in `stage`), or every load would be waited for before the next is issued.
  T raw[PRE];
  auto fetch = [&](int r0) {
    const int n = hi - r0 < LN_TOKENS ? hi - r0 : LN_TOKENS;
    const T* first = proj + (size_t)r0 * row_stride;
#pragma unroll
    for (int i = 0; i < PRE; ++i) raw[i] = first[(tok[i] < n && src[i] >= 0) ? src[i] : 0];
  };
  auto stage = [&](int n) {
#pragma unroll
    for (int i = 0; i < PRE; ++i) {
      if (i < pre && tok[i] < n) lds[dst[i]] = src[i] >= 0 ? silu_f32(to_f32(raw[i])) * mul[i] : 0.f;
    }
  };
  if (lo < hi) fetch(lo);
  for (int r0 = lo; r0 < hi; r0 += LN_TOKENS) {
    const int n = hi - r0 < LN_TOKENS ? hi - r0 : LN_TOKENS;
    __syncthreads();      // the stage before has been read (and the powers are written)
    stage(n);
    __syncthreads();
    if (r0 + LN_TOKENS < hi) fetch(r0 + LN_TOKENS);      // on its way while this stage is computed
    // (The row's sum over this thread's slice is returned, not stored: a store into LDS between two rows' reads of LDS
    // would keep the next row's reads from starting early.  Two running sums halve the chain of dependent FMAs.)
    auto row_scaled = [&](int t) {
      const float v = vs[t * VT + j];
      const float* kt = ks + t * padded + part * DPT;
      const float* qt = qs + t * padded + part * DPT;
      float even = 0.f, odd = 0.f;
#pragma unroll
      for (int e = 0; e < DPT; e += 4) {
        const float4 k4 = *reinterpret_cast<const float4*>(kt + e), q4 = *reinterpret_cast<const float4*>(qt + e);
        s[e] = fmaf(k4.x, v, s[e]);
        s[e + 1] = fmaf(k4.y, v, s[e + 1]);
        s[e + 2] = fmaf(k4.z, v, s[e + 2]);
        s[e + 3] = fmaf(k4.w, v, s[e + 3]);
        even = fmaf(s[e], q4.x, even);
        odd = fmaf(s[e + 1], q4.y, odd);
        even = fmaf(s[e + 2], q4.z, even);
        odd = fmaf(s[e + 3], q4.w, odd);
      }
      return even + odd;
    };
    auto row_plain = [&](int t) {
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
    };
    if (scaled) {
      if (n == LN_TOKENS) {      // a whole stage: every row's reads can start before the row before is done
        float row_sums[LN_TOKENS];
#pragma unroll
        for (int t = 0; t < LN_TOKENS; ++t) row_sums[t] = row_scaled(t);
#pragma unroll
        for (int t = 0; t < LN_TOKENS; ++t) sums[(t * parts + part) * VT + j] = row_sums[t];
      } else {
        for (int t = 0; t < n; ++t) sums[(t * parts + part) * VT + j] = row_scaled(t);
      }
      const float back = grow[n - 1];
#pragma unroll
      for (int e = 0; e < DPT; ++e) s[e] *= back;
    } else {
      for (int t = 0; t < n; ++t) row_plain(t);
    }
    __syncthreads();
    for (int e = threadIdx.x; e < n * VT; e += threads) {
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
      if (i < dim) left[(size_t)i * vdim + column] = s[e];
    }
  }
}

// A step of one row a sequence (decoding): the same tiles and slices, but nothing to prefetch and no stage to walk, so
// none of the registers that hold a stage's places: the state streams through at several workgroups a compute unit.
template <typename T, int DPT, int VT>
__global__ __launch_bounds__(DPT == 64 ? 1024 : 256) void lightning_step_kernel(
    const T* __restrict__ proj, int row_stride, int q_off, int k_off, int v_off, float* __restrict__ state,
    const float* __restrict__ decay, const int32_t* __restrict__ seq_start, const int32_t* __restrict__ seq_slot,
    float* __restrict__ out, int H, int dim, int vdim, int parts) {
  extern __shared__ __align__(16) float lds[];
  const int seq = blockIdx.x, head = blockIdx.y, tile = blockIdx.z;
  const int j = threadIdx.x % VT, part = threadIdx.x / VT;
  const int column = tile * VT + j, padded = parts * DPT;
  float* qs = lds;              // [padded]
  float* ks = qs + padded;      // [padded]
  float* vs = ks + padded;      // [VT]
  float* sums = vs + VT;        // [parts][VT]
  const int row = seq_start[seq];
  if (seq_start[seq + 1] <= row) return;
  const float lambda = decay[head];
  float* mine = state + (((size_t)seq_slot[seq] * H + head) * dim) * vdim;
  const bool live = column < vdim;
  float s[DPT];
#pragma unroll
  for (int e = 0; e < DPT; ++e) {
    const int i = part * DPT + e;
    s[e] = (live && i < dim) ? mine[(size_t)i * vdim + column] : 0.f;
  }
  const T* from = proj + (size_t)row * row_stride;
  for (int i = threadIdx.x; i < padded; i += blockDim.x) {
    qs[i] = i < dim ? silu_f32(to_f32(from[q_off + head * dim + i])) : 0.f;
    ks[i] = i < dim ? silu_f32(to_f32(from[k_off + head * dim + i])) : 0.f;
  }
  for (int c = threadIdx.x; c < VT; c += blockDim.x)
    vs[c] = tile * VT + c < vdim ? silu_f32(to_f32(from[v_off + head * vdim + tile * VT + c])) : 0.f;
  __syncthreads();
  const float v = vs[j];
  float acc = 0.f;
#pragma unroll
  for (int e = 0; e < DPT; ++e) {
    s[e] = fmaf(lambda, s[e], ks[part * DPT + e] * v);
    acc = fmaf(s[e], qs[part * DPT + e], acc);
  }
  sums[part * VT + j] = acc;
  if (live) {
#pragma unroll
    for (int e = 0; e < DPT; ++e) {
      const int i = part * DPT + e;
      if (i < dim) mine[(size_t)i * vdim + column] = s[e];
    }
  }
  __syncthreads();
  if (threadIdx.x < VT && tile * VT + threadIdx.x < vdim) {
    float total = 0.f;
    for (int p = 0; p < parts; ++p) total += sums[p * VT + threadIdx.x];
    out[((size_t)row * H + head) * vdim + tile * VT + threadIdx.x] = total;
  }
}

// The chunks of a sequence in order (see the top of the file): a thread an element of the state.
__global__ __launch_bounds__(256) void lightning_combine_kernel(float* __restrict__ chunk_state, float* __restrict__ state,
                                                                const float* __restrict__ decay,
                                                                const int32_t* __restrict__ seq_start,
                                                                const int32_t* __restrict__ seq_slot, int H, int size,
                                                                int n_chunks, int chunk_rows) {
  const int seq = blockIdx.x, head = blockIdx.y, at = blockIdx.z * 256 + threadIdx.x;
  if (at >= size) return;
  const int rows = seq_start[seq + 1] - seq_start[seq];
  if (rows <= 0) return;
  const float lambda = decay[head];
  const size_t apart = (size_t)H * size;
  float* z = chunk_state + ((size_t)seq * n_chunks * H + head) * size + at;
  float end = z[0];
  for (int c = 1; c * chunk_rows < rows; ++c) {
    const int here = rows - c * chunk_rows < chunk_rows ? rows - c * chunk_rows : chunk_rows;
    const float own = z[c * apart];
    z[c * apart] = end;      // what chunk c should have started from
    end = fmaf(powf(lambda, (float)here), end, own);
  }
  state[((size_t)seq_slot[seq] * H + head) * size + at] = end;
}

// out[row] += decay^(t+1) E^T silu(q[row]) for the rows of every chunk but a sequence's first, E the state the chunk
// should have started from: LC_ROWS rows of one chunk and head a workgroup, their queries through LDS, a thread a
// value column.
#define LC_ROWS 16
template <typename T>
__global__ __launch_bounds__(256) void lightning_carry_kernel(const T* __restrict__ proj, int row_stride, int q_off,
                                                              const float* __restrict__ chunk_state,
                                                              const float* __restrict__ decay,
                                                              const int32_t* __restrict__ seq_start, float* __restrict__ out,
                                                              int H, int dim, int vdim, int n_chunks, int chunk_rows) {
  extern __shared__ __align__(16) float xs[];      // [dim][LC_ROWS]
  const int per_chunk = chunk_rows / LC_ROWS;
  const int piece = blockIdx.x % per_chunk, chunk = 1 + (blockIdx.x / per_chunk) % (n_chunks - 1);
  const int seq = blockIdx.x / (per_chunk * (n_chunks - 1)), head = blockIdx.y;
  const int first = seq_start[seq] + chunk * chunk_rows, lo = first + piece * LC_ROWS;
  const int last = seq_start[seq + 1] < first + chunk_rows ? seq_start[seq + 1] : first + chunk_rows;
  if (lo >= last) return;
  const int rows = last - lo < LC_ROWS ? last - lo : LC_ROWS;
  const float lambda = decay[head];
  for (int e = threadIdx.x; e < dim * LC_ROWS; e += blockDim.x) {
    const int i = e / LC_ROWS, r = e % LC_ROWS;
    float value = 0.f;
    if (r < rows)
      value = silu_f32(to_f32(proj[(size_t)(lo + r) * row_stride + q_off + (size_t)head * dim + i])) *
              powf(lambda, (float)(piece * LC_ROWS + r + 1));
    xs[e] = value;
  }
  __syncthreads();
  const int column = blockIdx.z * blockDim.x + threadIdx.x;
  if (column >= vdim) return;
  const float* from = chunk_state + ((((size_t)seq * n_chunks + chunk) * H + head) * dim) * vdim + column;
  float acc[LC_ROWS] = {};
#pragma unroll 8      // eight elements of the state asked for before the first is used
  for (int i = 0; i < dim; ++i) {
    const float w = from[(size_t)i * vdim];
#pragma unroll
    for (int r = 0; r < LC_ROWS; r += 4) {
      const float4 x4 = *reinterpret_cast<const float4*>(xs + i * LC_ROWS + r);
      acc[r] = fmaf(x4.x, w, acc[r]);
      acc[r + 1] = fmaf(x4.y, w, acc[r + 1]);
      acc[r + 2] = fmaf(x4.z, w, acc[r + 2]);
      acc[r + 3] = fmaf(x4.w, w, acc[r + 3]);
    }
  }
#pragma unroll
  for (int r = 0; r < LC_ROWS; ++r)
    if (r < rows) out[((size_t)(lo + r) * H + head) * vdim + column] += acc[r];
}

// Into how many chunks of how many rows the sequences of a step are cut (1: not at all): as many as it takes to give
// every compute unit two workgroups of 64 value columns, chunks of 64 rows at least and whole stages of rows.
extern "C" int bh_lightning_chunks(int n_seqs, int n_rows, int max_rows, int H, int vdim, int* chunk_rows) {
  const int tiles = (vdim + 63) / 64;
  const long groups = (long)n_seqs * H * tiles, wanted = 2L * bh_compute_units();
  *chunk_rows = max_rows > 0 ? max_rows : 1;
  if (n_rows == n_seqs || max_rows < 128 || groups >= wanted) return 1;
  const long cuts = (wanted + groups - 1) / groups;
  int rows = (int)((max_rows + cuts - 1) / cuts);
  rows = rows < 64 ? 64 : (rows + LN_TOKENS - 1) / LN_TOKENS * LN_TOKENS;
  *chunk_rows = rows;
  return (max_rows + rows - 1) / rows;
}

template <typename T, int DPT, int VT>
static int launch_lightning(const void* proj, int row_stride, int q_off, int k_off, int v_off, float* state,
                            const float* decay, const int32_t* seq_start, const int32_t* seq_slot, float* out, int n_seqs,
                            int n_rows, int H, int dim, int vdim, int n_chunks, int chunk_rows, float* chunk_state,
                            hipStream_t stream) {
  const int parts = (dim + DPT - 1) / DPT;
  BH_REQUIRE(parts * VT <= 1024, "lightning: heads of %d x %d need more than 1024 threads", dim, vdim);
  const int tiles = (vdim + VT - 1) / VT;
  const size_t smem = (size_t)LN_TOKENS * (2 * parts * DPT + VT + parts * VT) * sizeof(float);
  BH_REQUIRE(smem <= 63 * 1024, "lightning: heads of %d x %d need %zu bytes of LDS", dim, vdim, smem);
  dim3 grid(n_seqs * n_chunks, H, tiles), block(parts * VT);
  if (n_rows == n_seqs) {      // one row each
    const size_t lean = (size_t)(2 * parts * DPT + VT + parts * VT) * sizeof(float);
    lightning_step_kernel<T, DPT, VT><<<grid, block, lean, stream>>>((const T*)proj, row_stride, q_off, k_off, v_off, state, decay,
                                                                     seq_start, seq_slot, out, H, dim, vdim, parts);
    return bh_check_launch("lightning_step");
  }
  lightning_scan_kernel<T, DPT, VT><<<grid, block, smem, stream>>>((const T*)proj, row_stride, q_off, k_off, v_off, state, decay,
                                                                   seq_start, seq_slot, out, H, dim, vdim, parts, n_chunks,
                                                                   chunk_rows, chunk_state);
  if (int status = bh_check_launch("lightning_scan")) return status;
  if (n_chunks == 1) return 0;
  const int size = dim * vdim;
  lightning_combine_kernel<<<dim3(n_seqs, H, (size + 255) / 256), dim3(256), 0, stream>>>(chunk_state, state, decay, seq_start,
                                                                                          seq_slot, H, size, n_chunks, chunk_rows);
  if (int status = bh_check_launch("lightning_combine")) return status;
  const int columns = vdim >= 256 ? 256 : (vdim + 63) / 64 * 64;
  dim3 carry(n_seqs * (n_chunks - 1) * (chunk_rows / LC_ROWS), H, (vdim + columns - 1) / columns);
  lightning_carry_kernel<T><<<carry, dim3(columns), (size_t)dim * LC_ROWS * sizeof(float), stream>>>(
      (const T*)proj, row_stride, q_off, chunk_state, decay, seq_start, out, H, dim, vdim, n_chunks, chunk_rows);
  return bh_check_launch("lightning_carry");
}

// proj [n_rows][row_stride]: a row holds q (H x dim) from q_off, k (H x dim) from k_off, v (H x vdim) from v_off, all
// before their silu.  state [slots][H][dim][vdim] float32; rows seq_start[b] .. seq_start[b + 1] - 1 belong to the
// sequence in slot seq_slot[b], in order, and every sequence has at least one.  out [n_rows][H * vdim] float32.
extern "C" int bh_lightning_scan(const void* proj, int dtype, int row_stride, int q_off, int k_off, int v_off, float* state,
                                 const float* decay, const int32_t* seq_start, const int32_t* seq_slot, float* out,
                                 int n_seqs, int n_rows, int max_rows, int H, int dim, int vdim, float* chunk_state,
                                 long chunk_state_floats, hipStream_t stream) {
  BH_REQUIRE(n_seqs > 0 && n_rows >= n_seqs && H > 0 && dim > 0 && vdim > 0,
             "lightning: sizes must be positive, and every sequence of the step brings a row");
  BH_REQUIRE(H <= 65535 && n_seqs <= 2147483647, "lightning: too many heads");
  BH_REQUIRE(dim <= 1024, "lightning: a key size of %d is above the limit of 1024", dim);
  BH_REQUIRE(q_off >= 0 && k_off >= 0 && v_off >= 0 && q_off + H * dim <= row_stride && k_off + H * dim <= row_stride &&
                 v_off + H * vdim <= row_stride,
             "lightning: q, k and v do not lie inside a row of %d", row_stride);
  // max_rows: no sequence of the step brings more rows (what the cut into chunks is made for)
  int chunk_rows = 0;
  const int n_chunks = bh_lightning_chunks(n_seqs, n_rows, max_rows > 0 && max_rows < n_rows ? max_rows : n_rows, H, vdim, &chunk_rows);
  BH_REQUIRE(n_chunks == 1 || (chunk_state != nullptr && chunk_state_floats >= (long)n_seqs * n_chunks * H * dim * vdim),
             "lightning: %d chunks a sequence need scratch memory for their states", n_chunks);
  BH_REQUIRE((long)n_seqs * n_chunks * (chunk_rows / LC_ROWS + 1) < (1L << 31), "lightning: too many workgroups");
  BH_REQUIRE((size_t)dim * LC_ROWS * sizeof(float) <= 63 * 1024, "lightning: a key size of %d is too large to cut a sequence into chunks", dim);
  // value columns a workgroup: 64 where that many workgroups fill the chip twice, else fewer, down to 16
  int vt = vdim > 32 ? 64 : (vdim > 16 ? 32 : 16);
  while (vt > 16 && (long)n_seqs * n_chunks * H * ((vdim + vt - 1) / vt) < 2L * bh_compute_units()) vt /= 2;
  const int slice = (dim + 256 / vt - 1) / (256 / vt);      // slices of dim that make the workgroup four waves
#define BH_LN(T, DPT)                                                                                                   \
  do {                                                                                                                  \
    if (vt == 64) return launch_lightning<T, DPT, 64>(proj, row_stride, q_off, k_off, v_off, state, decay, seq_start, seq_slot, out, n_seqs, n_rows, H, dim, vdim, n_chunks, chunk_rows, chunk_state, stream); \
    if (vt == 32) return launch_lightning<T, DPT, 32>(proj, row_stride, q_off, k_off, v_off, state, decay, seq_start, seq_slot, out, n_seqs, n_rows, H, dim, vdim, n_chunks, chunk_rows, chunk_state, stream); \
    return launch_lightning<T, DPT, 16>(proj, row_stride, q_off, k_off, v_off, state, decay, seq_start, seq_slot, out, n_seqs, n_rows, H, dim, vdim, n_chunks, chunk_rows, chunk_state, stream); \
  } while (0)
#define BH_LN_SIZES(T)            \
  if (slice <= 4) BH_LN(T, 4);    \
  if (slice <= 8) BH_LN(T, 8);    \
  if (slice <= 16) BH_LN(T, 16);  \
  if (slice <= 32) BH_LN(T, 32);  \
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
