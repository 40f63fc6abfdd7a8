// Device-side pieces of the token -> block index construction, as separate operators:
//   find_nonzero_indices  (src/nkilib_src/nkilib/core/subkernels/find_nonzero_indices.py:34-110;
//                          semantics find_nonzero_indices_torch_ref, find_nonzero_indices_torch.py:20-63)
//   indexed_flatten       (src/nkilib_src/nkilib/core/subkernels/indexed_flatten.py:28-86;
//                          semantics indexed_flatten_torch_ref, indexed_flatten_torch.py:18-66)
//   cumsum                (src/nkilib_src/nkilib/core/cumsum/cumsum.py:30-75; cumsum_torch.py:20-32)
// All three are HBM-bound integer / byte work: coalesced reads of 128-byte row segments, workgroup scans,
// no atomics (the order of the indices is part of the result).
#include "common.hpp"

namespace moe {

constexpr int IX_THREADS = 256;
constexpr int FNZ_COLS = 32;                       // columns per workgroup: 128-byte row segments of 4-byte elements
constexpr int FNZ_RSUB = IX_THREADS / FNZ_COLS;    // 8 row runs per workgroup
constexpr int FNZ_RUN = 64;                        // rows per run: one bit each in a 64-bit mask
constexpr int FNZ_CHUNK = FNZ_RSUB * FNZ_RUN;      // 512 rows per workgroup

__device__ __forceinline__ bool is_nonzero(const void* p, int dtype, int64_t i) {
  if (dtype == MOE_DT_INT32) return ((const int32_t*)p)[i] != 0;
  if (dtype == MOE_DT_FP32) return (((const uint32_t*)p)[i] & 0x7fffffffu) != 0;  // -0.0 is zero, NaN is not
  return (((const uint16_t*)p)[i] & 0x7fffu) != 0;                                // bf16 / fp16
}

// Workgroup (chunk, column group): thread (run r, column c) walks rows chunk*512 + 64 r .. + 63 of its column
// (the 32 threads of a run read one 128-byte segment per row) and keeps the nonzero flags in a 64-bit mask.
// WRITE == false: counts[chunk][col] = nonzeros of the chunk.  WRITE == true: base[chunk][col] (exclusive scan
// over chunks) + the nonzeros of the runs before + rank inside the run gives each index its slot.
template <bool WRITE>
__global__ __launch_bounds__(IX_THREADS) void fnz_kernel(const void* x, int dtype, int64_t T, int64_t C_full,
                                                         const int32_t* col_start_id, int64_t n_cols,
                                                         int32_t* chunk_counts, int32_t* indices) {
  __shared__ int cnt[FNZ_RSUB][FNZ_COLS];
  const int c = threadIdx.x % FNZ_COLS, r = threadIdx.x / FNZ_COLS;
  const int64_t col_out = (int64_t)blockIdx.y * FNZ_COLS + c;
  const int64_t col_in = col_out + (col_start_id ? (int64_t)col_start_id[0] : 0);
  const bool col_ok = col_out < n_cols && col_in >= 0 && col_in < C_full;
  const int64_t t0 = (int64_t)blockIdx.x * FNZ_CHUNK + (int64_t)r * FNZ_RUN;
  uint64_t mask = 0;
  if (col_ok) {
#pragma unroll 8
    for (int i = 0; i < FNZ_RUN; ++i) {
      const int64_t t = t0 + i;
      if (t < T && is_nonzero(x, dtype, t * C_full + col_in)) mask |= (uint64_t)1 << i;
    }
  }
  const int mine = __popcll(mask);
  cnt[r][c] = mine;
  __syncthreads();
  int before = 0, total = 0;
#pragma unroll
  for (int j = 0; j < FNZ_RSUB; ++j) {
    const int v = cnt[j][c];
    before += (j < r) ? v : 0;
    total += v;
  }
  if constexpr (!WRITE) {
    if (r == 0 && col_out < n_cols) chunk_counts[(int64_t)blockIdx.x * n_cols + col_out] = total;
  } else {
    if (!col_ok) return;
    int32_t* dst = indices + col_out * T + chunk_counts[(int64_t)blockIdx.x * n_cols + col_out] + before;
    while (mask) {
      const int i = __builtin_ctzll(mask);
      mask &= mask - 1;
      *dst++ = (int32_t)(t0 + i);
    }
  }
}

// One thread per column: chunk_counts[:, col] -> exclusive scan in place, total -> nonzero_counts[col].
__global__ void fnz_scan_kernel(int32_t* chunk_counts, int64_t n_chunks, int64_t n_cols, int32_t* nonzero_counts) {
  const int64_t col = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (col >= n_cols) return;
  int run = 0;
  for (int64_t k = 0; k < n_chunks; ++k) {
    const int v = chunk_counts[k * n_cols + col];
    chunk_counts[k * n_cols + col] = run;
    run += v;
  }
  nonzero_counts[col] = run;
}

// indices[col][count .. T) = -1
__global__ __launch_bounds__(IX_THREADS) void fnz_pad_kernel(int32_t* indices, const int32_t* nonzero_counts, int64_t T) {
  const int64_t col = blockIdx.y;
  const int64_t t = ((int64_t)blockIdx.x * IX_THREADS + threadIdx.x) * 4;
  const int64_t n = nonzero_counts[col];
  int32_t* row = indices + col * T;
  if (t >= T || t + 4 <= n) return;
  if (t >= n && t + 4 <= T && ((uintptr_t)(row + t) & 15) == 0) {
    *(v4i*)(row + t) = (v4i){-1, -1, -1, -1};
    return;
  }
  for (int i = 0; i < 4; ++i)
    if (t + i >= n && t + i < T) row[t + i] = -1;
}

// Workgroup per output block b of f_len elements: the source is block b - off(e) of the LAST row e whose range
// [off(e), off(e) + T / f_len) holds b (the reference writes the rows in ascending order, later rows over
// earlier ones); no such row: padding.
__global__ __launch_bounds__(IX_THREADS) void indexed_flatten_kernel(const int32_t* x, int64_t E, int64_t T,
                                                                     int64_t f_len, const int32_t* row_offsets,
                                                                     const int32_t* row_offsets_start, int64_t n_offsets,
                                                                     int32_t padding_val, int32_t* out) {
  __shared__ int win[IX_THREADS / WAVE];
  const int64_t b = blockIdx.x, per_row = T / f_len;
  const int64_t start = row_offsets_start ? (int64_t)row_offsets_start[0] : 0;
  int best = -1;
  for (int64_t e = threadIdx.x; e < E; e += IX_THREADS) {
    const int64_t k = start + e;
    if (k < 0 || k >= n_offsets) continue;
    const int64_t off = row_offsets[k];
    if (b >= off && b < off + per_row) best = (int)e;  // ascending e: the last match stays
  }
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) best = max(best, __shfl_xor(best, o, 64));
  if ((threadIdx.x & 63) == 0) win[threadIdx.x >> 6] = best;
  __syncthreads();
  best = max(max(win[0], win[1]), max(win[2], win[3]));
  int32_t* dst = out + b * f_len;
  if (best < 0) {
    for (int64_t i = threadIdx.x; i < f_len; i += IX_THREADS) dst[i] = padding_val;
  } else {
    const int32_t* src = x + (int64_t)best * T + (b - (int64_t)row_offsets[start + best]) * f_len;
    for (int64_t i = threadIdx.x; i < f_len; i += IX_THREADS) dst[i] = src[i];
  }
}

// Inclusive scan of each row of [rows, H] in tiles of 1024 elements: a thread owns 4 consecutive elements of a
// tile, the thread totals are scanned over the workgroup and the tile total is carried to the next tile.
// Floats accumulate in fp32 and are rounded to the element type on the store; int32 is exact (wrapping).
template <class Acc>
__device__ __forceinline__ Acc block_excl_scan_t(Acc v, Acc* ws, Acc* total) {
  const int lane = threadIdx.x & 63, w = threadIdx.x >> 6, nw = blockDim.x >> 6;
  Acc inc = v;
#pragma unroll
  for (int o = 1; o < 64; o <<= 1) {
    const Acc t = __shfl_up(inc, o, 64);
    if (lane >= o) inc += t;
  }
  __syncthreads();  // `ws` may still be read from the previous tile
  if (lane == 63) ws[w] = inc;
  __syncthreads();
  Acc base = 0, tot = 0;
  for (int i = 0; i < nw; ++i) {
    const Acc t = ws[i];
    base += (i < w) ? t : (Acc)0;
    tot += t;
  }
  *total = tot;
  Acc before = __shfl_up(inc, 1, 64);  // not inc - v: that would round twice for floats
  if (lane == 0) before = 0;
  return base + before;
}

template <class Acc>
__device__ __forceinline__ Acc cs_load(const void* p, int dtype, int64_t i) {
  if (dtype == MOE_DT_INT32) return (Acc)((const int32_t*)p)[i];
  return (Acc)load_as_f32(p, dtype, i);
}
template <class Acc>
__device__ __forceinline__ void cs_store(void* p, int dtype, int64_t i, Acc v) {
  if (dtype == MOE_DT_INT32) ((int32_t*)p)[i] = (int32_t)v;
  else if (dtype == MOE_DT_FP32) ((float*)p)[i] = (float)v;
  else if (dtype == MOE_DT_BF16) ((uint16_t*)p)[i] = f32_to_bf16_bits((float)v);
  else {
    const _Float16 h = (_Float16)(float)v;
    __builtin_memcpy((uint16_t*)p + i, &h, 2);
  }
}

template <class Acc>
__global__ __launch_bounds__(IX_THREADS) void cumsum_kernel(const void* x, void* y, int dtype, int64_t H) {
  __shared__ Acc ws[IX_THREADS / WAVE];
  const int64_t base = (int64_t)blockIdx.x * H;
  Acc carry = 0;
  for (int64_t h0 = 0; h0 < H; h0 += 4 * IX_THREADS) {
    const int64_t h = h0 + 4 * (int64_t)threadIdx.x;
    Acc v[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) v[i] = (h + i < H) ? cs_load<Acc>(x, dtype, base + h + i) : (Acc)0;
    v[1] += v[0];
    v[2] += v[1];
    v[3] += v[2];
    Acc total;
    const Acc before = carry + block_excl_scan_t<Acc>(v[3], ws, &total);
#pragma unroll
    for (int i = 0; i < 4; ++i)
      if (h + i < H) cs_store<Acc>(y, dtype, base + h + i, before + v[i]);
    carry += total;
  }
}

}  // namespace moe

using namespace moe;

static int64_t fnz_chunks(int64_t T) { return (T + FNZ_CHUNK - 1) / FNZ_CHUNK; }

extern "C" size_t moe_find_nonzero_indices_workspace_bytes(int64_t T, int64_t n_cols) {
  if (T < 0 || n_cols < 0) return 0;
  return (size_t)(fnz_chunks(T) * n_cols + 1) * sizeof(int32_t);
}

extern "C" int moe_find_nonzero_indices(const void* input, int dtype, int64_t T, int64_t C_full,
                                        const int32_t* col_start_id, int64_t n_cols, int32_t* indices,
                                        int32_t* nonzero_counts, void* workspace, size_t workspace_bytes,
                                        void* stream) {
  if (!input || !indices || !nonzero_counts) return MOE_E_BAD_ARG;
  if (dtype != MOE_DT_INT32 && dtype != MOE_DT_FP32 && dtype != MOE_DT_BF16 && dtype != MOE_DT_FP16) return MOE_E_BAD_ARG;
  if (T <= 0 || C_full <= 0 || n_cols <= 0) return MOE_E_BAD_ARG;
  if (!col_start_id && n_cols > C_full) return MOE_E_BAD_SHAPE;
  if (T >= (int64_t)1 << 31) return MOE_E_BAD_SHAPE;
  if (!workspace || workspace_bytes < moe_find_nonzero_indices_workspace_bytes(T, n_cols)) return MOE_E_WORKSPACE;
  const int64_t n_chunks = fnz_chunks(T), groups = (n_cols + FNZ_COLS - 1) / FNZ_COLS;
  if (groups > 65535 || n_cols > 65535) return MOE_E_BAD_SHAPE;
  int32_t* chunk_counts = (int32_t*)workspace;
  hipStream_t s = (hipStream_t)stream;
  const dim3 grid((unsigned)n_chunks, (unsigned)groups);
  hipLaunchKernelGGL(fnz_kernel<false>, grid, dim3(IX_THREADS), 0, s, input, dtype, T, C_full, col_start_id, n_cols,
                     chunk_counts, (int32_t*)nullptr);
  MOE_CHECK_LAUNCH();
  hipLaunchKernelGGL(fnz_scan_kernel, dim3((unsigned)((n_cols + 63) / 64)), dim3(64), 0, s, chunk_counts, n_chunks,
                     n_cols, nonzero_counts);
  MOE_CHECK_LAUNCH();
  hipLaunchKernelGGL(fnz_kernel<true>, grid, dim3(IX_THREADS), 0, s, input, dtype, T, C_full, col_start_id, n_cols,
                     chunk_counts, indices);
  MOE_CHECK_LAUNCH();
  hipLaunchKernelGGL(fnz_pad_kernel, dim3((unsigned)((T + 4 * IX_THREADS - 1) / (4 * IX_THREADS)), (unsigned)n_cols),
                     dim3(IX_THREADS), 0, s, indices, nonzero_counts, T);
  MOE_CHECK_LAUNCH();
  return MOE_OK;
}

extern "C" int moe_indexed_flatten(const int32_t* input, int64_t E, int64_t T, int64_t f_len, int64_t output_len,
                                   const int32_t* row_offsets, int64_t n_offsets, const int32_t* row_offsets_start,
                                   int32_t padding_val, int32_t* output, void* stream) {
  if (!input || !row_offsets || !output) return MOE_E_BAD_ARG;
  if (E <= 0 || T <= 0 || f_len <= 0 || output_len <= 0 || n_offsets <= 0) return MOE_E_BAD_ARG;
  if (T % f_len != 0 || output_len % f_len != 0) return MOE_E_BAD_SHAPE;
  if (!row_offsets_start && n_offsets != E) return MOE_E_BAD_SHAPE;
  if (row_offsets_start && n_offsets < E) return MOE_E_BAD_SHAPE;
  const int64_t n_blocks = output_len / f_len;
  if (n_blocks >= (int64_t)1 << 31) return MOE_E_BAD_SHAPE;
  hipLaunchKernelGGL(indexed_flatten_kernel, dim3((unsigned)n_blocks), dim3(IX_THREADS), 0, (hipStream_t)stream, input,
                     E, T, f_len, row_offsets, row_offsets_start, n_offsets, padding_val, output);
  MOE_CHECK_LAUNCH();
  return MOE_OK;
}

extern "C" int moe_cumsum(const void* x, void* y, int dtype, int64_t rows, int64_t H, void* stream) {
  if (!x || !y) return MOE_E_BAD_ARG;
  if (rows <= 0 || H <= 0 || rows >= (int64_t)1 << 31) return MOE_E_BAD_ARG;
  hipStream_t s = (hipStream_t)stream;
  if (dtype == MOE_DT_INT32)
    hipLaunchKernelGGL(cumsum_kernel<int32_t>, dim3((unsigned)rows), dim3(IX_THREADS), 0, s, x, y, dtype, H);
  else if (dtype == MOE_DT_FP32 || dtype == MOE_DT_BF16 || dtype == MOE_DT_FP16)
    hipLaunchKernelGGL(cumsum_kernel<float>, dim3((unsigned)rows), dim3(IX_THREADS), 0, s, x, y, dtype, H);
  else
    return MOE_E_BAD_ARG;
  MOE_CHECK_LAUNCH();
  return MOE_OK;
}
