// Block bookkeeping and the affinity-weighted combine (scatter-add) for the blockwise MoE.
//
// The reference accumulates each block's bf16 contribution into the output rows with a
// read-modify-write scatter in block order (bwmm_shard_on_block.py:1005-1038; golden
// test_moe_cte_common.py:430-434).  On the GPU the down GEMM writes every slot's contribution
// once (bf16, already multiplied by the affinity) and one pass per token then adds that
// token's contributions in ascending slot order -- the same order and the same bf16
// arithmetic as the golden, deterministic, and without atomics.  HBM traffic: each
// contribution row is written once and read once, each output row written once.
#include "combine.hpp"
#include "chunks.hpp"

namespace moe {

// n_active = index of the first zero in conditions (N when there is none / no conditions);
// valid_rows[b] = 1 + last row of block b holding a real token id (0 for an all-padding block
// or a block at/after n_active or with an expert id outside [0, E)).
__global__ __launch_bounds__(256) void prep_blocks_kernel(const int32_t* __restrict__ tp2id,
                                                          const int32_t* __restrict__ b2e,
                                                          const int32_t* __restrict__ conditions, int64_t n_conditions,
                                                          int64_t N, int64_t B, int64_t E, int64_t n_real,
                                                          int32_t* __restrict__ n_active,
                                                          int32_t* __restrict__ valid_rows,
                                                          int32_t* __restrict__ cnt) {
  __shared__ int s_first_zero;
  __shared__ int s_red[4];
  if (threadIdx.x == 0) s_first_zero = (int)N;
  __syncthreads();
  if (conditions) {
    const int64_t lim = n_conditions < N ? n_conditions : N;
    for (int64_t i = threadIdx.x; i < lim; i += blockDim.x)
      if (conditions[i] == 0) atomicMin(&s_first_zero, (int)i);
  }
  __syncthreads();
  const int na = s_first_zero;
  if (blockIdx.x == 0 && threadIdx.x == 0) *n_active = na;
  for (int64_t b = blockIdx.x; b < N; b += gridDim.x) {
    int v = 0;
    const int e = b2e[b];
    if (b < na && e >= 0 && e < E) {
      for (int64_t r = threadIdx.x; r < B; r += blockDim.x) {
        const int id = tp2id[b * B + r];
        if (id >= 0 && id < n_real) {
          v = (int)r + 1;
          atomicAdd(&cnt[id], 1);  // slots per token, for the token -> slot lists of the combine
        }
      }
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v = max(v, __shfl_xor(v, o, 64));
    __syncthreads();
    if ((threadIdx.x & 63) == 0) s_red[threadIdx.x >> 6] = v;
    __syncthreads();
    if (threadIdx.x == 0) valid_rows[b] = max(max(s_red[0], s_red[1]), max(s_red[2], s_red[3]));
  }
}

__global__ __launch_bounds__(256) void fill_zero_kernel(int32_t* __restrict__ p, int64_t n) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) p[i] = 0;
}

// Exclusive scan of cnt[0..n) into off[0..n] by one workgroup of 1024 threads: a thread owns 8 consecutive
// elements of each 8192-element tile.
__device__ __forceinline__ void inv_scan(const int32_t* __restrict__ cnt, int32_t* __restrict__ off, int64_t n,
                                         int* s_ws) {
  int carry = 0;
  for (int64_t base = 0; base < n; base += 8192) {
    const int64_t i0 = base + 8 * (int64_t)threadIdx.x;
    int v[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) v[j] = (i0 + j < n) ? cnt[i0 + j] : 0;
    int mine = 0;
#pragma unroll
    for (int j = 0; j < 8; ++j) mine += v[j];
    int total;
    int run = carry + block_excl_scan(mine, s_ws, &total);
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      if (i0 + j < n) off[i0 + j] = run;
      run += v[j];
    }
    carry += total;
  }
  if (threadIdx.x == 0) off[n] = carry;
}

// Two workgroups of 1024 threads, run after prep_blocks_kernel: workgroup 0 builds the expert chunks,
// workgroup 1 turns the slots-per-token counts into list offsets.  They share no data.
__global__ __launch_bounds__(1024) void chunks_and_offsets_kernel(
    const int32_t* __restrict__ b2e, const int32_t* __restrict__ n_active, const int32_t* __restrict__ valid_rows,
    int64_t N, int64_t B, int64_t E, int32_t* __restrict__ n_chunks, int32_t* __restrict__ chunk_slot,
    int32_t* __restrict__ chunk_rows, int32_t* __restrict__ chunk_expert, int32_t* __restrict__ chunk_xcd,
    int32_t* __restrict__ q_chunk, int32_t* __restrict__ q_off, int64_t max_chunks,
    const int32_t* __restrict__ cnt, int32_t* __restrict__ off, int64_t n_real, bool whole_blocks) {
  __shared__ int s_ws[16];
  if (blockIdx.x == 0)
    build_chunks(b2e, n_active, valid_rows, N, B, E, n_chunks, chunk_slot, chunk_rows, chunk_expert, chunk_xcd, q_chunk,
                 q_off, max_chunks, s_ws, whole_blocks);
  else
    inv_scan(cnt, off, n_real, s_ws);
}

// One workgroup: chunks and work queues from a block build's own valid rows (moe_build_blocks_plan).
__global__ __launch_bounds__(1024) void plan_chunks_kernel(
    const int32_t* __restrict__ b2e, const int32_t* __restrict__ n_active, const int32_t* __restrict__ valid_rows,
    int64_t N, int64_t B, int64_t E, int32_t* __restrict__ n_chunks, int32_t* __restrict__ chunk_slot,
    int32_t* __restrict__ chunk_rows, int32_t* __restrict__ chunk_expert, int32_t* __restrict__ chunk_xcd,
    int32_t* __restrict__ q_chunk, int32_t* __restrict__ q_off, int64_t max_chunks) {
  __shared__ int s_ws[16];
  build_chunks(b2e, n_active, valid_rows, N, B, E, n_chunks, chunk_slot, chunk_rows, chunk_expert, chunk_xcd, q_chunk,
               q_off, max_chunks, s_ws, false);
}

// The whole bookkeeping of a small problem (decode-sized: a few ten thousand slots) by ONE workgroup of 1024
// threads in one launch: clear the per-token counts, find the active blocks and their valid rows, count the slots
// per token, build the expert chunks and the work queues, scan the counts and fill the token -> slot lists.  The
// four launches it replaces take longer to start than to run at such sizes.  Steps communicate through global
// memory that this workgroup alone writes and reads, ordered by workgroup barriers.
__global__ __launch_bounds__(1024) void prep_small_kernel(
    const int32_t* __restrict__ tp2id, const int32_t* __restrict__ b2e, const int32_t* __restrict__ conditions,
    int64_t n_conditions, int64_t N, int64_t B, int64_t E, int64_t n_real, int32_t* __restrict__ n_active,
    int32_t* __restrict__ valid_rows, int32_t* __restrict__ cnt, int64_t clear_words, int32_t* __restrict__ n_chunks,
    int32_t* __restrict__ chunk_slot, int32_t* __restrict__ chunk_rows, int32_t* __restrict__ chunk_expert,
    int32_t* __restrict__ chunk_xcd, int32_t* __restrict__ q_chunk, int32_t* __restrict__ q_off, int64_t max_chunks,
    int32_t* __restrict__ off, int32_t* __restrict__ cursor, int32_t* __restrict__ list, bool whole_blocks) {
  __shared__ int s_ws[16];
  __shared__ int s_first_zero;
  for (int64_t i = threadIdx.x; i < clear_words; i += blockDim.x) cnt[i] = 0;  // cnt and cursor are adjacent
  for (int64_t b = threadIdx.x; b < N; b += blockDim.x) valid_rows[b] = 0;
  if (threadIdx.x == 0) s_first_zero = (int)N;
  __threadfence_block();
  __syncthreads();
  if (conditions) {
    const int64_t lim = n_conditions < N ? n_conditions : N;
    for (int64_t i = threadIdx.x; i < lim; i += blockDim.x)
      if (conditions[i] == 0) atomicMin(&s_first_zero, (int)i);
  }
  __syncthreads();
  const int na = s_first_zero;
  if (threadIdx.x == 0) *n_active = na;
  // A wave per active block, four blocks at a time so that a wave has their loads in flight together (blocks from
  // the first zero condition on hold nothing: a decode-sized batch is mostly such blocks, and their valid rows
  // were cleared above).  body(u, slot, row, id) runs for every slot that holds a token in a block with a valid
  // expert; after(u, block) once per block.
  constexpr int U = 4;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, nwaves = blockDim.x >> 6;
  const int iB = (int)B;
  auto over_blocks = [&](auto&& body, auto&& after) {
    for (int b0 = wave * U; b0 < na; b0 += nwaves * U) {
      int e[U];
#pragma unroll
      for (int u = 0; u < U; ++u) e[u] = (b0 + u < na) ? b2e[b0 + u] : -1;
      for (int r0 = 0; r0 < iB; r0 += 64) {
        const int r = r0 + lane;
        int id[U];
#pragma unroll
        for (int u = 0; u < U; ++u) id[u] = (b0 + u < na && r < iB) ? tp2id[(b0 + u) * iB + r] : -1;
#pragma unroll
        for (int u = 0; u < U; ++u)
          if (e[u] >= 0 && e[u] < E && id[u] >= 0 && id[u] < n_real) body(u, (b0 + u) * iB + r, r, id[u]);
      }
#pragma unroll
      for (int u = 0; u < U; ++u)
        if (b0 + u < na) after(u, b0 + u);
    }
  };
  int v[U];
#pragma unroll
  for (int u = 0; u < U; ++u) v[u] = 0;
  over_blocks(
      [&](int u, int, int r, int id) {
        v[u] = r + 1;  // rows ascend: the last one stays
        atomicAdd(&cnt[id], 1);
      },
      [&](int u, int b) {
        int m = v[u];
#pragma unroll
        for (int o = 32; o > 0; o >>= 1) m = max(m, __shfl_xor(m, o, 64));
        if (lane == 0) valid_rows[b] = m;  // valid rows = 1 + last row with a real token
        v[u] = 0;
      });
  __threadfence_block();
  __syncthreads();
  build_chunks(b2e, n_active, valid_rows, N, B, E, n_chunks, chunk_slot, chunk_rows, chunk_expert, chunk_xcd, q_chunk,
               q_off, max_chunks, s_ws, whole_blocks);
  __syncthreads();
  inv_scan(cnt, off, n_real, s_ws);
  __threadfence_block();
  __syncthreads();
  over_blocks(
      [&](int, int sl, int, int id) {
        const int p = atomicAdd(&cursor[id], 1);
        list[off[id] + p] = sl;
      },
      [&](int, int) {});
}

__global__ __launch_bounds__(256) void inv_fill_kernel(const int32_t* __restrict__ tp2id,
                                                       const int32_t* __restrict__ valid_rows, int64_t N, int64_t B,
                                                       int64_t n_real, const int32_t* __restrict__ off,
                                                       int32_t* __restrict__ cursor, int32_t* __restrict__ list) {
  const int64_t s = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (s >= N * B) return;
  const int64_t b = s / B, r = s % B;
  if (r >= valid_rows[b]) return;
  const int id = tp2id[s];
  if (id >= 0 && id < n_real) {
    const int p = atomicAdd(&cursor[id], 1);
    list[off[id] + p] = (int32_t)s;
  }
}

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

// One workgroup per output row (a few, side by side along the row, when the rows are too few to fill the GPU:
// gridDim.y).  D: bf16 [N*B, H] contributions.
__global__ __launch_bounds__(256) void combine_kernel(const uint16_t* __restrict__ D, const int32_t* __restrict__ off,
                                                      const int32_t* __restrict__ list, uint16_t* __restrict__ out,
                                                      uint16_t* __restrict__ out_shard1, int64_t out_row_stride,
                                                      int64_t H, int64_t n_real) {
  __shared__ int s_sorted[COMBINE_MAX_K];
  const int64_t t = blockIdx.x;
  int cnt = 0, base = 0;
  if (t < n_real) {
    base = off[t];
    cnt = off[t + 1] - base;
    if (cnt > COMBINE_MAX_K) cnt = COMBINE_MAX_K;  // rejected on the host: a token has at most E <= MAX_K slots
  }
  // rank sort: ascending slot index == block order of the reference's accumulation.  (A list handed over by the
  // block build has a fixed number of entries per token, -1 where the token has no slot: those are left out.)
  int holes = 0;
  for (int j = 0; j < cnt; ++j) holes += list[base + j] < 0;
  for (int i = threadIdx.x; i < cnt; i += blockDim.x) {
    const int mine = list[base + i];
    if (mine < 0) continue;
    int rank = 0;
    for (int j = 0; j < cnt; ++j) {
      const int other = list[base + j];
      rank += (other >= 0 && other < mine);
    }
    s_sorted[rank] = mine;
  }
  cnt -= holes;
  __syncthreads();
  uint16_t* orow = out + t * out_row_stride;
  uint16_t* zrow = out_shard1 ? out_shard1 + t * out_row_stride : nullptr;  // the other shard's row: zeros
  const bool vec = (H % 8 == 0) && ((out_row_stride % 8) == 0) && (((uintptr_t)out & 15) == 0) &&
                   (((uintptr_t)out_shard1 & 15) == 0);
  const int64_t vt = (int64_t)blockIdx.y * blockDim.x + threadIdx.x, vstride = (int64_t)gridDim.y * blockDim.x;
  if (vec) {
    for (int64_t c = vt * 8; c < H; c += vstride * 8) {
      float acc[8];
#pragma unroll
      for (int k = 0; k < 8; ++k) acc[k] = 0.f;
      // the additions form one dependent chain (bf16 rounding after each, in slot order), so the loads
      // are what can overlap: up to eight rows are requested before the first is added
      for (int j0 = 0; j0 < cnt; j0 += 8) {
        // (the contributions are read once and the result rows are not read again by this kernel: non-temporal,
        // so that neither displaces the other in the caches)
        u32x4 d[8];
#pragma unroll
        for (int j = 0; j < 8; ++j)
          if (j0 + j < cnt) d[j] = __builtin_nontemporal_load((const u32x4*)(D + (int64_t)s_sorted[j0 + j] * H + c));
#pragma unroll
        for (int j = 0; j < 8; ++j) {
          if (j0 + j < cnt) {
            const uint32_t w[4] = {d[j][0], d[j][1], d[j][2], d[j][3]};
#pragma unroll
            for (int k = 0; k < 4; ++k) {
              acc[2 * k] = round_to_bf16(acc[2 * k] + bf16_bits_to_f32((uint16_t)(w[k] & 0xffff)));
              acc[2 * k + 1] = round_to_bf16(acc[2 * k + 1] + bf16_bits_to_f32((uint16_t)(w[k] >> 16)));
            }
          }
        }
      }
      uint32_t o[4];
#pragma unroll
      for (int k = 0; k < 4; ++k)
        o[k] = (uint32_t)f32_to_bf16_bits(acc[2 * k]) | ((uint32_t)f32_to_bf16_bits(acc[2 * k + 1]) << 16);
      __builtin_nontemporal_store((u32x4){o[0], o[1], o[2], o[3]}, (u32x4*)(orow + c));
      if (zrow) __builtin_nontemporal_store((u32x4){0, 0, 0, 0}, (u32x4*)(zrow + c));
    }
  } else {
    for (int64_t c = vt; c < H; c += vstride) {
      float acc = 0.f;
      for (int j = 0; j < cnt; ++j) acc = round_to_bf16(acc + bf16_bits_to_f32(D[(int64_t)s_sorted[j] * H + c]));
      orow[c] = f32_to_bf16_bits(acc);
      if (zrow) zrow[c] = 0;
    }
  }
}

// ---- host-side orchestration used by moe_blockwise() -------------------------------------

size_t bookkeeping_bytes(int64_t T1, int64_t N, int64_t B) {
  // n_active[4] | valid_rows[N] | cnt[T1] | cursor[T1] | off[T1+1] | list[N*B] | n_chunks[4] | 6 x chunk[max_chunks] |
  // q_off[8][CHUNK_CLASSES + 1], each region 256-byte aligned
  auto al = [](size_t v) { return (v + 255) & ~(size_t)255; };
  return al(16) + al((size_t)N * 4) + 2 * al((size_t)T1 * 4) + al((size_t)(T1 + 1) * 4) + al((size_t)N * B * 4) +
         al(16) + 6 * al((size_t)max_chunks_for(N, B) * 4) + al((size_t)(8 * (CHUNK_CLASSES + 1) + 1) * 4);
}

Bookkeeping carve_bookkeeping(void* base, int64_t T1, int64_t N, int64_t B) {
  auto al = [](size_t v) { return (v + 255) & ~(size_t)255; };
  Bookkeeping k;
  uint8_t* p = (uint8_t*)base;
  k.n_active = (int32_t*)p; p += al(16);
  k.valid_rows = (int32_t*)p; p += al((size_t)N * 4);
  k.cnt = (int32_t*)p; p += al((size_t)T1 * 4);
  k.cursor = (int32_t*)p; p += al((size_t)T1 * 4);
  k.off = (int32_t*)p; p += al((size_t)(T1 + 1) * 4);
  k.list = (int32_t*)p; p += al((size_t)N * B * 4);
  k.max_chunks = max_chunks_for(N, B);
  k.n_chunks = (int32_t*)p; p += al(16);
  k.chunk_slot = (int32_t*)p; p += al((size_t)k.max_chunks * 4);
  k.chunk_rows = (int32_t*)p; p += al((size_t)k.max_chunks * 4);
  k.chunk_expert = (int32_t*)p; p += al((size_t)k.max_chunks * 4);
  k.chunk_xcd = (int32_t*)p; p += al((size_t)k.max_chunks * 4);
  k.q_chunk = (int32_t*)p; p += 2 * al((size_t)k.max_chunks * 4);
  k.q_off = (int32_t*)p;
  return k;
}

// up to this many slots and tokens the bookkeeping is one launch of one workgroup (prep_small_kernel)
constexpr int64_t PREP_SMALL_SLOTS = 40960, PREP_SMALL_TOKENS = 4096;

int launch_prep(const Bookkeeping& k, const moe_bwmm_args* a, int64_t n_real, hipStream_t s) {
  const bool whole_blocks = a->gate_up_activations_T != nullptr || a->down_activations != nullptr;
  // cnt and cursor are adjacent: one clear covers both.  A fill kernel rather than a memset
  // node, so that the sequence stays safe to record into a HIP graph.
  const int64_t clear_words = (int64_t)((uint8_t*)k.off - (uint8_t*)k.cnt) / 4;
  if (a->N * a->B <= PREP_SMALL_SLOTS && n_real <= PREP_SMALL_TOKENS) {
    hipLaunchKernelGGL(prep_small_kernel, dim3(1), dim3(1024), 0, s, a->token_position_to_id, a->block_to_expert,
                       a->conditions, a->n_conditions, a->N, a->B, a->E, n_real, k.n_active, k.valid_rows, k.cnt,
                       clear_words, k.n_chunks, k.chunk_slot, k.chunk_rows, k.chunk_expert, k.chunk_xcd, k.q_chunk,
                       k.q_off, k.max_chunks, k.off, k.cursor, k.list, whole_blocks);
    MOE_CHECK_LAUNCH();
    return MOE_OK;
  }
  hipLaunchKernelGGL(fill_zero_kernel, dim3((unsigned)((clear_words + 255) / 256)), dim3(256), 0, s, k.cnt,
                     clear_words);
  MOE_CHECK_LAUNCH();
  const unsigned g = (unsigned)(a->N < 1024 ? a->N : 1024);
  hipLaunchKernelGGL(prep_blocks_kernel, dim3(g), dim3(256), 0, s, a->token_position_to_id, a->block_to_expert,
                     a->conditions, a->n_conditions, a->N, a->B, a->E, n_real, k.n_active, k.valid_rows, k.cnt);
  MOE_CHECK_LAUNCH();
  hipLaunchKernelGGL(chunks_and_offsets_kernel, dim3(2), dim3(1024), 0, s, a->block_to_expert, k.n_active, k.valid_rows,
                     a->N, a->B, a->E, k.n_chunks, k.chunk_slot, k.chunk_rows, k.chunk_expert, k.chunk_xcd, k.q_chunk, k.q_off,
                     k.max_chunks, k.cnt, k.off, n_real, whole_blocks);
  MOE_CHECK_LAUNCH();
  const int64_t slots = a->N * a->B;
  const unsigned gs = (unsigned)((slots + 255) / 256);
  hipLaunchKernelGGL(inv_fill_kernel, dim3(gs), dim3(256), 0, s, a->token_position_to_id, k.valid_rows, a->N, a->B,
                     n_real, k.off, k.cursor, k.list);
  MOE_CHECK_LAUNCH();
  return MOE_OK;
}

int launch_plan_chunks(const Bookkeeping& k, const int32_t* block_to_expert, int64_t N, int64_t B, int64_t E,
                       hipStream_t s) {
  hipLaunchKernelGGL(plan_chunks_kernel, dim3(1), dim3(1024), 0, s, block_to_expert, k.n_active, k.valid_rows, N, B, E,
                     k.n_chunks, k.chunk_slot, k.chunk_rows, k.chunk_expert, k.chunk_xcd, k.q_chunk, k.q_off,
                     k.max_chunks);
  MOE_CHECK_LAUNCH();
  return MOE_OK;
}

int launch_combine(const Bookkeeping& k, const moe_bwmm_args* a, const void* D, int64_t n_real, hipStream_t s) {
  // few rows (decode): up to 8 workgroups share a row, 8 columns per thread each
  unsigned split = 1;
  if (a->T1 <= 256) {
    const int64_t per_wg = 256 * 8;
    split = (unsigned)((a->H + per_wg - 1) / per_wg);
    if (split > 8) split = 8;
    if (split < 1) split = 1;
  }
  hipLaunchKernelGGL(combine_kernel, dim3((unsigned)a->T1, split), dim3(256), 0, s, (const uint16_t*)D, k.off, k.list,
                     (uint16_t*)a->output, (uint16_t*)a->output_shard1, a->out_row_stride, a->H, n_real);
  MOE_CHECK_LAUNCH();
  return MOE_OK;
}

int launch_fill_zero_bytes(void* p, size_t bytes, hipStream_t s) {
  if (bytes == 0) return MOE_OK;
  if ((bytes & 3) != 0 || ((uintptr_t)p & 3) != 0) return MOE_E_BAD_ARG;
  const int64_t words = (int64_t)(bytes / 4);
  const int64_t grid = (words + 255) / 256;
  if (grid >= (int64_t)1 << 31) return MOE_E_BAD_SHAPE;
  hipLaunchKernelGGL(fill_zero_kernel, dim3((unsigned)grid), dim3(256), 0, s, (int32_t*)p, words);
  MOE_CHECK_LAUNCH();
  return MOE_OK;
}

}  // namespace moe
