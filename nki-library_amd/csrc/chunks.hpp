// The expert chunks and the per-XCD work queues of the large-tile GEMMs, built by one workgroup from the blocks'
// experts and valid rows.  Shared by the blockwise layer's own bookkeeping (csrc/combine.hip) and by the block build
// that hands its bookkeeping over (csrc/build_blocks.hip).
#pragma once

#include "combine.hpp"

namespace moe {

// One workgroup (a multiple of 64 threads, at most 1024).  A "run" is a maximal sequence of
// consecutive active blocks of one expert; the thread that owns a run's first block measures the
// run (slots up to its last real token) and, after a block-wide scan of the chunk counts, writes
// the run's chunks.  Chunk order follows block order.
__device__ __forceinline__ void build_chunks(const int32_t* __restrict__ b2e, const int32_t* __restrict__ n_active,
                                             const int32_t* __restrict__ valid_rows, int64_t N, int64_t B, int64_t E,
                                             int32_t* __restrict__ n_chunks, int32_t* __restrict__ chunk_slot,
                                             int32_t* __restrict__ chunk_rows, int32_t* __restrict__ chunk_expert,
                                             int32_t* __restrict__ chunk_xcd, int32_t* __restrict__ q_chunk,
                                             int32_t* __restrict__ q_off, int64_t max_chunks, int* s_ws,
                                             bool whole_blocks) {
  const int64_t na = *n_active;
  // The walk along a run below is a chain of dependent reads, one block after the other: from LDS when the active
  // blocks fit there (a global read per step made the run length the pace of this kernel).
  constexpr int BLOCKS_IN_LDS = 2048;
  __shared__ int s_e[BLOCKS_IN_LDS], s_v[BLOCKS_IN_LDS];
  const bool staged = na <= BLOCKS_IN_LDS;
  if (staged) {
    for (int64_t j = threadIdx.x; j < na; j += blockDim.x) {
      s_e[j] = b2e[j];
      s_v[j] = valid_rows[j];
    }
    __syncthreads();
  }
  auto expert_of = [&](int64_t j) { return staged ? s_e[j] : b2e[j]; };
  auto valid_of = [&](int64_t j) { return staged ? s_v[j] : valid_rows[j]; };
  // The chunk list as the later steps of this function read it: from LDS as well while it fits (each step would
  // otherwise begin with a round trip to the L2 for what the step before has just written).
  constexpr int CHUNKS_IN_LDS = 2048;
  __shared__ int s_cslot[CHUNKS_IN_LDS], s_cre[CHUNKS_IN_LDS], s_cx[CHUNKS_IN_LDS];
  int carry = 0;
  int runs = 0;  // runs that hold chunks (over this thread's runs)
  for (int64_t b0 = 0; b0 < na; b0 += blockDim.x) {
    const int64_t b = b0 + threadIdx.x;
    int nch = 0;
    int64_t last_end = -1;
    int e = -1;
    if (b < na) {
      e = expert_of(b);
      const bool start = (b == 0) || (expert_of(b - 1) != e);
      if (start && e >= 0 && e < E) {
        // (whole_blocks: activation checkpoints hold every row of every executed block, padding rows included, so
        // a run's chunks then cover its blocks to the end)
        for (int64_t j = b; j < na && expert_of(j) == e; ++j) {
          const int v = whole_blocks ? (int)B : valid_of(j);
          if (v > 0) last_end = j * B + v;
        }
        // chunks of CHUNK_ROWS rows; the last one absorbs a remainder of up to CHUNK_ROWS_MAX - CHUNK_ROWS
        // rows, which saves the pass over the expert's weights that a small chunk of its own would cost
        const int64_t len = last_end - b * B;
        if (len > 0) nch = (len <= CHUNK_ROWS_MAX) ? 1 : (int)((len - CHUNK_ROWS_MAX + CHUNK_ROWS - 1) / CHUNK_ROWS) + 1;
      }
    }
    runs += nch > 0;
    int total;
    const int base = carry + block_excl_scan(nch, s_ws, &total);
    for (int k = 0; k < nch; ++k) {
      const int64_t s0 = b * B + (int64_t)k * CHUNK_ROWS;
      const int32_t rows = (int32_t)((k + 1 < nch) ? CHUNK_ROWS : (last_end - s0));
      if (base + k < max_chunks) {
        chunk_slot[base + k] = (int32_t)s0;
        chunk_rows[base + k] = rows;
        chunk_expert[base + k] = e;
      }
      if (base + k < CHUNKS_IN_LDS) {
        s_cslot[base + k] = (int32_t)s0;
        s_cre[base + k] = rows | (e << 16);  // at most 320 rows, fewer than 32768 experts
      }
    }
    carry += total;
  }
  const int n = (int)((carry < max_chunks) ? carry : max_chunks);
  if (threadIdx.x == 0) *n_chunks = (int32_t)n;
  // Work queues: a counting sort of the chunks by (XCD that owns them, class).  The chunk arrays were written by
  // this workgroup: make them visible to all of its threads first.
  __shared__ int s_cnt[8 * CHUNK_CLASSES + 1];
  __shared__ int s_runs;
  if (threadIdx.x == 0) s_runs = 0;
  __threadfence_block();
  __syncthreads();
  if (runs > 0) atomicAdd(&s_runs, runs);
  __syncthreads();
  // How many chunks of one expert the large-tile GEMMs work on side by side (the kernels read it behind q_off).
  // While experts hold fewer than three chunks on average: 1, i.e. a round of an XCD's workgroups covers the column
  // tiles of one chunk after the other and shares that chunk's activation tile.  With three and more (few experts
  // with many rows each): that average, up to 8, i.e. the item order of a class alternates between G neighbouring
  // chunks, which are then mostly chunks of one expert: they work on the same weight tile at the same time and
  // share it through the L2 instead of streaming it from memory once per chunk.  (Applied to a skewed router's
  // few hot experts among many single-chunk ones it costs more in activation sharing than it saves, and at two
  // chunks per expert on average it changes nothing: both measured.)
  const int avg = s_runs > 0 ? (n + s_runs / 2) / s_runs : 1;
  // (not beyond the number of chunks whose keys fit in LDS for the rank order below)
  constexpr int KEYS_IN_LDS = 4096;
  const int interleave = (avg < 3 || n > KEYS_IN_LDS) ? 1 : (avg > 8 ? 8 : avg);
  if (threadIdx.x == 0) q_off[8 * (CHUNK_CLASSES + 1)] = interleave;
  for (int i = threadIdx.x; i <= 8 * CHUNK_CLASSES; i += blockDim.x) s_cnt[i] = 0;
  // Which XCD takes which chunks: contiguous parts of the list (chunks of one expert, and experts that follow each
  // other, stay behind one L2) of about equal work.  Work = row tiles of the kernel variant that runs the chunk
  // plus a fixed cost (its column tiles are the same for all); a chunk goes where the middle of its span of the
  // running total falls.
  // (Equal chunk counts left the XCDs up to a tenth apart in work at ragged expert loads, and a launch ends when
  // its last XCD does.)
  const bool in_lds = n <= CHUNKS_IN_LDS;
  auto rows_of = [&](int i) { return in_lds ? (s_cre[i] & 0xffff) : chunk_rows[i]; };
  auto chunk_expert_of = [&](int i) { return in_lds ? (s_cre[i] >> 16) : chunk_expert[i]; };
  auto slot_of = [&](int i) { return in_lds ? s_cslot[i] : chunk_slot[i]; };
  auto xcd_of = [&](int i) { return in_lds ? s_cx[i] : chunk_xcd[i]; };
  auto xcd_put = [&](int i, int v) {
    if (in_lds) s_cx[i] = v;
    else chunk_xcd[i] = v;
  };
  // (what a chunk costs per K slice is its loads, the same for every chunk, plus its MFMAs: measured over the
  // row-tile classes 1.16 us + 0.055 us per row tile, i.e. 21 row tiles' worth of fixed cost)
  auto work_of = [&](int i) { return chunk_row_tiles(rows_of(i), true) + CHUNK_FIXED_COST_TILES; };
  int wcarry = 0;
  for (int i0 = 0; i0 < n; i0 += (int)blockDim.x) {
    const int i = i0 + threadIdx.x;
    int total;
    const int pre = wcarry + block_excl_scan(i < n ? work_of(i) : 0, s_ws, &total);
    if (i < n) xcd_put(i, pre);
    wcarry += total;
  }
  __threadfence_block();
  __syncthreads();
  for (int i = threadIdx.x; i < n; i += blockDim.x) {
    const int64_t mid2 = 2 * (int64_t)xcd_of(i) + work_of(i);  // twice the middle of the chunk's span
    const int x = (int)(mid2 * 8 / (2 * (int64_t)wcarry));
    xcd_put(i, x > 7 ? 7 : x);
  }
  __threadfence_block();
  __syncthreads();
  // (interleaved chunks share their weight tiles through the L2: none of them streams the weights past it, so
  // "last chunk of its expert" is no class of its own then)
  auto key_of = [&](int i) {
    const bool last = interleave == 1 && ((i + 1 >= n) || (chunk_expert_of(i + 1) != chunk_expert_of(i)));
    return xcd_of(i) * CHUNK_CLASSES + chunk_class(rows_of(i), last);
  };
  __shared__ uint8_t s_key[KEYS_IN_LDS];  // the chunks' keys, for the rank loop below
  for (int i = threadIdx.x; i < n; i += blockDim.x) {
    const int key = key_of(i);
    if (i < KEYS_IN_LDS) s_key[i] = (uint8_t)key;
    atomicAdd(&s_cnt[key], 1);
  }
  __syncthreads();
  {
    // exclusive scan of the (XCD, class) counts: the queues' first items (a thread per count; one thread walking
    // all of them took longer than the rest of a decode-sized call)
    static_assert(8 * CHUNK_CLASSES <= 256, "a thread per queue");
    // queue entries and the LDS chunk list pack (expert << 16 | rows) into one non-negative int
    static_assert(CHUNK_ROWS_MAX < (1 << 16) && COMBINE_MAX_K <= (1 << 15), "rows | expert << 16 fits an int32");
    const int k = threadIdx.x;
    const bool mine = k < 8 * CHUNK_CLASSES;
    const int c = mine ? s_cnt[k] : 0;
    int total;
    const int run = block_excl_scan(c, s_ws, &total);
    if (mine) {
      s_cnt[k] = run;
      q_off[(k / CHUNK_CLASSES) * (CHUNK_CLASSES + 1) + k % CHUNK_CLASSES] = run;
      if (k % CHUNK_CLASSES == CHUNK_CLASSES - 1) q_off[(k / CHUNK_CLASSES) * (CHUNK_CLASSES + 1) + CHUNK_CLASSES] = run + c;
    }
  }
  __syncthreads();
  // (the order inside one class is whatever order the atomics are served in: it decides which chunks run at the
  // same time, never a result)
  // With interleaving neighbours in the queue must be chunks of the same expert, so a chunk's place in its class
  // is its rank by chunk index (the chunks of this shape family are few).
  for (int i = threadIdx.x; i < n; i += blockDim.x) {
    const int key = key_of(i);
    int pos;
    if (interleave == 1) {
      pos = atomicAdd(&s_cnt[key], 1);
    } else {
      int rank = 0;
      for (int j = 0; j < i; ++j) rank += s_key[j] == key;
      pos = s_cnt[key] + rank;
    }
    q_chunk[2 * pos] = slot_of(i);
    q_chunk[2 * pos + 1] = rows_of(i) | (chunk_expert_of(i) << 16);  // at most 320 rows, fewer than 32768 experts
  }
}

}  // namespace moe
