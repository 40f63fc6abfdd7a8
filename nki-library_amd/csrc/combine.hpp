// Block bookkeeping shared by the blockwise MoE driver and the combine kernels.
#pragma once

#include "common.hpp"

namespace moe {

constexpr int COMBINE_MAX_K = 512;  // most slots one token may own (one per expert it selected)

struct Bookkeeping {
  int32_t* n_active;    // [1]  blocks before the first conditions[b] == 0
  int32_t* valid_rows;  // [N]  rows of block b up to and including its last real token
  int32_t* cnt;         // [T1] slots per token
  int32_t* cursor;      // [T1]
  int32_t* off;         // [T1+1] exclusive scan of cnt
  int32_t* list;        // [N*B] slot indices grouped by token
  // Expert chunks: maximal runs of consecutive active blocks of one expert, cut into pieces of
  // CHUNK_ROWS slots (the last piece: up to CHUNK_ROWS_MAX).  chunk c covers slots [chunk_slot[c], chunk_slot[c] + chunk_rows[c]).
  int32_t* n_chunks;      // [1]
  int32_t* chunk_slot;    // [max_chunks]
  int32_t* chunk_rows;    // [max_chunks]
  int32_t* chunk_expert;  // [max_chunks]
  int32_t* chunk_xcd;     // [max_chunks] the XCD whose queue holds the chunk
  // Work queues of the large-tile MX kernels.  The chunk list is cut into eight contiguous parts of about equal
  // work (row tiles), one per XCD; q_chunk holds a part's chunks grouped by class (row-tile variant x last chunk of its expert, CHUNK_CLASSES of them), two
  // words per chunk: its first slot, and rows | expert << 16; q_off[x][c] .. q_off[x][c+1] are the positions of
  // class c of XCD x in q_chunk.
  int32_t* q_chunk;       // [max_chunks][2]
  int32_t* q_off;         // [8][CHUNK_CLASSES + 1], then one word: the chunk interleave (see build_chunks)
  int64_t max_chunks;
};

constexpr int CHUNK_CLASSES = 8;
// class of a chunk: its row-tile variant (0: up to 64 rows, 1: 128, 2: 256, 3: 320), largest first, then whether
// it is the last chunk of its expert
__host__ __device__ inline int chunk_class(int rows, bool last) {
  const int v = rows <= 64 ? 0 : rows <= 128 ? 1 : rows <= 256 ? 2 : 3;
  return (3 - v) * 2 + (last ? 1 : 0);
}

constexpr int CHUNK_ROWS = 256;      // rows of every chunk of a run but the last
constexpr int CHUNK_ROWS_MAX = 320;  // the last chunk of a run takes up to this many
inline int64_t max_chunks_for(int64_t N, int64_t B) { return N * ((B + CHUNK_ROWS - 1) / CHUNK_ROWS); }

size_t bookkeeping_bytes(int64_t T1, int64_t N, int64_t B);
Bookkeeping carve_bookkeeping(void* base, int64_t T1, int64_t N, int64_t B);
// n_real: number of real token rows (ids in [0, n_real) are tokens, everything else is padding).
int launch_prep(const Bookkeeping& k, const moe_bwmm_args* a, int64_t n_real, hipStream_t s);
int launch_combine(const Bookkeeping& k, const moe_bwmm_args* a, const void* D, int64_t n_real, hipStream_t s);
// Zero `bytes` bytes at p (a multiple of 4, p 4-byte aligned) with a kernel, so that callers may capture it in a graph.
int launch_fill_zero_bytes(void* p, size_t bytes, hipStream_t s);

}  // namespace moe
