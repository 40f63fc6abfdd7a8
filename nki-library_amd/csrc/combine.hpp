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

// Classes of chunks = instances of the large-tile kernels' tile loop: how many 16-row tiles the instance multiplies
// (at least the chunk's rows / 16) and whether the chunk is the last one of its expert (its weights are then
// streamed past the L2).  Last chunks, which carry an expert's ragged remainder, choose among eight row-tile counts,
// so that at most one or two tiles of a chunk multiply padding (a router's 256 +- 15 rows per expert made one MFMA in
// eight multiply padding with the counts 4 / 8 / 16 / 20 alone); chunks that are not the last of their expert hold
// exactly CHUNK_ROWS rows unless chunks are interleaved (see build_chunks), and choose among four.  Queue order =
// class order: largest tiles first, so that a launch ends on its small ones.
constexpr int CHUNK_CLASSES = 12;
constexpr int CHUNK_CLASS_TILES[CHUNK_CLASSES] = {20, 20, 18, 16, 16, 14, 12, 10, 8, 8, 4, 4};
constexpr bool CHUNK_CLASS_LAST[CHUNK_CLASSES] = {false, true, true, false, true, true, true, true, false, true, false, true};
// 16-row tiles of the instance that runs a chunk of `rows` rows
__host__ __device__ inline int chunk_row_tiles(int rows, bool last) {
  if (!last) return rows <= 64 ? 4 : rows <= 128 ? 8 : rows <= 256 ? 16 : 20;
  return rows <= 64 ? 4 : rows <= 128 ? 8 : 2 * ((rows + 31) / 32);
}
__host__ __device__ inline int chunk_class(int rows, bool last) {
  const int t = chunk_row_tiles(rows, last);
  if (!last) return t == 20 ? 0 : t == 16 ? 3 : t == 8 ? 8 : 10;
  return t == 20 ? 1 : t == 18 ? 2 : t == 16 ? 4 : t == 14 ? 5 : t == 12 ? 6 : t == 10 ? 7 : t == 8 ? 9 : 11;
}

constexpr int CHUNK_ROWS = 256;      // rows of every chunk of a run but the last
constexpr int CHUNK_FIXED_COST_TILES = 20;  // a chunk's loads per K slice, in row tiles of MFMA time (XCD balance)
constexpr int CHUNK_ROWS_MAX = 320;  // the last chunk of a run takes up to this many
inline int64_t max_chunks_for(int64_t N, int64_t B) { return N * ((B + CHUNK_ROWS - 1) / CHUNK_ROWS); }

size_t bookkeeping_bytes(int64_t T1, int64_t N, int64_t B);
Bookkeeping carve_bookkeeping(void* base, int64_t T1, int64_t N, int64_t B);
// n_real: number of real token rows (ids in [0, n_real) are tokens, everything else is padding).
int launch_prep(const Bookkeeping& k, const moe_bwmm_args* a, int64_t n_real, hipStream_t s);
// The chunk list and the work queues alone, from valid_rows / n_active that the caller has filled in (the block
// build's hand-over, see moe_build_blocks_plan).
int launch_plan_chunks(const Bookkeeping& k, const int32_t* block_to_expert, int64_t N, int64_t B, int64_t E,
                       hipStream_t s);
int launch_combine(const Bookkeeping& k, const moe_bwmm_args* a, const void* D, int64_t n_real, hipStream_t s);
// Zero `bytes` bytes at p (a multiple of 4, p 4-byte aligned) with a kernel, so that callers may capture it in a graph.
int launch_fill_zero_bytes(void* p, size_t bytes, hipStream_t s);

}  // namespace moe
