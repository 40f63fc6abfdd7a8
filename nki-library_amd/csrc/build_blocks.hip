// Token -> block index construction on the GPU (integer, bit exact with the reference helper
// generate_token_position_to_id_and_experts,
// test/integration/nkilib/core/moe/moe_cte/test_moe_cte_common.py:199-264).
//
// A stable counting sort of the routed (token, expert) pairs by expert that reads the ids twice and nothing
// else: the tokens are cut into at most 64 slabs, one workgroup each.
//   1. count_kernel    per slab, 256 tokens at a time: every token sets its bit in the LDS bitmap of each expert
//                      it selected; population counts give the slab's tokens per expert.  The grid also fills
//                      token_position_to_id with the pad id.
//   2. layout_kernel   one workgroup: per expert the sum of the slabs' counts; blocks per expert, padding blocks to the last
//                      expert (or split), exclusive scan -> first slot of every expert, block_to_expert, conditions
//   3. scatter_kernel  per slab, the same bitmaps again: a token's rank among the tokens of its expert is the
//                      number of set bits below its own, plus the slab's offset; writes the token ids
// The work is latency bound (a few hundred KB of int32), so each step is a single small launch.
#include <mutex>

#include "chunks.hpp"
#include "combine.hpp"
#include "common.hpp"

namespace moe {

constexpr int BB_THREADS = 256;

constexpr int BB_SLABS_MAX = 64;
constexpr int64_t BB_SINGLE_MAX_TOKENS = 1024;  // up to this many tokens form one slab, built by a single launch
constexpr int64_t BB_SINGLE_MAX_SLOTS = 1 << 17;  // one workgroup fills the pad ids of up to this many slots itself
constexpr int BB_E_MAX = 1024;  // bitmaps and running counts of all experts in LDS: 36 bytes per expert
constexpr size_t BB_CHUNKS_STATIC_LDS = 46 * 1024;  // static LDS of build_chunks (csrc/chunks.hpp), rounded up

// What the block build can tell the blockwise layer without another pass over the slots (all null: nothing):
// the blocks in use, the valid rows of every block, and for every routed (token, j) pair the slot it was given.
struct BlockPlanOut {
  int32_t* n_active;    // [1]   blocks that hold tokens' experts (those before the padding blocks)
  int32_t* valid_rows;  // [N]   rows of a block that hold tokens (they are packed from the block's first row)
  int32_t* off;         // [T+1] first list entry of token t: t * k
  int32_t* list;        // [T*k] slot of (t, j), or -1 (id outside [0, E), an id listed before in the row, no room)
  // The layout step's workgroup goes on to cut the expert chunks and fill the work queues (build_chunks) when
  // chunks_inline is set: the tables that takes (all of the blockwise layer's Bookkeeping).
  int chunks_inline;
  Bookkeeping k;
};

// The bitmaps of 256 tokens: bit (tid & 31) of word bm[(tid >> 5) * E + e] says that token t0 + tid selected
// expert e.  Ids outside [0, E) are ignored; an id listed twice sets its bit once.
__device__ __forceinline__ void bb_mark(const int32_t* __restrict__ ids, int64_t t, bool live, int64_t k, int64_t E,
                                        uint32_t* bm, int my[8]) {
  const uint32_t bit = 1u << (threadIdx.x & 31);
  uint32_t* row = bm + (threadIdx.x >> 5) * E;
  if (k == 8) {  // two 16-byte loads
    int4 a = make_int4(-1, -1, -1, -1), b = a;
    if (live) {
      a = ((const int4*)(ids + t * 8))[0];
      b = ((const int4*)(ids + t * 8))[1];
    }
    my[0] = a.x; my[1] = a.y; my[2] = a.z; my[3] = a.w;
    my[4] = b.x; my[5] = b.y; my[6] = b.z; my[7] = b.w;
#pragma unroll
    for (int j = 0; j < 8; ++j)
      if (my[j] >= 0 && my[j] < E) atomicOr(&row[my[j]], bit);
  } else if (live) {
    for (int64_t j = 0; j < k; ++j) {
      const int e = ids[t * k + j];
      if (e >= 0 && e < E) atomicOr(&row[e], bit);
    }
  }
}

__device__ __forceinline__ int bb_bits(const uint32_t* bm, int64_t E, int64_t e) {
  int n = 0;
#pragma unroll
  for (int w = 0; w < 8; ++w) n += __popc(bm[w * E + e]);
  return n;
}

// This workgroup's share of the pad ids: 16 bytes per store where the table allows it.
__device__ __forceinline__ void bb_fill_pad(int32_t* __restrict__ tp2id, int64_t NB, int pad_id, int64_t slab,
                                            int64_t n_wg) {
  if ((NB & 3) == 0 && ((uintptr_t)tp2id & 15) == 0) {
    const int4 v = make_int4(pad_id, pad_id, pad_id, pad_id);
    for (int64_t i = slab * BB_THREADS + threadIdx.x; i < NB / 4; i += n_wg * BB_THREADS) ((int4*)tp2id)[i] = v;
  } else {
    for (int64_t i = slab * BB_THREADS + threadIdx.x; i < NB; i += n_wg * BB_THREADS) tp2id[i] = pad_id;
  }
}

// Workgroup = slab of slab_tokens tokens (a multiple of 256).  slab_counts[slab][e] = tokens of the slab that
// selected e.  All workgroups together also fill token_position_to_id with the pad id, which the scatter
// overwrites where tokens sit.
// (slab = this workgroup's slab, n_wg = workgroups that share the pad fill; bb_lds = 9 E words of LDS)
__device__ __forceinline__ void bb_count_body(const int32_t* __restrict__ ids, int64_t T, int64_t k, int64_t E,
                                              int64_t slab_tokens, int32_t* __restrict__ slab_counts,
                                              int32_t* __restrict__ tp2id, int64_t NB, int pad_id, int64_t slab,
                                              int64_t n_wg, uint32_t* bb_lds) {
  uint32_t* bm = bb_lds;            // [8][E]
  int* run = (int*)(bb_lds + 8 * E);  // [E]
  for (int64_t e = threadIdx.x; e < E; e += BB_THREADS) run[e] = 0;
  const int64_t t_begin = slab * slab_tokens;
  for (int64_t sub = 0; sub < slab_tokens && t_begin + sub < T; sub += BB_THREADS) {
    for (int64_t i = threadIdx.x; i < 8 * E; i += BB_THREADS) bm[i] = 0;
    __syncthreads();
    const int64_t t = t_begin + sub + threadIdx.x;
    int my[8];
    bb_mark(ids, t, t < T, k, E, bm, my);
    __syncthreads();
    for (int64_t e = threadIdx.x; e < E; e += BB_THREADS) run[e] += bb_bits(bm, E, e);
    __syncthreads();
  }
  for (int64_t e = threadIdx.x; e < E; e += BB_THREADS) slab_counts[slab * E + e] = run[e];
  bb_fill_pad(tp2id, NB, pad_id, slab, n_wg);
}

__global__ __launch_bounds__(BB_THREADS) void bb_count_kernel(const int32_t* __restrict__ ids, int64_t T, int64_t k,
                                                             int64_t E, int64_t slab_tokens,
                                                             int32_t* __restrict__ slab_counts,
                                                             int32_t* __restrict__ tp2id, int64_t NB, int pad_id) {
  extern __shared__ uint32_t bb_lds[];
  bb_count_body(ids, T, k, E, slab_tokens, slab_counts, tp2id, NB, pad_id, blockIdx.x, gridDim.x, bb_lds);
}

// ws layout: first_slot[E] | slab_counts[BB_SLABS_MAX][E]
// One workgroup: blocks per expert (padding blocks to the last expert, or split), exclusive scan ->
// first slot of every expert, block_to_expert, conditions; sums and scans over the experts are
// workgroup-wide (shuffles + one exchange), a tile of one expert per thread at a time.
__device__ __forceinline__ void bb_layout_body(const int32_t* __restrict__ slab_counts, int64_t n_slabs,
                                               int32_t* __restrict__ first_slot, int32_t* __restrict__ block_to_expert,
                                               int32_t* __restrict__ conditions, int64_t n_conditions, int64_t E,
                                               int64_t B, int64_t N, int use_split_padding,
                                               int32_t* __restrict__ status, int* s_nb, const BlockPlanOut plan) {
  // s_nb: [E] blocks per expert, then [E] first block of every expert, then [E] tokens of every expert
  int* s_first = s_nb + E;
  int* s_count = s_nb + 2 * E;
  const int64_t nthr = blockDim.x;  // 256 in the single launch of a small batch, 1024 in a launch of its own
  __shared__ int s_npad;
  __shared__ int s_ws[16];
  // blocks per expert and their sum
  int mine = 0;
  for (int64_t e = threadIdx.x; e < E; e += nthr) {
    int64_t count = 0;
#pragma unroll 8
    for (int64_t sl = 0; sl < n_slabs; ++sl) count += slab_counts[sl * E + e];
    const int nb = (int)((count + B - 1) / B);
    s_count[e] = (int)count;
    s_nb[e] = nb;
    mine += nb;
  }
  int used;
  (void)block_excl_scan(mine, s_ws, &used);
  if (threadIdx.x == 0) {
    int64_t npad = N - used;
    if (status) *status = npad < 0;
    if (npad < 0) npad = 0;
    s_npad = (int)npad;
    if (use_split_padding) {
      s_nb[(E - 1) / 2] += (int)(npad / 2);
      s_nb[E - 1] += (int)(npad - npad / 2);
    } else {
      s_nb[E - 1] += (int)npad;
    }
  }
  __syncthreads();
  // first block of every expert: exclusive scan over the experts, a tile of nthr at a time
  int carry = 0;
  for (int64_t base = 0; base < E; base += nthr) {
    const int64_t e = base + threadIdx.x;
    const int v = (e < E) ? s_nb[e] : 0;
    int total;
    const int ex = block_excl_scan(v, s_ws, &total);
    if (e < E) s_first[e] = carry + ex;
    carry += total;
  }
  __syncthreads();
  for (int64_t e = threadIdx.x; e < E; e += nthr) first_slot[e] = (int32_t)((int64_t)s_first[e] * B);
  // A block's expert is the last one whose first block is not beyond it (experts without blocks share their first
  // block with the next expert, so the last of equals is the one that owns the block).  A search per block: the
  // padding blocks of a small batch all belong to one expert, and a loop per expert would write them one by one.
  for (int64_t b = threadIdx.x; b < N; b += nthr) {
    int lo = 0, hi = (int)E;  // s_first[lo] <= b < s_first[hi]  (s_first[0] == 0, s_first[E] = infinity)
    while (hi - lo > 1) {
      const int mid = (lo + hi) >> 1;
      if (s_first[mid] <= b) lo = mid;
      else hi = mid;
    }
    block_to_expert[b] = lo;
    if (plan.valid_rows) {
      // tokens of expert lo less those in its earlier blocks
      const int64_t left = (int64_t)s_count[lo] - (b - s_first[lo]) * B;
      plan.valid_rows[b] = (int32_t)(left < 0 ? 0 : left > B ? B : left);
    }
  }
  if (plan.n_active && threadIdx.x == 0) *plan.n_active = (int32_t)(N - s_npad);
  if (conditions) {
    // ones, then zeros over the trailing (npad + n_conditions - N) entries
    const int64_t n_zero = s_npad + (n_conditions - N);
    for (int64_t i = threadIdx.x; i < n_conditions; i += nthr)
      conditions[i] = (i < n_conditions - n_zero) ? 1 : 0;
  }
  if (plan.chunks_inline) {
    // block_to_expert, the valid rows and the number of blocks in use were written by this workgroup
    __threadfence_block();
    __syncthreads();
    build_chunks(block_to_expert, plan.n_active, plan.valid_rows, N, B, E, plan.k.n_chunks, plan.k.chunk_slot,
                 plan.k.chunk_rows, plan.k.chunk_expert, plan.k.chunk_xcd, plan.k.q_chunk, plan.k.q_off,
                 plan.k.max_chunks, s_ws, false);
  }
}

__global__ __launch_bounds__(1024) void bb_layout_kernel(const int32_t* __restrict__ slab_counts, int64_t n_slabs,
                                                              int32_t* __restrict__ first_slot,
                                                              int32_t* __restrict__ block_to_expert,
                                                              int32_t* __restrict__ conditions, int64_t n_conditions,
                                                              int64_t E, int64_t B, int64_t N, int use_split_padding,
                                                              int32_t* __restrict__ status, const BlockPlanOut plan) {
  extern __shared__ int s_nb_dyn[];
  bb_layout_body(slab_counts, n_slabs, first_slot, block_to_expert, conditions, n_conditions, E, B, N,
                 use_split_padding, status, s_nb_dyn, plan);
}

// Workgroup = slab.  A token's slot for expert e: first slot of e + tokens of e in the slabs before (summed here
// from the slab counts) + tokens of e earlier in this slab.
__device__ __forceinline__ void bb_scatter_body(const int32_t* __restrict__ ids, int64_t T, int64_t k, int64_t E,
                                                int64_t slab_tokens, const int32_t* __restrict__ slab_counts,
                                                const int32_t* __restrict__ first_slot, int32_t* __restrict__ tp2id,
                                                int64_t NB, int64_t slab, uint32_t* bb_lds, const BlockPlanOut plan) {
  uint32_t* bm = bb_lds;
  int* run = (int*)(bb_lds + 8 * E);
  for (int64_t e = threadIdx.x; e < E; e += BB_THREADS) {
    int before = first_slot[e];
#pragma unroll 8
    for (int64_t sl = 0; sl < slab; ++sl) before += slab_counts[sl * E + e];
    run[e] = before;
  }
  const int64_t t_begin = slab * slab_tokens;
  const int wd = threadIdx.x >> 5;
  const uint32_t below = (1u << (threadIdx.x & 31)) - 1u;
  for (int64_t sub = 0; sub < slab_tokens && t_begin + sub < T; sub += BB_THREADS) {
    for (int64_t i = threadIdx.x; i < 8 * E; i += BB_THREADS) bm[i] = 0;
    __syncthreads();
    const int64_t t = t_begin + sub + threadIdx.x;
    const bool live = t < T;
    int my[8];
    bb_mark(ids, t, live, k, E, bm, my);
    __syncthreads();
    if (live) {
      // the slot of token t under expert e: the expert's first free slot + the tokens of e before t in this pass
      auto place = [&](int e) -> int32_t {
        if (e < 0 || e >= E) return -1;
        int r = __popc(bm[wd * E + e] & below);
        for (int w = 0; w < wd; ++w) r += __popc(bm[w * E + e]);
        const int64_t pos = (int64_t)run[e] + r;
        if (pos >= NB) return -1;
        tp2id[pos] = (int32_t)t;
        return (int32_t)pos;
      };
      // (for the plan: an id that the row lists twice owns one slot, the second mention adds nothing)
      if (k == 8) {
        int32_t slot[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) {
          slot[j] = place(my[j]);
#pragma unroll
          for (int j2 = 0; j2 < j; ++j2)
            if (my[j2] == my[j]) slot[j] = -1;
        }
        if (plan.list) {  // two 16-byte stores (the plan is 256-byte aligned)
          ((int4*)(plan.list + t * 8))[0] = make_int4(slot[0], slot[1], slot[2], slot[3]);
          ((int4*)(plan.list + t * 8))[1] = make_int4(slot[4], slot[5], slot[6], slot[7]);
        }
      } else {
        for (int64_t j = 0; j < k; ++j) {
          const int e = ids[t * k + j];
          int32_t slot = place(e);
          if (plan.list) {
            for (int64_t j2 = 0; j2 < j; ++j2)
              if (ids[t * k + j2] == e) slot = -1;
            plan.list[t * k + j] = slot;
          }
        }
      }
      if (plan.off) {
        plan.off[t] = (int32_t)(t * k);
        if (t == T - 1) plan.off[T] = (int32_t)(T * k);
      }
    }
    __syncthreads();
    for (int64_t e = threadIdx.x; e < E; e += BB_THREADS) run[e] += bb_bits(bm, E, e);
    __syncthreads();  // the bitmaps are cleared next
  }
}

__global__ __launch_bounds__(BB_THREADS) void bb_scatter_kernel(const int32_t* __restrict__ ids, int64_t T, int64_t k,
                                                               int64_t E, int64_t slab_tokens,
                                                               const int32_t* __restrict__ slab_counts,
                                                               const int32_t* __restrict__ first_slot,
                                                               int32_t* __restrict__ tp2id, int64_t NB,
                                                               const BlockPlanOut plan) {
  extern __shared__ uint32_t bb_lds[];
  bb_scatter_body(ids, T, k, E, slab_tokens, slab_counts, first_slot, tp2id, NB, blockIdx.x, bb_lds, plan);
}

// Few tokens (one slab): the three steps in one launch by one workgroup.  What one step leaves in global memory
// (the slab's counts, the first slots, the pad ids under the tokens' slots) the next reads or overwrites after a
// workgroup barrier: all of it goes through this CU's L1.
__global__ __launch_bounds__(BB_THREADS) void bb_single_slab_kernel(
    const int32_t* __restrict__ ids, int64_t T, int64_t k, int64_t E, int64_t slab_tokens,
    int32_t* __restrict__ slab_counts, int32_t* __restrict__ first_slot, int32_t* __restrict__ tp2id, int64_t NB,
    int pad_id, int32_t* __restrict__ block_to_expert, int32_t* __restrict__ conditions, int64_t n_conditions, int64_t B,
    int64_t N, int use_split_padding, int32_t* __restrict__ status, const BlockPlanOut plan) {
  extern __shared__ uint32_t bb_lds[];  // 9 E words of the count / scatter steps, then 3 E of the layout step
  bb_count_body(ids, T, k, E, slab_tokens, slab_counts, tp2id, NB, pad_id, 0, 1, bb_lds);
  __syncthreads();
  bb_layout_body(slab_counts, 1, first_slot, block_to_expert, conditions, n_conditions, E, B, N, use_split_padding,
                 status, (int*)(bb_lds + 9 * E), plan);
  __syncthreads();
  bb_scatter_body(ids, T, k, E, slab_tokens, slab_counts, first_slot, tp2id, NB, 0, bb_lds, plan);
}

}  // namespace moe

using namespace moe;

extern "C" size_t moe_build_blocks_workspace_bytes(int64_t E) {
  return (size_t)((1 + BB_SLABS_MAX) * E + 4) * sizeof(int32_t);
}

namespace {

// Shared by the two entry points: `ws` is device memory of at least moe_build_blocks_workspace_bytes(E) bytes,
// laid out as first_slot[E] | slab_counts[BB_SLABS_MAX][E].  Every word of it that a kernel reads was written
// earlier in the same call (the count step writes the counts of every slab it launches, the layout step every
// first slot), so stale contents of an earlier call are never seen and nothing has to be cleared.
int build_blocks_launch(const int32_t* topk_ids, int64_t T, int64_t k, int64_t E, int64_t B, int64_t N, int skip_token,
                        int use_split_padding, int32_t* token_position_to_id, int32_t* block_to_expert,
                        int32_t* conditions, int64_t n_conditions, int32_t* ws, int32_t* status_out, hipStream_t s,
                        BlockPlanOut plan = BlockPlanOut{}) {
  // at most BB_SLABS_MAX slabs of a multiple of 256 tokens
  int64_t slab_tokens = (T + BB_SLABS_MAX - 1) / BB_SLABS_MAX;
  slab_tokens = (slab_tokens + BB_THREADS - 1) / BB_THREADS * BB_THREADS;
  if (slab_tokens == 0) slab_tokens = BB_THREADS;
  if (T <= BB_SINGLE_MAX_TOKENS) slab_tokens = (T + BB_THREADS - 1) / BB_THREADS * BB_THREADS;  // one slab
  if (slab_tokens == 0) slab_tokens = BB_THREADS;
  int64_t n_slabs = (T + slab_tokens - 1) / slab_tokens;
  if (n_slabs == 0) n_slabs = 1;  // T == 0: one slab with no tokens still fills the pad ids
  int32_t* first_slot = ws;
  int32_t* slab_counts = first_slot + E;
  const size_t lds = (size_t)9 * E * sizeof(int32_t);
  const bool planned = plan.valid_rows != nullptr;
  if (n_slabs == 1 && N * B <= BB_SINGLE_MAX_SLOTS) {
    // (the chunk builder's tables are static LDS of the kernel: it runs in this launch while both fit in 64 KB)
    plan.chunks_inline = planned && lds + 3 * E * sizeof(int32_t) + BB_CHUNKS_STATIC_LDS <= 65536;
    hipLaunchKernelGGL(bb_single_slab_kernel, dim3(1), dim3(BB_THREADS), lds + 3 * E * sizeof(int32_t), s, topk_ids, T,
                       k, E, slab_tokens, slab_counts, first_slot, token_position_to_id, N * B,
                       skip_token ? -1 : (int)T, block_to_expert, conditions, n_conditions, B, N, use_split_padding,
                       status_out, plan);
    MOE_CHECK_LAUNCH();
    if (planned && !plan.chunks_inline) return launch_plan_chunks(plan.k, block_to_expert, N, B, E, s);
    return MOE_OK;
  }
  hipLaunchKernelGGL(bb_count_kernel, dim3((unsigned)n_slabs), dim3(BB_THREADS), lds, s, topk_ids, T, k, E, slab_tokens,
                     slab_counts, token_position_to_id, N * B, skip_token ? -1 : (int)T);
  MOE_CHECK_LAUNCH();
  plan.chunks_inline = planned;  // (3 E words of dynamic LDS beside the chunk builder's tables: E <= 1024 fits)
  hipLaunchKernelGGL(bb_layout_kernel, dim3(1), dim3(planned ? 1024 : BB_THREADS), 3 * E * sizeof(int), s, slab_counts, n_slabs,
                     first_slot, block_to_expert, conditions, n_conditions, E, B, N, use_split_padding, status_out,
                     plan);
  MOE_CHECK_LAUNCH();
  hipLaunchKernelGGL(bb_scatter_kernel, dim3((unsigned)n_slabs), dim3(BB_THREADS), lds, s, topk_ids, T, k, E,
                     slab_tokens, slab_counts, first_slot, token_position_to_id, N * B, plan);
  MOE_CHECK_LAUNCH();
  return MOE_OK;
}

int build_blocks_check(const int32_t* topk_ids, int64_t T, int64_t k, int64_t E, int64_t B, int64_t N,
                       const int32_t* token_position_to_id, const int32_t* block_to_expert, const int32_t* conditions,
                       int64_t n_conditions) {
  if (!topk_ids || !token_position_to_id || !block_to_expert) return MOE_E_BAD_ARG;
  if (T < 0 || k <= 0 || E <= 0 || B <= 0 || N <= 0) return MOE_E_BAD_ARG;
  if (conditions && n_conditions < N) return MOE_E_BAD_SHAPE;
  if (N * B >= (int64_t)1 << 31 || E > BB_E_MAX) return MOE_E_BAD_SHAPE;
  return MOE_OK;
}

// ---- the entry point that allocates nothing -------------------------------------------------------------
// Its scratch (first slots and per-slab counts, what moe_build_blocks takes as `workspace`) is a file-scope device
// array sized for MOE_BUILD_BLOCKS_STATIC_MAX_E experts.  Every GPU holds its own copy of the array at its own
// address for the life of the process; host code never uses the array's name as an address, only the per-device
// pointer obtained once from hipGetSymbolAddress with that device current.
}  // namespace

constexpr size_t BB_STATIC_BYTES = (size_t)((1 + BB_SLABS_MAX) * MOE_BUILD_BLOCKS_STATIC_MAX_E + 4) * sizeof(int32_t);
static_assert(BB_STATIC_BYTES == MOE_BUILD_BLOCKS_STATIC_BYTES, "the header states the size of the built-in scratch");
static_assert(MOE_BUILD_BLOCKS_STATIC_MAX_E <= BB_E_MAX, "the built-in scratch covers a subset of moe_build_blocks");
static __device__ __align__(256) unsigned char scratch[BB_STATIC_BYTES];

namespace {

constexpr int BB_MAX_DEVICES = 64;
std::mutex g_scratch_mutex;
void* g_scratch_ptr[BB_MAX_DEVICES];  // per device: address of that device's copy of `scratch`, null until first use

// The current device's scratch, looked up on the first call on that device.
int static_scratch(void** out) {
  int dev = -1;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= BB_MAX_DEVICES) return MOE_E_NO_DEVICE;
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  if (!g_scratch_ptr[dev]) {
    void* p = nullptr;
    if (hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)) != hipSuccess || !p) return MOE_E_LAUNCH;
    g_scratch_ptr[dev] = p;
  }
  *out = g_scratch_ptr[dev];
  return MOE_OK;
}

}  // namespace

namespace moe {
// Called by moe_check_device(): looks the current device's scratch up ahead of the first moe_build_blocks_static
// call, so that a caller who records that call into a graph has no symbol lookup inside the capture.
int build_blocks_static_setup() {
  void* p = nullptr;
  return static_scratch(&p);
}
}  // namespace moe

extern "C" int moe_build_blocks(const int32_t* topk_ids, int64_t T, int64_t k, int64_t E, int64_t B, int64_t N,
                                int skip_token, int use_split_padding, int32_t* token_position_to_id,
                                int32_t* block_to_expert, int32_t* conditions, int64_t n_conditions, void* workspace,
                                size_t workspace_bytes, int32_t* status_out, void* stream) {
  const int rc = build_blocks_check(topk_ids, T, k, E, B, N, token_position_to_id, block_to_expert, conditions, n_conditions);
  if (rc != MOE_OK) return rc;
  if (!workspace) return MOE_E_BAD_ARG;
  if (workspace_bytes < moe_build_blocks_workspace_bytes(E)) return MOE_E_WORKSPACE;
  return build_blocks_launch(topk_ids, T, k, E, B, N, skip_token, use_split_padding, token_position_to_id,
                             block_to_expert, conditions, n_conditions, (int32_t*)workspace, status_out,
                             (hipStream_t)stream);
}

extern "C" int moe_build_blocks_static(const int32_t* topk_ids, int64_t T, int64_t k, int64_t E, int64_t B, int64_t N,
                                       int skip_token, int use_split_padding, int32_t* token_position_to_id,
                                       int32_t* block_to_expert, int32_t* conditions, int64_t n_conditions,
                                       int32_t* status_out, void* stream) {
  int rc = build_blocks_check(topk_ids, T, k, E, B, N, token_position_to_id, block_to_expert, conditions, n_conditions);
  if (rc != MOE_OK) return rc;
  if (E > MOE_BUILD_BLOCKS_STATIC_MAX_E) return MOE_E_STATIC_LIMIT;  // checked before any device call
  void* ws = nullptr;
  rc = static_scratch(&ws);
  if (rc != MOE_OK) return rc;
  return build_blocks_launch(topk_ids, T, k, E, B, N, skip_token, use_split_padding, token_position_to_id,
                             block_to_expert, conditions, n_conditions, (int32_t*)ws, status_out, (hipStream_t)stream);
}

// ---- the block build that also hands the blockwise layer its bookkeeping ----------------------------------
extern "C" size_t moe_block_plan_bytes(int64_t T, int64_t B, int64_t N, int skip_token) {
  if (T < 1 || B <= 0 || N <= 0) return 0;
  return bookkeeping_bytes(skip_token ? T : T + 1, N, B);
}

extern "C" int moe_build_blocks_plan(const int32_t* topk_ids, int64_t T, int64_t k, int64_t E, int64_t B, int64_t N,
                                     int skip_token, int use_split_padding, int32_t* token_position_to_id,
                                     int32_t* block_to_expert, int32_t* conditions, int64_t n_conditions,
                                     void* workspace, size_t workspace_bytes, int32_t* status_out, void* plan,
                                     size_t plan_bytes, void* stream) {
  const int rc = build_blocks_check(topk_ids, T, k, E, B, N, token_position_to_id, block_to_expert, conditions, n_conditions);
  if (rc != MOE_OK) return rc;
  if (!workspace || !plan || ((uintptr_t)plan & 255) != 0) return MOE_E_BAD_ARG;
  // (split padding puts padding blocks in the middle of the list while `conditions` still ends with as many zeros:
  // which blocks run then depends on whether the caller passes `conditions`, which a plan cannot know)
  if (use_split_padding) return MOE_E_UNSUPPORTED;
  if (workspace_bytes < moe_build_blocks_workspace_bytes(E)) return MOE_E_WORKSPACE;
  // a plan lists T * k slots in the N * B words that the slot lists of the blockwise layer occupy
  if (T < 1 || T * k > N * B || E > COMBINE_MAX_K) return MOE_E_BAD_SHAPE;
  if (plan_bytes < moe_block_plan_bytes(T, B, N, skip_token)) return MOE_E_WORKSPACE;
  const Bookkeeping bk = carve_bookkeeping(plan, skip_token ? T : T + 1, N, B);
  BlockPlanOut out{};
  out.n_active = bk.n_active;
  out.valid_rows = bk.valid_rows;
  out.off = bk.off;
  out.list = bk.list;
  out.k = bk;
  return build_blocks_launch(topk_ids, T, k, E, B, N, skip_token, use_split_padding, token_position_to_id,
                             block_to_expert, conditions, n_conditions, (int32_t*)workspace, status_out,
                             (hipStream_t)stream, out);
}
