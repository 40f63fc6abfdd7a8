// Token -> block index construction on the GPU (integer, bit exact with the reference helper
// generate_token_position_to_id_and_experts,
// test/integration/nkilib/core/moe/moe_cte/test_moe_cte_common.py:199-264).
//
// A stable counting sort of the routed (token, expert) pairs by expert:
//   1. count_kernel    one workgroup per expert counts the tokens that selected it; the grid also
//                      fills token_position_to_id with the pad id
//   2. layout_kernel   one workgroup: blocks per expert, padding blocks to the last expert (or
//                      split), exclusive scan -> first slot of every expert, block_to_expert,
//                      conditions
//   3. scatter_kernel  one workgroup per expert ranks its tokens in ascending token id with a
//                      block-wide scan and writes their ids
// The work is latency bound (a few hundred KB of int32), so each step is a single small launch.
#include "common.hpp"

namespace moe {

constexpr int BB_THREADS = 256;

// 1 if token t lists expert e among its k choices.  k == 8 (two 16-byte loads) is the common case.
__device__ __forceinline__ int token_selects(const int32_t* ids, int64_t t, int64_t k, int e) {
  if (k == 8) {
    const int4 a = ((const int4*)(ids + t * 8))[0], b = ((const int4*)(ids + t * 8))[1];
    return (a.x == e) | (a.y == e) | (a.z == e) | (a.w == e) | (b.x == e) | (b.y == e) | (b.z == e) | (b.w == e);
  }
  int hit = 0;
  for (int64_t j = 0; j < k; ++j) hit |= (ids[t * k + j] == e);
  return hit;
}

// One workgroup per expert counts its tokens (a ballot and a population count per 64 tokens); all
// workgroups together also fill token_position_to_id with the pad id, which the scatter overwrites
// where tokens sit.
__global__ __launch_bounds__(BB_THREADS) void bb_count_kernel(const int32_t* __restrict__ ids, int64_t T, int64_t k,
                                                             int32_t* __restrict__ counts,
                                                             int32_t* __restrict__ tp2id, int64_t NB, int pad_id) {
  __shared__ int red[BB_THREADS / 64];
  const int e = blockIdx.x;
  int c = 0;
  for (int64_t t0 = 0; t0 < T; t0 += BB_THREADS) {
    const int64_t t = t0 + threadIdx.x;
    const int hit = (t < T) ? token_selects(ids, t, k, e) : 0;
    c += __popcll(__ballot(hit));
  }
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = c;
  __syncthreads();
  if (threadIdx.x == 0) {
    int s = 0;
    for (int i = 0; i < BB_THREADS / 64; ++i) s += red[i];
    counts[e] = s;
  }
  for (int64_t i = (int64_t)blockIdx.x * BB_THREADS + threadIdx.x; i < NB; i += (int64_t)gridDim.x * BB_THREADS)
    tp2id[i] = pad_id;
}

// ws layout: counts[E] | first_slot[E] | n_padding[1]
// One workgroup: blocks per expert (padding blocks to the last expert, or split), exclusive scan ->
// first slot of every expert, block_to_expert, conditions; sums and scans over the experts are
// workgroup-wide (shuffles + one exchange), a tile of BB_THREADS experts at a time.
__global__ __launch_bounds__(BB_THREADS) void bb_layout_kernel(const int32_t* __restrict__ counts,
                                                              int32_t* __restrict__ first_slot,
                                                              int32_t* __restrict__ block_to_expert,
                                                              int32_t* __restrict__ conditions, int64_t n_conditions,
                                                              int64_t E, int64_t B, int64_t N, int use_split_padding,
                                                              int32_t* __restrict__ status) {
  extern __shared__ int s_nb[];  // [E] blocks per expert, then [E] first block of every expert
  int* s_first = s_nb + E;
  __shared__ int s_npad;
  __shared__ int s_ws[16];
  // blocks per expert and their sum
  int mine = 0;
  for (int64_t e = threadIdx.x; e < E; e += BB_THREADS) {
    const int nb = (int)((counts[e] + B - 1) / B);
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
  // first block of every expert: exclusive scan over the experts, a tile of BB_THREADS at a time
  int carry = 0;
  for (int64_t base = 0; base < E; base += BB_THREADS) {
    const int64_t e = base + threadIdx.x;
    const int v = (e < E) ? s_nb[e] : 0;
    int total;
    const int ex = block_excl_scan(v, s_ws, &total);
    if (e < E) s_first[e] = carry + ex;
    carry += total;
  }
  __syncthreads();
  for (int64_t e = threadIdx.x; e < E; e += BB_THREADS) {
    const int64_t blk = s_first[e];
    first_slot[e] = (int32_t)(blk * B);
    for (int64_t j = 0; j < s_nb[e] && blk + j < N; ++j) block_to_expert[blk + j] = (int32_t)e;
  }
  if (conditions) {
    // ones, then zeros over the trailing (npad + n_conditions - N) entries
    const int64_t n_zero = s_npad + (n_conditions - N);
    for (int64_t i = threadIdx.x; i < n_conditions; i += BB_THREADS)
      conditions[i] = (i < n_conditions - n_zero) ? 1 : 0;
  }
}

// One workgroup per expert ranks its tokens in ascending token id (ballot + population count below
// the lane, plus the counts of the waves before) and writes their ids.
__global__ __launch_bounds__(BB_THREADS) void bb_scatter_kernel(const int32_t* __restrict__ ids, int64_t T, int64_t k,
                                                               const int32_t* __restrict__ first_slot,
                                                               int32_t* __restrict__ tp2id, int64_t NB) {
  __shared__ int wsum[2][BB_THREADS / 64];
  const int e = blockIdx.x;
  const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
  int base = first_slot[e];
  int buf = 0;
  for (int64_t t0 = 0; t0 < T; t0 += BB_THREADS, buf ^= 1) {
    const int64_t t = t0 + threadIdx.x;
    const int hit = (t < T) ? token_selects(ids, t, k, e) : 0;
    const unsigned long long m = __ballot(hit);
    const int below = __popcll(m & ((1ull << lane) - 1ull));
    if (lane == 0) wsum[buf][w] = __popcll(m);
    __syncthreads();  // wsum[buf] is rewritten two iterations later, after the next barrier
    int before = 0, total = 0;
#pragma unroll
    for (int i = 0; i < BB_THREADS / 64; ++i) {
      const int v = wsum[buf][i];
      before += (i < w) ? v : 0;
      total += v;
    }
    if (hit) {
      const int64_t pos = (int64_t)base + before + below;
      if (pos < NB) tp2id[pos] = (int32_t)t;
    }
    base += total;
  }
}

}  // namespace moe

using namespace moe;

extern "C" size_t moe_build_blocks_workspace_bytes(int64_t E) { return (size_t)(2 * E + 4) * sizeof(int32_t); }

extern "C" int moe_build_blocks(const int32_t* topk_ids, int64_t T, int64_t k, int64_t E, int64_t B, int64_t N,
                                int skip_token, int use_split_padding, int32_t* token_position_to_id,
                                int32_t* block_to_expert, int32_t* conditions, int64_t n_conditions, void* workspace,
                                size_t workspace_bytes, int32_t* status_out, void* stream) {
  if (!topk_ids || !token_position_to_id || !block_to_expert || !workspace) return MOE_E_BAD_ARG;
  if (T < 0 || k <= 0 || E <= 0 || B <= 0 || N <= 0) return MOE_E_BAD_ARG;
  if (conditions && n_conditions < N) return MOE_E_BAD_SHAPE;
  if (workspace_bytes < moe_build_blocks_workspace_bytes(E)) return MOE_E_WORKSPACE;
  if (N * B >= (int64_t)1 << 31) return MOE_E_BAD_SHAPE;
  int32_t* counts = (int32_t*)workspace;
  int32_t* first_slot = counts + E;
  hipStream_t s = (hipStream_t)stream;
  hipLaunchKernelGGL(bb_count_kernel, dim3((unsigned)E), dim3(BB_THREADS), 0, s, topk_ids, T, k, counts,
                     token_position_to_id, N * B, skip_token ? -1 : (int)T);
  MOE_CHECK_LAUNCH();
  if (2 * E * sizeof(int) > 48 * 1024) return MOE_E_BAD_SHAPE;
  hipLaunchKernelGGL(bb_layout_kernel, dim3(1), dim3(BB_THREADS), 2 * E * sizeof(int), s, counts, first_slot,
                     block_to_expert, conditions, n_conditions, E, B, N, use_split_padding, status_out);
  MOE_CHECK_LAUNCH();
  hipLaunchKernelGGL(bb_scatter_kernel, dim3((unsigned)E), dim3(BB_THREADS), 0, s, topk_ids, T, k, first_slot,
                     token_position_to_id, N * B);
  MOE_CHECK_LAUNCH();
  return MOE_OK;
}
