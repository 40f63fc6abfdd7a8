// Token -> block index construction on the GPU (integer, bit exact with the reference helper
// generate_token_position_to_id_and_experts,
// test/integration/nkilib/core/moe/moe_cte/test_moe_cte_common.py:199-264).
//
// A stable counting sort of the routed (token, expert) pairs by expert:
//   1. count_kernel    one workgroup per expert counts the tokens that selected it
//   2. layout_kernel   one workgroup: blocks per expert, padding blocks to the last expert (or
//                      split), exclusive scan -> first slot of every expert, block_to_expert,
//                      conditions, and the pad fill of token_position_to_id
//   3. scatter_kernel  one workgroup per expert ranks its tokens in ascending token id with a
//                      block-wide scan and writes their ids
// The work is latency bound (a few hundred KB of int32), so each step is a single small launch.
#include "common.hpp"

namespace moe {

constexpr int BB_THREADS = 256;

__device__ __forceinline__ int token_selects(const int32_t* ids, int64_t t, int64_t k, int e) {
  int hit = 0;
  for (int64_t j = 0; j < k; ++j) hit |= (ids[t * k + j] == e);
  return hit;
}

__global__ __launch_bounds__(BB_THREADS) void bb_count_kernel(const int32_t* __restrict__ ids, int64_t T, int64_t k,
                                                             int32_t* __restrict__ counts) {
  __shared__ int red[BB_THREADS / 64];
  const int e = blockIdx.x;
  int c = 0;
  for (int64_t t = threadIdx.x; t < T; t += BB_THREADS) c += token_selects(ids, t, k, e);
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) c += __shfl_xor(c, o, 64);
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = c;
  __syncthreads();
  if (threadIdx.x == 0) {
    int s = 0;
    for (int i = 0; i < BB_THREADS / 64; ++i) s += red[i];
    counts[e] = s;
  }
}

// ws layout: counts[E] | first_slot[E] | n_padding[1]
__global__ __launch_bounds__(BB_THREADS) void bb_layout_kernel(const int32_t* __restrict__ counts,
                                                              int32_t* __restrict__ first_slot,
                                                              int32_t* __restrict__ block_to_expert,
                                                              int32_t* __restrict__ conditions, int64_t n_conditions,
                                                              int32_t* __restrict__ tp2id, int64_t E, int64_t B,
                                                              int64_t N, int pad_id, int use_split_padding,
                                                              int32_t* __restrict__ status) {
  __shared__ int s_npad;
  __shared__ int s_bad;
  // Serial part: E is at most a few hundred.
  if (threadIdx.x == 0) {
    int64_t used = 0;
    for (int64_t e = 0; e < E; ++e) used += (counts[e] + B - 1) / B;
    int64_t npad = N - used;
    s_bad = npad < 0;
    if (npad < 0) npad = 0;
    s_npad = (int)npad;
    int64_t blk = 0;
    for (int64_t e = 0; e < E; ++e) {
      int64_t nb = (counts[e] + B - 1) / B;
      if (use_split_padding) {
        if (e == (E - 1) / 2) nb += npad / 2;
        if (e == E - 1) nb += npad - npad / 2;
      } else if (e == E - 1) {
        nb += npad;
      }
      first_slot[e] = (int32_t)(blk * B);
      for (int64_t j = 0; j < nb && blk + j < N; ++j) block_to_expert[blk + j] = (int32_t)e;
      blk += nb;
    }
    if (status) *status = s_bad;
  }
  __syncthreads();
  const int64_t npad = s_npad;
  if (conditions) {
    // ones, then zeros over the trailing (npad + n_conditions - N) entries
    const int64_t n_zero = npad + (n_conditions - N);
    for (int64_t i = threadIdx.x; i < n_conditions; i += BB_THREADS)
      conditions[i] = (i < n_conditions - n_zero) ? 1 : 0;
  }
  for (int64_t i = threadIdx.x; i < N * B; i += BB_THREADS) tp2id[i] = pad_id;
}

__global__ __launch_bounds__(BB_THREADS) void bb_scatter_kernel(const int32_t* __restrict__ ids, int64_t T, int64_t k,
                                                               const int32_t* __restrict__ first_slot,
                                                               int32_t* __restrict__ tp2id, int64_t NB) {
  __shared__ int wsum[BB_THREADS / 64];
  __shared__ int s_base;
  const int e = blockIdx.x;
  const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
  if (threadIdx.x == 0) s_base = first_slot[e];
  __syncthreads();
  for (int64_t t0 = 0; t0 < T; t0 += BB_THREADS) {
    const int64_t t = t0 + threadIdx.x;
    const int hit = (t < T) ? token_selects(ids, t, k, e) : 0;
    // inclusive scan of hit inside the wave
    int inc = hit;
#pragma unroll
    for (int o = 1; o < 64; o <<= 1) {
      int n = __shfl_up(inc, o, 64);
      if (lane >= o) inc += n;
    }
    if (lane == 63) wsum[w] = inc;
    __syncthreads();
    int before = 0, total = 0;
    for (int i = 0; i < BB_THREADS / 64; ++i) {
      if (i < w) before += wsum[i];
      total += wsum[i];
    }
    const int base = s_base;
    if (hit) {
      const int64_t pos = (int64_t)base + before + inc - 1;
      if (pos < NB) tp2id[pos] = (int32_t)t;
    }
    __syncthreads();
    if (threadIdx.x == 0) s_base = base + total;
    __syncthreads();
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
  hipLaunchKernelGGL(bb_count_kernel, dim3((unsigned)E), dim3(BB_THREADS), 0, s, topk_ids, T, k, counts);
  MOE_CHECK_LAUNCH();
  hipLaunchKernelGGL(bb_layout_kernel, dim3(1), dim3(BB_THREADS), 0, s, counts, first_slot, block_to_expert,
                     conditions, n_conditions, token_position_to_id, E, B, N, skip_token ? -1 : (int)T,
                     use_split_padding, status_out);
  MOE_CHECK_LAUNCH();
  hipLaunchKernelGGL(bb_scatter_kernel, dim3((unsigned)E), dim3(BB_THREADS), 0, s, topk_ids, T, k, first_slot,
                     token_position_to_id, N * B);
  MOE_CHECK_LAUNCH();
  return MOE_OK;
}
