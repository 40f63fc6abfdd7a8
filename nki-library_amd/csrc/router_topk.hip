// Router top-k front end for gfx950: logits = x @ w (+ bias), top-k selection, affinities.
//
// Semantics: router_topk_torch_ref, src/nkilib_src/nkilib/core/router_topk/router_topk_torch.py:23-135
// (kernel signature src/nkilib_src/nkilib/core/router_topk/router_topk.py:55-75).
//
// Two launches:
//   1. transpose_w_kernel   w [H,E] -> wt [E,H] (a few MB), so that both GEMM operands are contiguous
//                           along K, which is what an MFMA lane wants (8 consecutive K values);
//   2. router_kernel<NT,MT> a workgroup of 4 waves owns 64*MT tokens and all E = 16*NT experts.  Each wave
//                           multiplies its 16*MT tokens (fragments straight from global) with the
//                           K slice of wt that the workgroup stages in LDS, with
//                           v_mfma_f32_16x16x32_bf16 into MT*NT accumulator tiles, and then selects the top
//                           k per token without leaving registers: a token's E logits sit in 16 lanes x
//                           NT registers, so k rounds of (local argmax, 4-step lane reduction, retire the
//                           winner) pick them in descending order, ties to the lower expert index.
// Everything after the GEMM is fp32: softmax over all E (or over the k selected), sigmoid, the optional
// division by the sum of the selected values.
// For E <= 256 the K loop is software-pipelined (MT = 1): the 64-wide K slices of wt go global -> LDS
// directly into a ring of three stages (two steps ahead), XOR-swizzled on the global side so that the
// fragment reads are conflict free, and the token fragments into six register sets (five steps ahead:
// that stream comes from HBM); loads and waits are written as instructions (a wave's loads complete in
// issue order, so a wait names how many of the most recent ones may still be out), one barrier per
// step.  What bounds a step is what the CU's L1 can bring in: 40 KB per step and workgroup (the 32 KB slice
// of wt from L2, 8 KB of token rows), about 16 bytes per cycle.
#include <type_traits>

#include "common.hpp"

namespace moe {

constexpr int RT_THREADS = 256;
constexpr int RT_K = 64;         // K elements per LDS stage
constexpr int RT_PITCH = RT_K + 8;  // bf16 elements per staged row of wt (16-byte aligned, conflict-spreading pad)

__global__ __launch_bounds__(256) void transpose_w_kernel(const uint16_t* __restrict__ w, uint16_t* __restrict__ wt,
                                                          int64_t H, int64_t E) {
  __shared__ uint16_t tile[32][33];
  const int64_t h0 = (int64_t)blockIdx.x * 32, e0 = (int64_t)blockIdx.y * 32;
  const int tx = threadIdx.x & 31, ty = threadIdx.x >> 5;
  for (int r = ty; r < 32; r += 8) {
    const int64_t h = h0 + r, e = e0 + tx;
    tile[r][tx] = (h < H && e < E) ? w[h * E + e] : (uint16_t)0;
  }
  __syncthreads();
  for (int r = ty; r < 32; r += 8) {
    const int64_t e = e0 + r, h = h0 + tx;
    if (e < E && h < H) wt[e * H + h] = tile[tx][r];
  }
}

__global__ __launch_bounds__(256) void fill_zero_bytes_kernel(uint8_t* __restrict__ p, int64_t n) {
  for (int64_t i = threadIdx.x; i < n; i += 256) p[i] = 0;
}

struct RouterArgs {
  const uint16_t* x;   // bf16 [T, H]
  const uint16_t* wt;  // bf16 [E, H]
  const void* bias;    // [E] or null
  int bias_dtype;
  int64_t T, H, E;
  int k, act_fn, pre_norm, norm_topk, mask_to_topk;
  void* logits_out;    // [T, E] or null
  int logits_dtype;
  int32_t* index_out;  // [T, k] or null
  void* aff_out;       // [T (+1), E]
  int aff_dtype;
  float* topk_aff_out; // [T, k] or null
};

__device__ __forceinline__ void store_val(void* p, int dtype, int64_t i, float v) {
  if (dtype == MOE_DT_BF16) ((uint16_t*)p)[i] = f32_to_bf16_bits(v);
  else ((float*)p)[i] = v;
}

// max / sum over the 16 lanes that share a token row (lanes with equal lane >> 4)
__device__ __forceinline__ float row16_max(float v) {
#pragma unroll
  for (int o = 1; o < 16; o <<= 1) v = fmaxf(v, __shfl_xor(v, o, 64));
  return v;
}
__device__ __forceinline__ float row16_sum(float v) {
#pragma unroll
  for (int o = 1; o < 16; o <<= 1) v += __shfl_xor(v, o, 64);
  return v;
}

template <int I, int N, class F>
__device__ __forceinline__ void rt_static_for(F&& f) {
  if constexpr (I < N) {
    f(std::integral_constant<int, I>{});
    rt_static_for<I + 1, N>(f);
  }
}
__device__ __forceinline__ int rt_uni(int v) { return __builtin_amdgcn_readfirstlane(v); }
__device__ __forceinline__ v4i rt_rsrc(const void* p, uint32_t bytes) {
  const uint64_t addr = (uint64_t)p;
  v4i d;
  d[0] = rt_uni((int)(uint32_t)addr);
  d[1] = rt_uni((int)(uint32_t)(addr >> 32)) & 0xffff;
  d[2] = rt_uni((int)bytes);
  d[3] = 0x00020000;
  return d;
}
// (s_nop 4: a scalar operand that a vector instruction has just written -- the compiler reloads spilled scalars
// with v_readlane -- must not be read by a memory instruction within the next few cycles, and the compiler does
// not know that these statements are memory instructions)
__device__ __forceinline__ void rt_ld_lds(uint32_t lds, uint32_t voff, const v4i& rsrc, int soff) {
  asm volatile("s_nop 4\n\ts_mov_b32 m0, %0\n\tbuffer_load_dwordx4 %1, %2, %3 offen lds"
               : : "s"(lds), "v"(voff), "s"(rsrc), "s"(soff) : "memory", "m0");
}
__device__ __forceinline__ void rt_ld(v4i& d, uint32_t voff, const v4i& rsrc, int soff) {
  asm volatile("s_nop 4\n\tbuffer_load_dwordx4 %0, %1, %2, %3 offen" : "+v"(d) : "v"(voff), "s"(rsrc), "s"(soff) : "memory");
}

template <int NT, int MT, bool PIPE>
__global__ __launch_bounds__(RT_THREADS) void router_kernel(const RouterArgs a) {
  extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
  uint16_t* sW = (uint16_t*)smem;  // [16*NT][RT_PITCH]
  const int tid = threadIdx.x, lane = tid & 63, w = tid >> 6;
  const int c = lane & 15, g = lane >> 4;
  const int64_t t0 = (int64_t)blockIdx.x * (64 * MT) + w * (16 * MT);
  constexpr int EP = 16 * NT;  // experts covered by this instantiation (>= a.E)

  v4f acc[MT][NT];
#pragma unroll
  for (int m = 0; m < MT; ++m)
#pragma unroll
    for (int n = 0; n < NT; ++n) acc[m][n] = (v4f){0.f, 0.f, 0.f, 0.f};

  const int nsteps = (int)(a.H / RT_K);
  if constexpr (!PIPE) {
  // A rows: lane (c, g) of row tile m reads token t0 + 16m + c, K elements 8g .. 8g+7 of each 32-wide step
  const uint16_t* xr[MT];
#pragma unroll
  for (int m = 0; m < MT; ++m) {
    int64_t t = t0 + 16 * m + c;
    if (t >= a.T) t = a.T - 1;  // rows past the end repeat the last token; nothing is written for them
    xr[m] = a.x + t * a.H + 8 * g;
  }
  for (int s = 0; s < nsteps; ++s) {
    const int64_t k0 = (int64_t)s * RT_K;
    __syncthreads();
    // stage wt[:, k0 .. k0+63]: 16*NT rows of 128 bytes, 8 chunks of 16 bytes each
    for (int i = tid; i < EP * 8; i += RT_THREADS) {
      const int e = i >> 3, ch = i & 7;
      v4i v = {0, 0, 0, 0};
      if (e < a.E) v = *(const v4i*)(a.wt + (int64_t)e * a.H + k0 + ch * 8);
      *(v4i*)(sW + e * RT_PITCH + ch * 8) = v;
    }
    __syncthreads();
#pragma unroll
    for (int kk = 0; kk < 2; ++kk) {
      v8bf af[MT];
#pragma unroll
      for (int m = 0; m < MT; ++m) af[m] = *(const v8bf*)(xr[m] + k0 + kk * 32);
#pragma unroll
      for (int n = 0; n < NT; ++n) {
        const v8bf bf = *(const v8bf*)(sW + (n * 16 + c) * RT_PITCH + kk * 32 + 8 * g);
#pragma unroll
        for (int m = 0; m < MT; ++m) acc[m][n] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(af[m], bf, acc[m][n], 0, 0, 0);
      }
    }
  }
  } else {
    static_assert(MT == 1, "the pipelined loop handles one row tile per wave");
    constexpr int STAGE = EP * 128;       // bytes of one K slice of wt in LDS (row pitch 128 bytes)
    constexpr int NI = EP * 8 / RT_THREADS;  // 16-byte pieces of a slice per thread
    constexpr int NL = NI + 2;            // loads per step and wave: NI weight pieces + 2 token fragments
    const uint32_t lds0 = (uint32_t)(uintptr_t)smem;
    const int wu = rt_uni(w);
    // weight pieces: wave instruction i covers 8 rows x 128 bytes; lane l fills slot l&7 of row 8(NI w + i) + (l>>3)
    // with the global chunk slot ^ (row & 7)
    uint32_t w_voff[NI];
#pragma unroll
    for (int i = 0; i < NI; ++i) {
      int row = 8 * (NI * w + i) + (lane >> 3);
      const int ch = (lane & 7) ^ ((row >> 1) & 7);
      if (row >= a.E) row = (int)a.E - 1;  // padding rows repeat the last expert; their logits are never used
      w_voff[i] = (uint32_t)(row * a.H * 2 + ch * 16);
    }
    int64_t t = t0 + c;
    if (t >= a.T) t = a.T - 1;  // rows past the end repeat the last token; nothing is written for them
    const uint32_t x_voff = (uint32_t)(t * a.H * 2 + g * 16);
    const v4i rw_ = rt_rsrc(a.wt, (uint32_t)(a.E * a.H * 2)), rx_ = rt_rsrc(a.x, (uint32_t)(a.T * a.H * 2));
    // rings: three LDS stages of wt (loads two steps ahead, L2 hits), RA register sets of token fragments
    // (loads RA-1 steps ahead: this is the stream that comes from HBM, and what is in flight bounds its rate)
    constexpr int RA = 6;
    v4i af[RA][2];
#pragma unroll
    for (int u = 0; u < RA; ++u) af[u][0] = af[u][1] = (v4i){0, 0, 0, 0};
    // descriptors of zero records past the end: no traffic, zeros
    auto issue_w = [&](int s, int stage) {
      v4i rw;
      rw[0] = rt_uni(rw_[0]); rw[1] = rt_uni(rw_[1]); rw[2] = rt_uni(s < nsteps ? rw_[2] : 0); rw[3] = rt_uni(rw_[3]);
      const int koff = rt_uni(s * RT_K * 2);
      const uint32_t lds = rt_uni((int)(lds0 + (uint32_t)stage * STAGE + (uint32_t)(NI * wu) * 1024));
#pragma unroll
      for (int i = 0; i < NI; ++i) rt_ld_lds(lds + i * 1024, w_voff[i], rw, koff);
    };
    auto issue_a = [&](int s, v4i& f0, v4i& f1) {
      v4i rx;
      rx[0] = rt_uni(rx_[0]); rx[1] = rt_uni(rx_[1]); rx[2] = rt_uni(s < nsteps ? rx_[2] : 0); rx[3] = rt_uni(rx_[3]);
      const int koff = rt_uni(s * RT_K * 2);
      rt_ld(f0, x_voff, rx, koff);
      rt_ld(f1, x_voff, rx, koff + 64);
    };
    const int rd0 = c * 128;  // fragment reads: row n*16 + c, chunk 4 kk + g, swizzled
    auto step = [&](auto u_, int s) {
      constexpr int U = decltype(u_)::value, stage = U % 3;
      // out at most: the fragments issued in step s-2 and everything of step s-1
      asm volatile("s_waitcnt vmcnt(%0)" : : "n"(NI + 4) : "memory");
      asm volatile("" : "+v"(af[U][0]), "+v"(af[U][1]));
      __syncthreads();  // every wave's pieces of this step are in; every wave has left step s-1
      // into the stage and the registers that step s-1 read
      issue_w(s + 2, (stage + 2) % 3);
      issue_a(s + RA - 1, af[(U + RA - 1) % RA][0], af[(U + RA - 1) % RA][1]);
      const v8bf a0 = __builtin_bit_cast(v8bf, af[U][0]), a1 = __builtin_bit_cast(v8bf, af[U][1]);
      const uint8_t* base = smem + stage * STAGE + rd0;
#pragma unroll
      for (int n = 0; n < NT; ++n) {
        const v8bf b0 = *(const v8bf*)(base + n * 16 * 128 + ((g ^ ((c >> 1) & 7)) * 16));
        const v8bf b1 = *(const v8bf*)(base + n * 16 * 128 + (((4 + g) ^ ((c >> 1) & 7)) * 16));
        acc[0][n] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a0, b0, acc[0][n], 0, 0, 0);
        acc[0][n] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a1, b1, acc[0][n], 0, 0, 0);
      }
      // instruction order of the step: 8 fragment reads ahead, then 2 reads per 2 MFMAs, so that no
      // MFMA waits for the LDS round trip of its own operand (one wave per SIMD has no other cover)
      __builtin_amdgcn_sched_group_barrier(0x100, 8, 0);
#pragma unroll
      for (int i = 0; i < NT - 4; ++i) {
        __builtin_amdgcn_sched_group_barrier(0x008, 2, 0);
        __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);
      }
      __builtin_amdgcn_sched_group_barrier(0x008, 8, 0);
    };
    // prologue in the order the steps before the first would have issued
    issue_a(0, af[0][0], af[0][1]);
    issue_a(1, af[1][0], af[1][1]);
    issue_a(2, af[2][0], af[2][1]);
    issue_w(0, 0);
    issue_a(3, af[3][0], af[3][1]);
    issue_w(1, 1);
    issue_a(4, af[4][0], af[4][1]);
    int s = 0;
    for (; s + RA <= nsteps; s += RA)
      rt_static_for<0, RA>([&](auto u) { step(u, s + decltype(u)::value); });
    rt_static_for<0, RA - 1>([&](auto u) {
      if (s + decltype(u)::value < nsteps) step(u, s + decltype(u)::value);
    });
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    // the loads past the end still arrive (as zeros): their registers stay reserved until here
#pragma unroll
    for (int u = 0; u < RA; ++u) asm volatile("" : : "v"(af[u][0]), "v"(af[u][1]));
  }

  // ---- epilogue: per token (row tile m, row 4g + r); the lane's experts are n*16 + c --------------
  float bias[NT];
#pragma unroll
  for (int n = 0; n < NT; ++n) {
    const int e = n * 16 + c;
    bias[n] = (a.bias && e < a.E) ? load_as_f32(a.bias, a.bias_dtype, e) : 0.f;
  }
  const float NEG = -__builtin_inff();
#pragma unroll
  for (int m = 0; m < MT; ++m) {
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const int64_t t = t0 + 16 * m + 4 * g + r;
      const bool live = t < a.T;  // uniform over the 16 lanes of the row
      float v[NT];
#pragma unroll
      for (int n = 0; n < NT; ++n) v[n] = (n * 16 + c < a.E) ? acc[m][n][r] + bias[n] : NEG;
      if (a.logits_out && live) {
#pragma unroll
        for (int n = 0; n < NT; ++n)
          if (n * 16 + c < a.E) store_val(a.logits_out, a.logits_dtype, t * a.E + n * 16 + c, v[n]);
      }
      // full activation (pre-norm pipeline)
      float fullv[NT];
      if (a.pre_norm) {
        if (a.act_fn == 1) {  // softmax over all experts
          float mx = NEG;
#pragma unroll
          for (int n = 0; n < NT; ++n) mx = fmaxf(mx, v[n]);
          mx = row16_max(mx);
          float sum = 0.f;
#pragma unroll
          for (int n = 0; n < NT; ++n) {
            fullv[n] = (v[n] == NEG) ? 0.f : expf(v[n] - mx);
            sum += fullv[n];
          }
          sum = row16_sum(sum);
#pragma unroll
          for (int n = 0; n < NT; ++n) fullv[n] = fullv[n] / sum;
        } else {
#pragma unroll
          for (int n = 0; n < NT; ++n) fullv[n] = 1.0f / (1.0f + expf(-v[n]));
        }
      }
      // k rounds of argmax, ties to the lower expert index
      unsigned taken = 0;  // bit n: the lane's expert n*16 + c has been selected
      float selv[8];
      int seli[8];
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        selv[j] = 0.f;
        seli[j] = 0;
      }
      for (int j = 0; j < a.k; ++j) {
        float bv = NEG;
        int bi = 0x7fffffff;
#pragma unroll
        for (int n = 0; n < NT; ++n) {
          const bool free_ = !((taken >> n) & 1u) && (n * 16 + c < a.E);
          if (free_ && v[n] > bv) {  // ascending n: the lower index wins ties inside the lane
            bv = v[n];
            bi = n * 16 + c;
          }
        }
#pragma unroll
        for (int o = 1; o < 16; o <<= 1) {
          const float ov = __shfl_xor(bv, o, 64);
          const int oi = __shfl_xor(bi, o, 64);
          if (ov > bv || (ov == bv && oi < bi)) {
            bv = ov;
            bi = oi;
          }
        }
        if ((bi & 15) == c && bi < (int)a.E) taken |= 1u << (bi >> 4);
#pragma unroll
        for (int jj = 0; jj < 8; ++jj)
          if (jj == j) {
            selv[jj] = bv;
            seli[jj] = bi;
          }
      }
      // affinities of the selected experts
      float affk[8];
      if (a.pre_norm) {
        float ssum = 0.f;
#pragma unroll
        for (int n = 0; n < NT; ++n) ssum += ((taken >> n) & 1u) ? fullv[n] : 0.f;
        ssum = row16_sum(ssum);
#pragma unroll
        for (int n = 0; n < NT; ++n) {
          float o = fullv[n];
          if (a.norm_topk) o = ((taken >> n) & 1u) ? fullv[n] / ssum : 0.f;
          else if (a.mask_to_topk) o = ((taken >> n) & 1u) ? fullv[n] : 0.f;
          fullv[n] = o;
        }
      } else {
        // activate the k selected logits only
        float mx = selv[0], sum = 0.f;
#pragma unroll
        for (int j = 0; j < 8; ++j)
          if (j < a.k) {
            affk[j] = (a.act_fn == 1) ? expf(selv[j] - mx) : 1.0f / (1.0f + expf(-selv[j]));
            sum += affk[j];
          }
#pragma unroll
        for (int n = 0; n < NT; ++n) fullv[n] = 0.f;
#pragma unroll
        for (int j = 0; j < 8; ++j)
          if (j < a.k) {
            if (a.act_fn == 1) affk[j] = affk[j] / sum;
            if ((seli[j] & 15) == c) {
#pragma unroll
              for (int n = 0; n < NT; ++n)
                if (n == (seli[j] >> 4)) fullv[n] = affk[j];
            }
          }
      }
      if (live) {
#pragma unroll
        for (int n = 0; n < NT; ++n)
          if (n * 16 + c < a.E) store_val(a.aff_out, a.aff_dtype, t * a.E + n * 16 + c, fullv[n]);
        if (c == 0) {
          for (int j = 0; j < a.k; ++j) {
            if (a.index_out) a.index_out[t * a.k + j] = seli[j];
          }
        }
        if (a.topk_aff_out) {
          // the lane that owns the selected expert knows its final affinity
#pragma unroll
          for (int j = 0; j < 8; ++j)
            if (j < a.k && (seli[j] & 15) == c) {
#pragma unroll
              for (int n = 0; n < NT; ++n)
                if (n == (seli[j] >> 4)) a.topk_aff_out[t * a.k + j] = fullv[n];
            }
        }
      }
    }
  }
}

template <int NT, int MT, bool PIPE>
static int launch_router(const RouterArgs& a, hipStream_t s) {
  const unsigned grid = (unsigned)((a.T + 64 * MT - 1) / (64 * MT));
  const size_t lds = PIPE ? (size_t)3 * 16 * NT * 128 : (size_t)16 * NT * RT_PITCH * 2;
  hipError_t err = hipFuncSetAttribute((const void*)router_kernel<NT, MT, PIPE>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
  if (err != hipSuccess) return MOE_E_LAUNCH;
  hipLaunchKernelGGL((router_kernel<NT, MT, PIPE>), dim3(grid), dim3(RT_THREADS), lds, s, a);
  MOE_CHECK_LAUNCH();
  return MOE_OK;
}

}  // namespace moe

using namespace moe;

extern "C" size_t moe_router_topk_workspace_bytes(int64_t H, int64_t E) { return (size_t)(H * E * 2 + 256); }

extern "C" int moe_router_topk(const void* x, const void* w, const void* w_bias, int bias_dtype, int64_t T, int64_t H,
                               int64_t E, int k, int act_fn, int router_pre_norm, int norm_topk_prob, int mask_to_topk,
                               int pad_row, void* router_logits, int logits_dtype, int32_t* expert_index,
                               void* expert_affinities, int aff_dtype, float* topk_affinities, void* workspace,
                               size_t workspace_bytes, void* stream) {
  if (!x || !w || !expert_affinities || !workspace) return MOE_E_BAD_ARG;
  if (T < 0 || H <= 0 || E <= 0 || k <= 0 || k > 8 || k > E) return MOE_E_BAD_ARG;
  if (act_fn != 0 && act_fn != 1) return MOE_E_BAD_ARG;
  if (H % RT_K != 0 || E > 512) return MOE_E_BAD_SHAPE;
  if (aff_dtype != MOE_DT_BF16 && aff_dtype != MOE_DT_FP32) return MOE_E_BAD_ARG;
  if (router_logits && logits_dtype != MOE_DT_BF16 && logits_dtype != MOE_DT_FP32) return MOE_E_BAD_ARG;
  if (w_bias && bias_dtype != MOE_DT_BF16 && bias_dtype != MOE_DT_FP32 && bias_dtype != MOE_DT_FP16) return MOE_E_BAD_ARG;
  if (workspace_bytes < moe_router_topk_workspace_bytes(H, E)) return MOE_E_WORKSPACE;
  hipStream_t s = (hipStream_t)stream;
  if (pad_row) {
    // row T of the affinity table is the padding token's: zeros (E elements)
    const int64_t n = E * (aff_dtype == MOE_DT_BF16 ? 2 : 4);
    hipLaunchKernelGGL(fill_zero_bytes_kernel, dim3(1), dim3(256), 0, s,
                       (uint8_t*)expert_affinities + T * n, n);
    MOE_CHECK_LAUNCH();
  }
  if (T == 0) return MOE_OK;
  uint16_t* wt = (uint16_t*)workspace;
  hipLaunchKernelGGL(transpose_w_kernel, dim3((unsigned)((H + 31) / 32), (unsigned)((E + 31) / 32)), dim3(256), 0, s,
                     (const uint16_t*)w, wt, H, E);
  MOE_CHECK_LAUNCH();
  RouterArgs a;
  a.x = (const uint16_t*)x; a.wt = wt; a.bias = w_bias; a.bias_dtype = bias_dtype;
  a.T = T; a.H = H; a.E = E; a.k = k; a.act_fn = act_fn; a.pre_norm = router_pre_norm; a.norm_topk = norm_topk_prob;
  a.mask_to_topk = mask_to_topk;
  a.logits_out = router_logits; a.logits_dtype = logits_dtype; a.index_out = expert_index;
  a.aff_out = expert_affinities; a.aff_dtype = aff_dtype; a.topk_aff_out = topk_affinities;
  // the pipelined kernel addresses x and wt with 32-bit byte offsets
  const bool small = T * H * 2 < ((int64_t)1 << 31) && E * H * 2 < ((int64_t)1 << 31);
  if (E <= 128) return small ? launch_router<8, 1, true>(a, s) : launch_router<8, 2, false>(a, s);
  if (E <= 256) return small ? launch_router<16, 1, true>(a, s) : launch_router<16, 2, false>(a, s);
  return launch_router<32, 2, false>(a, s);
}
