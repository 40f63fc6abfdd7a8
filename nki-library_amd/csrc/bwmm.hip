// Blockwise expert GEMMs for gfx950: gate/up projection with fused act(gate)*up (stage 1) and
// down projection with fused bias / affinity (stage 2), for three precisions:
//   BF16     v_mfma_f32_16x16x32_bf16, weights bf16 or fp8 (+ per-channel fp32 scale)
//   FP8_ROW  v_mfma_scale_f32_16x16x128_f8f6f4 with unit block scales; per-row activation and
//            per-channel weight scales applied to the fp32 accumulators
//   MXFP8    v_mfma_scale_f32_16x16x128_f8f6f4, E8M0 block scales of both operands applied by
//            the matrix core
// This file holds the general tiled kernel: a 256-thread workgroup owns 128 rows of one block
// (one expert) and 128 output columns (256 in stage 1: gate and up), stages one 128-byte
// K-slice of both operands in LDS in K-contiguous order and lets each of the four waves run
// 2 x (8|16) MFMA tiles over it.  Rows are gathered through token_position_to_id while the A
// operand is staged (the gather is fused into the load, no gathered copy exists in HBM).
// The bf16 and fp8-row weights arrive N-contiguous ([E, H, 2, I], [E, I, H]); both MFMA operands
// are read along K, so a transposition kernel first writes K-contiguous copies of them, after
// which both operands are 16-byte copies into LDS and the K loop is software pipelined (loads
// of step k+1 in flight under the MFMAs of step k).  MXFP8 weights outside the large-tile path
// keep the reference's x4 layouts and a plain loop.
//
// Reference semantics: generate_blockwise_numpy_golden,
//   test/integration/nkilib/core/moe/moe_cte/test_moe_cte_common.py:267-447 (bf16 / fp8 weight),
//   test/integration/nkilib/core/moe/moe_cte/test_utils.py:474-735 with
//   test/integration/nkilib/core/mlp/test_mlp_common.py:550-682 (MXFP8),
//   test/integration/nkilib/core/mlp/test_mlp_common.py:978-1022,1114-1116 (fp8 row scales).
#include <type_traits>

#include "bwmm.hpp"

namespace moe {

constexpr int GT = 256;       // threads per workgroup
constexpr int TM = 128;       // rows per workgroup tile
constexpr int LROW = 144;     // LDS bytes per staged row: 128 bytes of K + 16 pad (16-byte aligned)

__device__ __forceinline__ float load_aff(const void* aff, int dtype, int64_t idx) {
  return dtype == MOE_DT_BF16 ? bf16_bits_to_f32(((const uint16_t*)aff)[idx]) : ((const float*)aff)[idx];
}
__device__ __forceinline__ float load_bias(const void* p, int dtype, int64_t idx) {
  return dtype == MOE_DT_BF16 ? bf16_bits_to_f32(((const uint16_t*)p)[idx]) : ((const float*)p)[idx];
}

// Operand fragment of v_mfma_scale_f32_16x16x128_f8f6f4 for one row / column whose 128 K bytes
// sit contiguously at `row`: lane group g = lane/16 supplies K bytes [16g, 16g+16) in its first
// four registers and [64+16g, 64+16g+16) in the last four.  With that placement the hardware's
// K index equals the byte offset, and the scale byte a lane supplies (lanes 16j..16j+15 scale
// K block j = bytes [32j, 32j+32) of their row) lines up with consecutive 32-byte MX blocks.
__device__ __forceinline__ v8i lds_read_frag(const uint8_t* row, int g) {
  const v4i lo = *(const v4i*)(row + 16 * g);
  const v4i hi = *(const v4i*)(row + 64 + 16 * g);
  v8i r;
  r[0] = lo[0]; r[1] = lo[1]; r[2] = lo[2]; r[3] = lo[3];
  r[4] = hi[0]; r[5] = hi[1]; r[6] = hi[2]; r[7] = hi[3];
  return r;
}

// (the bf16 and fp8-row kinds are held to 256 registers in stage 1 and 168 in stage 2 so that two / three workgroups
// share a CU: each keeps the CU's loads flowing while the others wait at their barriers or run MFMAs; the
// 128 x 256 stage-1 tile alone needs 128 accumulator registers)
// The same fragment from a 128-byte row whose 16-byte pieces are swizzled with sw = row & 7.
__device__ __forceinline__ v8i lds_read_frag_swz(const uint8_t* row, int g, int sw) {
  const v4i lo = *(const v4i*)(row + ((g ^ sw) * 16));
  const v4i hi = *(const v4i*)(row + (((g + 4) ^ sw) * 16));
  v8i r;
  r[0] = lo[0]; r[1] = lo[1]; r[2] = lo[2]; r[3] = lo[3];
  r[4] = hi[0]; r[5] = hi[1]; r[6] = hi[2]; r[7] = hi[3];
  return r;
}

template <int KIND, int STAGE>
__global__ __launch_bounds__(GT) __attribute__((amdgpu_waves_per_eu(KIND == MOE_KIND_MXFP8 ? 1 : (STAGE == 2 ? 3 : 2), 8))) void bwmm_kernel(
    const GemmArgs a) {
  constexpr int NCOLS = (STAGE == 1) ? 256 : 128;
  constexpr int NT = NCOLS / 16;
  // bf16 / fp8-row: 128-byte rows whose 16-byte pieces are XOR-swizzled with the row's low three bits (piece j of
  // row r sits at j ^ (r & 7)): the 16 lanes that a 16-byte LDS read serves in one pass (lanes 0-3, 12-15, 20-23,
  // 24-27 of a wave, and so on) then touch 64 different banks, which rows padded to 144 bytes do not achieve
  // (a third of the LDS cycles were bank conflicts).  MXFP8: padded rows, staged by 4-byte transposing stores.
  constexpr int SROW = (KIND == MOE_KIND_MXFP8) ? LROW : 128;
  __shared__ __attribute__((aligned(16))) uint8_t sA[TM * SROW];
  __shared__ __attribute__((aligned(16))) uint8_t sB[NCOLS * SROW];
  __shared__ uint32_t sAs[TM];   // MX: the 4 E8M0 bytes of this k-step; FP8_ROW: fp32 row scale bits
  __shared__ uint32_t sBs[NCOLS];
  __shared__ int s_tok[TM];
  __shared__ float s_aff[TM];

  const int tid = threadIdx.x;
  const int rt = blockIdx.y;
  const int b = rt / a.tiles_per_block;
  const int r0 = (rt % a.tiles_per_block) * TM;
  if (b >= *a.n_active) return;
  // with checkpoint outputs every row of an executed block is computed: padding rows are zero inputs
  const int vr = a.ckpt ? (int)a.B : a.valid_rows[b];
  if (r0 >= vr) return;
  const int e = a.b2e[b];
  const int64_t slot0 = (int64_t)b * a.B + r0;

  // ---- column tile geometry -------------------------------------------------------------
  // MX stage 1: blockIdx.x = tI*4 + pg; columns are (gu, q, pl) with weight column
  // i = tI*512 + q*Pt + p0 + pl, Pt = valid partitions of intermediate tile tI.
  int tI = 0, p0 = 0, Pt = 0;
  int64_t c0 = 0;  // first output column (BF16 / FP8_ROW stage 1: i0; stage 2: h0)
  if (KIND == MOE_KIND_MXFP8 && STAGE == 1) {
    tI = blockIdx.x >> 2;
    p0 = (blockIdx.x & 3) * 32;
    const int rows_t = (int)((a.I - (int64_t)tI * 512 < 512) ? (a.I - (int64_t)tI * 512) : 512);
    Pt = rows_t / 4;
    if (p0 >= Pt) return;
  } else {
    c0 = (int64_t)blockIdx.x * 128;
  }

  if (tid < TM) {
    const int r = r0 + tid;
    int id = -1;
    if (r < a.B) id = a.tp2id[(int64_t)b * a.B + r];
    if (id < 0 || id >= a.n_real) id = -1;
    s_tok[tid] = id;
    float af = 0.f;
    if (id >= 0 && a.aff) af = load_aff(a.aff, a.aff_dtype, (int64_t)id * a.E + e);
    s_aff[tid] = af;
    if (KIND == MOE_KIND_FP8_ROW) {
      float rs = 0.f;
      if (STAGE == 1) {
        if (id >= 0) rs = *(const float*)(a.A + (int64_t)id * a.a_stride + a.H);
      } else {
        if (r < vr) rs = ((const float*)a.A_scale)[slot0 + tid];
      }
      sAs[tid] = __float_as_uint(rs);
    }
  }
  __syncthreads();

  const int lane = tid & 63, w = tid >> 6;
  const int c = lane & 15, g = lane >> 4;
  // MXFP8: a wave owns 32 rows and every column tile.  bf16 / fp8-row: the four waves form a 2 x 2 grid, a wave
  // owns 64 rows and half the column tiles (stage 1: four gate tiles and the matching four up tiles), which
  // takes a third fewer fragment bytes out of LDS per MFMA than 32 rows x all columns.
  constexpr bool GRID2 = (KIND != MOE_KIND_MXFP8);
  constexpr int MT = GRID2 ? 4 : 2;
  constexpr int NTW = GRID2 ? NT / 2 : NT;
  const int m0 = GRID2 ? (w >> 1) * 64 : w * 32;
  const int wn = GRID2 ? (w & 1) : 0;
  // column tile (16 staged columns) behind accumulator index nt
  auto ctile = [&](int nt) -> int {
    if constexpr (!GRID2) return nt;
    else if constexpr (STAGE == 1) return (nt < 4) ? wn * 4 + nt : 4 + wn * 4 + nt;
    else return wn * 4 + nt;
  };

  v4f acc[NTW][MT];
#pragma unroll
  for (int nt = 0; nt < NTW; ++nt)
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) acc[nt][mt] = (v4f){0.f, 0.f, 0.f, 0.f};

  // ---- K loop ---------------------------------------------------------------------------
  const bool fp4 = KIND == MOE_KIND_MXFP8 && a.weight_dtype == MOE_DT_FP4_E2M1;  // 4-bit weights
  int nks;
  if (KIND == MOE_KIND_MXFP8) nks = (STAGE == 1) ? (int)(a.H / 128) : a.nI * 4;
  else if (KIND == MOE_KIND_BF16) nks = (int)((a.K + 63) / 64);
  else nks = (int)((a.K + 127) / 128);

  if constexpr (KIND == MOE_KIND_FP8_ROW || KIND == MOE_KIND_BF16) {
    // Both operands are plain 16-byte copies here (the weights were transposed to K-contiguous rows of Kp bytes
    // beforehand), so the loop is software pipelined: the global loads of k-step ks+1 are in flight while the
    // MFMAs of k-step ks run.  A k-step is 128 bytes of K: 128 fp8 or 64 bf16 elements.
    const int64_t kbytes = (KIND == MOE_KIND_BF16) ? a.K * 2 : a.K;
    constexpr int PB = NCOLS * 8 / GT;
    uint4 ra[4], rb[PB];
    // What a thread stages does not change over the K loop: 16-byte piece tid & 7 of rows / columns (tid >> 3) + 32 j.
    // The addresses are worked out once: the A rows as 32-bit offsets (in units of 4 bytes) from a.A, the weight
    // rows as one pointer plus offsets that are the same for the whole workgroup.
    const int pc = tid & 7, rl = tid >> 3;
    uint32_t ao[4];  // ~0: no such row
    unsigned b_ok = 0;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int row = rl + 32 * j;
      int64_t off = -1;
      if (STAGE == 1) {
        const int tok = s_tok[row];
        if (tok >= 0) off = (int64_t)tok * a.a_stride;
      } else {
        if (r0 + row < vr) off = (slot0 + row) * a.a_stride;
      }
      ao[j] = (off >= 0) ? (uint32_t)((off + pc * 16) >> 2) : ~0u;
    }
    const uint8_t* wb;
    if (STAGE == 1) wb = a.W + (((int64_t)e * 2) * a.I + c0 + rl) * a.Kp + pc * 16;
    else wb = a.W + ((int64_t)e * a.H + c0 + rl) * a.Kp + pc * 16;
#pragma unroll
    for (int j = 0; j < PB; ++j) {
      const int64_t cj = c0 + rl + 32 * (STAGE == 1 ? (j & 3) : j);  // stage 1: j < 4 gate columns, j >= 4 up columns
      if (cj < (STAGE == 1 ? a.I : a.H)) b_ok |= 1u << j;
    }
    auto fetch = [&](int ks) {
      const int64_t a_off = (int64_t)ks * 128;
      const bool a_in = pc * 16 + 16 <= kbytes - a_off;  // A rows end at K; the weight rows are zero padded to Kp
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        uint4 val = make_uint4(0, 0, 0, 0);
        if (ao[j] != ~0u && a_in) {
          const uint8_t* src = a.A + ((int64_t)ao[j] << 2) + a_off;
          if (KIND == MOE_KIND_FP8_ROW && STAGE == 1) {  // rows of H + 4 bytes are only 4-byte aligned
            const uint32_t* s4 = (const uint32_t*)src;
            val = make_uint4(s4[0], s4[1], s4[2], s4[3]);
          } else {
            val = *(const uint4*)src;
          }
        }
        ra[j] = val;
      }
#pragma unroll
      for (int j = 0; j < PB; ++j) {
        const int64_t wj = (STAGE == 1) ? ((int64_t)(j >> 2) * a.I + 32 * (j & 3)) * a.Kp : (int64_t)(32 * j) * a.Kp;
        uint4 val = make_uint4(0, 0, 0, 0);
        if ((b_ok >> j) & 1u) val = *(const uint4*)(wb + wj + a_off);
        rb[j] = val;
      }
    };
    fetch(0);
    for (int ks = 0; ks < nks; ++ks) {
#pragma unroll
      for (int j = 0; j < 4; ++j) *(uint4*)(sA + ((tid >> 3) + 32 * j) * SROW + (((tid & 7) ^ ((tid >> 3) & 7)) * 16)) = ra[j];
#pragma unroll
      for (int j = 0; j < PB; ++j) {
        const int idx = tid + GT * j;  // row idx >> 3 has the low bits of tid >> 3 as well
        *(uint4*)(sB + (idx >> 3) * SROW + (((tid & 7) ^ ((tid >> 3) & 7)) * 16)) = rb[j];
      }
      __syncthreads();
      if (ks + 1 < nks) fetch(ks + 1);
      if constexpr (KIND == MOE_KIND_BF16) {
#pragma unroll
        for (int sub = 0; sub < 2; ++sub) {
          v8bf af[MT];
#pragma unroll
          for (int mt = 0; mt < MT; ++mt) af[mt] = *(const v8bf*)(sA + (m0 + 16 * mt + c) * SROW + (((sub * 4 + g) ^ (c & 7)) * 16));
#pragma unroll
          for (int nt = 0; nt < NTW; ++nt) {
            const v8bf bf = *(const v8bf*)(sB + (ctile(nt) * 16 + c) * SROW + (((sub * 4 + g) ^ (c & 7)) * 16));
#pragma unroll
            for (int mt = 0; mt < MT; ++mt)
              acc[nt][mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(af[mt], bf, acc[nt][mt], 0, 0, 0);
          }
        }
      } else {
        v8i af[MT];
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) af[mt] = lds_read_frag_swz(sA + (m0 + 16 * mt + c) * SROW, g, c & 7);
#pragma unroll
        for (int nt = 0; nt < NTW; ++nt) {
          const v8i bf = lds_read_frag_swz(sB + (ctile(nt) * 16 + c) * SROW, g, c & 7);
#pragma unroll
          for (int mt = 0; mt < MT; ++mt)
            acc[nt][mt] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(af[mt], bf, acc[nt][mt], 0, 0, 0, 127, 0, 127);
        }
      }
      __syncthreads();
    }
  } else
  for (int ks = 0; ks < nks; ++ks) {  // MXFP8: the weights stay in the reference's x4 layouts
    // position of this k-step: K tile (H or I tile), partition group, valid partitions
    const int kt = ks >> 2, pb = ks & 3;
    int Ptk = 128;
    int a_valid = 128;                  // valid bytes of the slice
    if (STAGE == 2) {
      const int rows_t = (int)((a.I - (int64_t)kt * 512 < 512) ? (a.I - (int64_t)kt * 512) : 512);
      Ptk = rows_t / 4;
      if (pb * 32 >= Ptk) continue;
      a_valid = (Ptk - pb * 32) * 4 < 128 ? (Ptk - pb * 32) * 4 : 128;
    }
    const int64_t a_off = (int64_t)kt * 512 + pb * 128;  // byte offset of the slice inside an A row

    // ---- stage A: 128 rows x 128 bytes, 8 threads per row ---------------------------------
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int row = (tid >> 3) + 32 * j;
      const int ch = tid & 7;
      uint4 val = make_uint4(0, 0, 0, 0);
      const uint8_t* src = nullptr;
      if (STAGE == 1) {
        const int tok = s_tok[row];
        if (tok >= 0) src = a.A + (int64_t)tok * a.a_stride;
      } else {
        if (r0 + row < vr) src = a.A + (slot0 + row) * a.a_stride;
      }
      if (src != nullptr && ch * 16 + 16 <= a_valid) {
        val = *(const uint4*)(src + a_off + ch * 16);
      }
      *(uint4*)(sA + row * LROW + ch * 16) = val;
    }
    if (tid < TM) {
      uint32_t sv = 0;
      if (STAGE == 1) {
        const int tok = s_tok[tid];
        if (tok >= 0) sv = *(const uint32_t*)(a.A_scale + (int64_t)tok * a.a_scale_stride + ks * 4);
      } else {
        if (r0 + tid < vr) sv = *(const uint32_t*)(a.A_scale + (slot0 + tid) * a.a_scale_stride + kt * 16 + pb * 4);
        const int kbv = a_valid >> 5;  // valid 32-blocks in this slice
        if (kbv < 4) sv &= (1u << (8 * kbv)) - 1u;
      }
      sAs[tid] = sv;
    }

    // ---- stage B, transposed into K-contiguous rows ---------------------------------------
    if (KIND == MOE_KIND_MXFP8) {
      const uint32_t* W4 = (const uint32_t*)a.W;
      const uint16_t* W2 = (const uint16_t*)a.W;
      if (STAGE == 1) {
        // column = tid: (gu, q, pl); rows rho = partitions 32*pb + rho of H tile kt
        const int gu = tid >> 7, q = (tid >> 5) & 3, pl = tid & 31;
        const bool cv = (p0 + pl) < Pt;
        const int64_t i = (int64_t)tI * 512 + (int64_t)q * Pt + p0 + pl;
        const int64_t nH = a.H / 512;
        const int64_t pstride = 2 * nH * a.I;
        const int64_t base = ((((int64_t)e * 128 + pb * 32) * 2 + gu) * nH + kt) * a.I + i;
        if (fp4) {  // 2-byte x4 elements: a row's 128 K values are 64 bytes
#pragma unroll 8
          for (int rho = 0; rho < 32; ++rho) *(uint16_t*)(sB + tid * LROW + rho * 2) = cv ? W2[base + rho * pstride] : (uint16_t)0;
        } else {
#pragma unroll 8
          for (int rho = 0; rho < 32; ++rho) {
            const uint32_t v = cv ? W4[base + rho * pstride] : 0u;
            *(uint32_t*)(sB + tid * LROW + rho * 4) = v;
          }
        }
        uint32_t sv = 0;
        if (cv) {
          const int64_t sbase = ((((int64_t)e * 16 + pb * 4) * 2 + gu) * nH + kt) * a.I + i;
#pragma unroll
          for (int k = 0; k < 4; ++k) sv |= (uint32_t)a.W_scale[sbase + k * pstride] << (8 * k);
        }
        sBs[tid] = sv;
      } else {
        const int col = tid & 127, half = tid >> 7;
        const int64_t h = c0 + col;
        const bool cv = h < a.H;
        const int64_t pstride = (int64_t)a.nI * a.H;
        const int64_t base = (((int64_t)e * a.pI + pb * 32) * a.nI + kt) * a.H + h;
#pragma unroll 8
        for (int j = 0; j < 16; ++j) {
          const int rho = 2 * j + half;
          const bool ok = cv && pb * 32 + rho < Ptk;
          if (fp4) *(uint16_t*)(sB + col * LROW + rho * 2) = ok ? W2[base + rho * pstride] : (uint16_t)0;
          else *(uint32_t*)(sB + col * LROW + rho * 4) = ok ? W4[base + rho * pstride] : 0u;
        }
        if (half == 0) {
          uint32_t sv = 0;
          const int64_t sbase = (((int64_t)e * ((a.pI + 7) / 8) + pb * 4) * a.nI + kt) * a.H + h;
#pragma unroll
          for (int k = 0; k < 4; ++k)
            if (cv && (pb * 4 + k) * 8 < Ptk) sv |= (uint32_t)a.W_scale[sbase + k * pstride] << (8 * k);
          sBs[col] = sv;
        }
      }
    }
    __syncthreads();

    // ---- MFMA ------------------------------------------------------------------------------
    {
      v8i af[2];
      int sa[2];
#pragma unroll
      for (int mt = 0; mt < 2; ++mt) {
        const int row = m0 + 16 * mt + c;
        af[mt] = lds_read_frag(sA + row * LROW, g);
        sa[mt] = (int)((sAs[row] >> (8 * g)) & 0xffu);
      }
      // the element format of the weights is an immediate of the instruction (blgp: 0 e4m3, 1 e5m2, 4 e2m1); a
      // 4-bit operand is four registers, lane group g holding K 32g .. 32g+31 = bytes [16g, 16g+16) of the row
      auto columns = [&](auto blgp_) {
        constexpr int BLGP = decltype(blgp_)::value;
#pragma unroll
        for (int nt = 0; nt < NT; ++nt) {
          const int col = nt * 16 + c;
          v8i bf;
          if constexpr (BLGP == 4) {
            const v4i lo = *(const v4i*)(sB + col * LROW + 16 * g);
            bf = (v8i){lo[0], lo[1], lo[2], lo[3], 0, 0, 0, 0};
          } else {
            bf = lds_read_frag(sB + col * LROW, g);
          }
          const int sb = (int)((sBs[col] >> (8 * g)) & 0xffu);
#pragma unroll
          for (int mt = 0; mt < 2; ++mt)
            acc[nt][mt] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(af[mt], bf, acc[nt][mt], 0, BLGP, 0, sa[mt], 0, sb);
        }
      };
      if (a.weight_dtype == MOE_DT_FP8_E5M2) columns(std::integral_constant<int, 1>{});
      else if (fp4) columns(std::integral_constant<int, 4>{});
      else columns(std::integral_constant<int, 0>{});
    }
    __syncthreads();
  }

  // ---- epilogue ----------------------------------------------------------------------------
  // accumulator element r of tile (nt, mt) is (row m0 + 16*mt + 4*g + r, column nt*16 + c)
  if constexpr (STAGE == 1) {
    const bool pre = (a.scaling_mode == MOE_SCALE_PRE || a.scaling_mode == MOE_SCALE_PRE_DELAYED);
    if constexpr (KIND == MOE_KIND_MXFP8) {
      uint8_t* Yq = (uint8_t*)a.out;
#pragma unroll
      for (int half = 0; half < 2; ++half) {
        const int p = p0 + 16 * half + c;
        const bool pv = p < Pt;
        float bg[4] = {0.f, 0.f, 0.f, 0.f}, bu[4] = {0.f, 0.f, 0.f, 0.f};
        if (a.bias && pv) {
#pragma unroll
          for (int q = 0; q < 4; ++q) {
            // bias [E, pI, 2, nI, 4]
            bg[q] = load_bias(a.bias, a.bias_dtype, ((((int64_t)e * a.pI + p) * 2 + 0) * a.nI + tI) * 4 + q);
            bu[q] = load_bias(a.bias, a.bias_dtype, ((((int64_t)e * a.pI + p) * 2 + 1) * a.nI + tI) * 4 + q);
          }
        }
#pragma unroll
        for (int mt = 0; mt < 2; ++mt) {
#pragma unroll
          for (int r = 0; r < 4; ++r) {
            const int row = m0 + 16 * mt + 4 * g + r;
            float y[4];
            float am = 0.f;
#pragma unroll
            for (int q = 0; q < 4; ++q) {
              float gv = acc[q * 2 + half][mt][r] + bg[q];
              float uv = acc[8 + q * 2 + half][mt][r] + bu[q];
              if (a.clamp_mask & MOE_CLAMP_GATE_LO) gv = fmaxf(gv, a.clamp[1]);
              if (a.clamp_mask & MOE_CLAMP_GATE_HI) gv = fminf(gv, a.clamp[0]);
              if (a.clamp_mask & MOE_CLAMP_UP_LO) uv = fmaxf(uv, a.clamp[3]);
              if (a.clamp_mask & MOE_CLAMP_UP_HI) uv = fminf(uv, a.clamp[2]);
              y[q] = pv ? act_apply(gv, a.act_fn) * uv : 0.f;
              am = fmaxf(am, fabsf(y[q]));
            }
            // MX block = 8 consecutive partitions x 4 q: reduce over the 8-lane group
            am = fmaxf(am, __shfl_xor(am, 1, 64));
            am = fmaxf(am, __shfl_xor(am, 2, 64));
            am = fmaxf(am, __shfl_xor(am, 4, 64));
            const uint32_t sbyte = mx_scale_byte(am);
            const float is = mx_inv_scale(sbyte);
            const uint32_t dw = pack4_e4m3(clip448(y[0] * is), clip448(y[1] * is), clip448(y[2] * is), clip448(y[3] * is));
            if (pv && r0 + row < vr) {
              const int64_t slot = slot0 + row;
              *(uint32_t*)(Yq + slot * a.out_stride + tI * 512 + p * 4) = dw;
              if ((c & 7) == 0) a.out_scale[slot * a.out_scale_stride + tI * 16 + (p >> 3)] = (uint8_t)sbyte;
            }
          }
        }
      }
    } else {
      const float* wsc = (const float*)a.W_scale;
      const int64_t wsb = (a.w_scale_experts > 1) ? (int64_t)e * 2 * a.I : 0;
#pragma unroll
      for (int nt = 0; nt < NTW / 2; ++nt) {  // gate tile nt of this wave, its up tile is accumulator nt + NTW / 2
        const int64_t i = c0 + ctile(nt) * 16 + c;
        const bool iv = i < a.I;
        float sg = 1.f, su = 1.f, bg = 0.f, bu = 0.f;
        if (iv && wsc) { sg = wsc[wsb + i]; su = wsc[wsb + a.I + i]; }
        if (iv && a.bias) {
          bg = load_bias(a.bias, a.bias_dtype, ((int64_t)e * 2 + 0) * a.I + i);
          bu = load_bias(a.bias, a.bias_dtype, ((int64_t)e * 2 + 1) * a.I + i);
        }
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
#pragma unroll
          for (int r = 0; r < 4; ++r) {
            const int row = m0 + 16 * mt + 4 * g + r;
            float gv = acc[nt][mt][r], uv = acc[nt + NTW / 2][mt][r];
            if (KIND == MOE_KIND_BF16) {
              if (pre) { gv *= s_aff[row]; uv *= s_aff[row]; }
              gv *= sg; uv *= su;
            } else {
              // PRE_SCALE: the affinity scales the token's row, i.e. its dequantisation scale
              const float rs = pre ? __uint_as_float(sAs[row]) * s_aff[row] : __uint_as_float(sAs[row]);
              gv = (gv * sg) * rs; uv = (uv * su) * rs;
            }
            gv += bg; uv += bu;
            if (a.clamp_mask & MOE_CLAMP_GATE_LO) gv = fmaxf(gv, a.clamp[1]);
            if (a.clamp_mask & MOE_CLAMP_GATE_HI) gv = fminf(gv, a.clamp[0]);
            if (a.clamp_mask & MOE_CLAMP_UP_LO) uv = fmaxf(uv, a.clamp[3]);
            if (a.clamp_mask & MOE_CLAMP_UP_HI) uv = fminf(uv, a.clamp[2]);
            if (KIND == MOE_KIND_BF16 && a.ckpt && iv && r0 + row < a.B) {
              uint16_t* ck = a.ckpt + (((int64_t)b * 2) * a.I + i) * a.B + r0 + row;
              ck[0] = f32_to_bf16_bits(gv);
              ck[a.I * a.B] = f32_to_bf16_bits(uv);
            }
            const float y = iv ? act_apply(gv, a.act_fn) * uv : 0.f;
            if (r0 + row < vr) {
              const int64_t slot = slot0 + row;
              if (KIND == MOE_KIND_BF16) {
                if (i * 2 < a.out_stride) *(uint16_t*)((uint8_t*)a.out + slot * a.out_stride + i * 2) = f32_to_bf16_bits(y);
              } else {
                if (iv) *(float*)((uint8_t*)a.out + slot * a.out_stride + i * 4) = y;
              }
            }
          }
        }
      }
    }
  } else {
    uint16_t* D = (uint16_t*)a.out;
    const float* wsc = (KIND == MOE_KIND_MXFP8) ? nullptr : (const float*)a.W_scale;
    const int64_t wsb = (a.w_scale_experts > 1) ? (int64_t)e * a.H : 0;
    const bool post = a.scaling_mode == MOE_SCALE_POST;
#pragma unroll
    for (int nt = 0; nt < NTW; ++nt) {
      const int64_t h = c0 + ctile(nt) * 16 + c;
      if (h >= a.H) continue;
      const float sd = wsc ? wsc[wsb + h] : 1.f;
      const float bd = a.bias ? load_bias(a.bias, a.bias_dtype, (int64_t)e * a.H + h) : 0.f;
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) {
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          const int row = m0 + 16 * mt + 4 * g + r;
          if (s_tok[row] < 0 && !(KIND == MOE_KIND_BF16 && a.ckpt)) continue;
          float d = acc[nt][mt][r];
          if (KIND == MOE_KIND_BF16) d *= sd;
          if (KIND == MOE_KIND_FP8_ROW) d = (d * sd) * __uint_as_float(sAs[row]);
          d += bd;
          if (KIND == MOE_KIND_BF16 && a.ckpt) {
            if (r0 + row < a.B) a.ckpt[(slot0 + row) * a.H + h] = f32_to_bf16_bits(d);
            if (s_tok[row] < 0) continue;
          }
          if (post) d *= s_aff[row];
          D[(slot0 + row) * a.H + h] = f32_to_bf16_bits(d);
        }
      }
    }
  }
}

// Per-row fp8 re-quantisation of the fp8-row intermediate: scale = max(amax/240, 1e-5),
// q = e4m3(y / scale)  (test_mlp_common.py:978-986).  One workgroup per slot row.
__global__ __launch_bounds__(256) void row_requant_kernel(const float* __restrict__ Y, uint8_t* __restrict__ Yq,
                                                          float* __restrict__ ys, const int32_t* __restrict__ n_active,
                                                          const int32_t* __restrict__ valid_rows, int64_t B, int64_t I,
                                                          int64_t Iw) {
  __shared__ float red[16];
  const int64_t slot = blockIdx.x;
  const int64_t b = slot / B, r = slot % B;
  if (b >= *n_active || r >= valid_rows[b]) return;
  const float* y = Y + slot * I;
  uint8_t* q = Yq + slot * Iw;
  constexpr int MAXV = 16;  // float4 per thread kept in registers: rows of up to 16384 values are read once
  if (I % 4 == 0 && I <= (int64_t)MAXV * 4 * 256) {
    float4 v[MAXV];
    float am = 0.f;
#pragma unroll
    for (int j = 0; j < MAXV; ++j) {
      const int64_t i = ((int64_t)j * 256 + threadIdx.x) * 4;
      v[j] = (i < I) ? *(const float4*)(y + i) : make_float4(0.f, 0.f, 0.f, 0.f);
      am = fmaxf(fmaxf(am, fmaxf(fabsf(v[j].x), fabsf(v[j].y))), fmaxf(fabsf(v[j].z), fabsf(v[j].w)));
    }
    am = block_max(am, red);
    const float sc = fmaxf(am / 240.0f, 1e-05f);
    if (threadIdx.x == 0) ys[slot] = sc;
#pragma unroll
    for (int j = 0; j < MAXV; ++j) {
      const int64_t i = ((int64_t)j * 256 + threadIdx.x) * 4;
      if (i < Iw) *(uint32_t*)(q + i) = pack4_e4m3(v[j].x / sc, v[j].y / sc, v[j].z / sc, v[j].w / sc);
    }
    return;
  }
  float am = 0.f;
  for (int64_t i = threadIdx.x; i < I; i += blockDim.x) am = fmaxf(am, fabsf(y[i]));
  am = block_max(am, red);
  const float sc = fmaxf(am / 240.0f, 1e-05f);
  if (threadIdx.x == 0) ys[slot] = sc;
  for (int64_t i = (int64_t)threadIdx.x * 4; i < Iw; i += (int64_t)blockDim.x * 4) {
    float v[4];
#pragma unroll
    for (int k = 0; k < 4; ++k) v[k] = (i + k < I) ? y[i + k] / sc : 0.f;
    *(uint32_t*)(q + i) = pack4_e4m3(v[0], v[1], v[2], v[3]);
  }
}

// Byte-matrix transpose for the fp8 weights: batches of [R, C] (row stride src_row_stride) -> [C, Kp] with
// Kp >= R a multiple of 64, the tail of every output row zero.  The GEMM wants K-contiguous weight rows (both
// MFMA operands are read along K), the reference stores them N-contiguous.  64 x 64 tiles through LDS.
__global__ __launch_bounds__(256) void transpose_fp8_kernel(const uint8_t* __restrict__ src, uint8_t* __restrict__ dst,
                                                            int64_t R, int64_t C, int64_t src_row_stride, int64_t Kp,
                                                            int nb1, int64_t src_bs0, int64_t src_bs1, int64_t dst_bs) {
  __shared__ __attribute__((aligned(16))) uint8_t tile[64][80];
  const int b = blockIdx.z;
  const uint8_t* S = src + (int64_t)(b / nb1) * src_bs0 + (int64_t)(b % nb1) * src_bs1;
  uint8_t* D = dst + (int64_t)b * dst_bs;
  const int64_t n0 = (int64_t)blockIdx.x * 64, k0 = (int64_t)blockIdx.y * 64;
  {
    const int r = threadIdx.x >> 2, c16 = (threadIdx.x & 3) * 16;
    const int64_t k = k0 + r, n = n0 + c16;
    uint4 v = make_uint4(0, 0, 0, 0);
    if (k < R) {
      const uint8_t* p = S + k * src_row_stride + n;
      if (n + 16 <= C && (((uintptr_t)p) & 15) == 0) {
        v = *(const uint4*)p;
      } else {
        uint8_t t[16];
        for (int j = 0; j < 16; ++j) t[j] = (n + j < C) ? p[j] : (uint8_t)0;
        __builtin_memcpy(&v, t, 16);
      }
    }
    *(uint4*)(&tile[r][c16]) = v;
  }
  __syncthreads();
  const int nn = threadIdx.x >> 2, kc = (threadIdx.x & 3) * 16;
  if (n0 + nn < C) {
    uint32_t w[4];
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      w[q] = (uint32_t)tile[kc + 4 * q][nn] | ((uint32_t)tile[kc + 4 * q + 1][nn] << 8) |
             ((uint32_t)tile[kc + 4 * q + 2][nn] << 16) | ((uint32_t)tile[kc + 4 * q + 3][nn] << 24);
    }
    *(uint4*)(D + (n0 + nn) * Kp + k0 + kc) = make_uint4(w[0], w[1], w[2], w[3]);
  }
}

// The same for the bf16 kind: batches of [R, C] bf16 (W8 == false) or fp8-e4m3 widened to bf16 (W8 == true)
// -> bf16 [C, Kp] with Kp (elements) a multiple of 64.
template <bool W8>
__global__ __launch_bounds__(256) void transpose_w16_kernel(const uint8_t* __restrict__ src, uint16_t* __restrict__ dst,
                                                            int64_t R, int64_t C, int64_t src_row_stride, int64_t Kp,
                                                            int nb1, int64_t src_bs0, int64_t src_bs1, int64_t dst_bs) {
  __shared__ __attribute__((aligned(16))) uint16_t tile[64][72];
  constexpr int ES = W8 ? 1 : 2;
  const int b = blockIdx.z;
  const uint8_t* S = src + ((int64_t)(b / nb1) * src_bs0 + (int64_t)(b % nb1) * src_bs1) * ES;
  uint16_t* D = dst + (int64_t)b * dst_bs;
  const int64_t n0 = (int64_t)blockIdx.x * 64, k0 = (int64_t)blockIdx.y * 64;
#pragma unroll
  for (int j = 0; j < 2; ++j) {
    const int idx = threadIdx.x + 256 * j;
    const int r = idx >> 3, c8 = (idx & 7) * 8;
    const int64_t k = k0 + r, n = n0 + c8;
    uint16_t v[8];
#pragma unroll
    for (int q = 0; q < 8; ++q) v[q] = 0;
    if (k < R) {
      const uint8_t* p = S + (k * src_row_stride + n) * ES;
      if (n + 8 <= C && (((uintptr_t)p) & (8 * ES - 1)) == 0) {
        if (W8) {
          const uint2 raw = *(const uint2*)p;
#pragma unroll
          for (int q = 0; q < 8; ++q)
            v[q] = f32_to_bf16_bits(e4m3_to_f32(((q < 4 ? raw.x : raw.y) >> (8 * (q & 3))) & 0xffu));
        } else {
          *(uint4*)v = *(const uint4*)p;
        }
      } else {
        for (int q = 0; q < 8; ++q)
          if (n + q < C) v[q] = W8 ? f32_to_bf16_bits(e4m3_to_f32(p[q])) : ((const uint16_t*)p)[q];
      }
    }
    *(uint4*)(&tile[r][c8]) = *(const uint4*)v;
  }
  __syncthreads();
#pragma unroll
  for (int j = 0; j < 2; ++j) {
    const int idx = threadIdx.x + 256 * j;
    const int nn = idx >> 3, kc = (idx & 7) * 8;
    if (n0 + nn < C) {
      uint32_t w[4];
#pragma unroll
      for (int q = 0; q < 4; ++q) w[q] = (uint32_t)tile[kc + 2 * q][nn] | ((uint32_t)tile[kc + 2 * q + 1][nn] << 16);
      *(uint4*)(D + (n0 + nn) * Kp + k0 + kc) = make_uint4(w[0], w[1], w[2], w[3]);
    }
  }
}

int launch_transpose_w16(const void* src, int w8, uint16_t* dst, int64_t R, int64_t C, int64_t src_row_stride, int64_t Kp,
                         int64_t nb0, int nb1, int64_t src_bs0, int64_t src_bs1, hipStream_t s) {
  if ((Kp & 63) != 0 || Kp < R || (((uintptr_t)dst) & 15) != 0) return MOE_E_BAD_ARG;
  const int64_t gx = (C + 63) / 64, gy = Kp / 64, gz = nb0 * nb1;
  if (gy > 65535 || gz > 65535) return MOE_E_BAD_SHAPE;
  const dim3 grid((unsigned)gx, (unsigned)gy, (unsigned)gz);
  if (w8)
    hipLaunchKernelGGL(transpose_w16_kernel<true>, grid, dim3(256), 0, s, (const uint8_t*)src, dst, R, C, src_row_stride,
                       Kp, nb1, src_bs0, src_bs1, C * Kp);
  else
    hipLaunchKernelGGL(transpose_w16_kernel<false>, grid, dim3(256), 0, s, (const uint8_t*)src, dst, R, C, src_row_stride,
                       Kp, nb1, src_bs0, src_bs1, C * Kp);
  MOE_CHECK_LAUNCH();
  return MOE_OK;
}

int launch_transpose_fp8(const uint8_t* src, uint8_t* dst, int64_t R, int64_t C, int64_t src_row_stride, int64_t Kp,
                         int64_t nb0, int nb1, int64_t src_bs0, int64_t src_bs1, hipStream_t s) {
  if ((Kp & 63) != 0 || Kp < R || (((uintptr_t)dst) & 15) != 0) return MOE_E_BAD_ARG;
  const int64_t gx = (C + 63) / 64, gy = Kp / 64, gz = nb0 * nb1;
  if (gy > 65535 || gz > 65535) return MOE_E_BAD_SHAPE;
  hipLaunchKernelGGL(transpose_fp8_kernel, dim3((unsigned)gx, (unsigned)gy, (unsigned)gz), dim3(256), 0, s, src, dst, R,
                     C, src_row_stride, Kp, nb1, src_bs0, src_bs1, C * Kp);
  MOE_CHECK_LAUNCH();
  return MOE_OK;
}

// One thread per four adjacent output columns: four 4-byte reads (the four K rows of the x4 elements), a 4 x 4 byte
// transpose, one 16-byte write.  I % 4 == 0 and H % 4 == 0 on this path.
__device__ __forceinline__ uint4 bytes_4x4_transposed(const uint32_t (&r)[4]) {
  uint32_t o[4];
#pragma unroll
  for (int c = 0; c < 4; ++c)
    o[c] = ((r[0] >> (8 * c)) & 0xffu) | (((r[1] >> (8 * c)) & 0xffu) << 8) | (((r[2] >> (8 * c)) & 0xffu) << 16) |
           (((r[3] >> (8 * c)) & 0xffu) << 24);
  return make_uint4(o[0], o[1], o[2], o[3]);
}
__global__ __launch_bounds__(256) void relayout_gu_x4_kernel(const uint8_t* __restrict__ W, uint32_t* __restrict__ X,
                                                             int64_t H, int64_t I, int64_t total4) {
  const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;  // over [E, 128, 2, nH, I / 4]
  if (idx >= total4) return;
  const int64_t nH = H / 512, I4 = I / 4;
  const int64_t i = (idx % I4) * 4, t = (idx / I4) % nH, gu = (idx / (I4 * nH)) % 2, p = (idx / (I4 * nH * 2)) % 128,
                e = idx / (I4 * nH * 2 * 128);
  const int64_t h = t * 512 + p * 4;
  uint32_t r[4];
#pragma unroll
  for (int q = 0; q < 4; ++q) r[q] = *(const uint32_t*)(W + ((e * H + h + q) * 2 + gu) * I + i);
  *(uint4*)(X + idx * 4) = bytes_4x4_transposed(r);
}
__global__ __launch_bounds__(256) void relayout_down_x4_kernel(const uint8_t* __restrict__ W, uint32_t* __restrict__ X,
                                                               int64_t H, int64_t I, int64_t I_pad, int64_t pI,
                                                               int64_t nI, int64_t total4) {
  const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;  // over [E, pI, nI, H / 4]
  if (idx >= total4) return;
  const int64_t H4 = H / 4;
  const int64_t h = (idx % H4) * 4, t = (idx / H4) % nI, p = (idx / (H4 * nI)) % pI, e = idx / (H4 * nI * pI);
  const int64_t i0 = t * 512 + p * 4;
  uint32_t r[4];
#pragma unroll
  for (int q = 0; q < 4; ++q) r[q] = (i0 + q < I) ? *(const uint32_t*)(W + (e * I_pad + i0 + q) * H + h) : 0u;
  *(uint4*)(X + idx * 4) = bytes_4x4_transposed(r);
}
__global__ __launch_bounds__(256) void fill_bytes_kernel(uint32_t* __restrict__ p, int64_t words, uint32_t v) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i < words) p[i] = v;
}

int launch_fill_bytes(void* p, size_t bytes, uint8_t value, hipStream_t s) {
  if (bytes == 0) return MOE_OK;
  if ((bytes & 3) != 0 || ((uintptr_t)p & 3) != 0) return MOE_E_BAD_ARG;
  const int64_t words = (int64_t)(bytes / 4);
  hipLaunchKernelGGL(fill_bytes_kernel, dim3((unsigned)((words + 255) / 256)), dim3(256), 0, s, (uint32_t*)p, words,
                     0x01010101u * value);
  MOE_CHECK_LAUNCH();
  return MOE_OK;
}

int launch_relayout_x4(const uint8_t* gate_up, const uint8_t* down, uint8_t* dst, int which, int64_t E, int64_t H,
                       int64_t I, int64_t I_pad, hipStream_t s) {
  if ((((uintptr_t)dst) & 15) != 0 || (((uintptr_t)gate_up) & 3) != 0 || (((uintptr_t)down) & 3) != 0)
    return MOE_E_BAD_ARG;
  if (which == 0) {
    const int64_t total = E * 128 * 2 * (H / 512) * (I / 4);
    if ((total + 255) / 256 >= (int64_t)1 << 31) return MOE_E_BAD_SHAPE;
    hipLaunchKernelGGL(relayout_gu_x4_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, s, gate_up,
                       (uint32_t*)dst, H, I, total);
  } else {
    const int64_t nI = (I + 511) / 512, pI = I > 512 ? 128 : I / 4;
    const int64_t total = E * pI * nI * (H / 4);
    if ((total + 255) / 256 >= (int64_t)1 << 31) return MOE_E_BAD_SHAPE;
    hipLaunchKernelGGL(relayout_down_x4_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, s, down,
                       (uint32_t*)dst, H, I, I_pad, pI, nI, total);
  }
  MOE_CHECK_LAUNCH();
  return MOE_OK;
}

// bf16 weights (W8: fp8-e4m3 weights widened to bf16 on the way, exactly): one thread per four adjacent output
// columns, two 8-byte (4-byte) reads (the two K rows of the x4 elements), one 16-byte write.
template <bool W8>
__device__ __forceinline__ uint2 four_as_bf16(const void* W, int64_t elem) {
  if constexpr (W8) {
    const uint32_t raw = *(const uint32_t*)((const uint8_t*)W + elem);
    uint32_t v[4];
#pragma unroll
    for (int q = 0; q < 4; ++q) v[q] = f32_to_bf16_bits(e4m3_to_f32((raw >> (8 * q)) & 0xffu));
    return make_uint2(v[0] | (v[1] << 16), v[2] | (v[3] << 16));
  } else {
    return *(const uint2*)((const uint16_t*)W + elem);
  }
}
__device__ __forceinline__ uint4 pairs_of_4(const uint2& r0, const uint2& r1) {
  return make_uint4((r0.x & 0xffffu) | (r1.x << 16), (r0.x >> 16) | (r1.x & 0xffff0000u), (r0.y & 0xffffu) | (r1.y << 16),
                    (r0.y >> 16) | (r1.y & 0xffff0000u));
}
template <bool W8>
__global__ __launch_bounds__(256) void relayout_gu_x4_bf16_kernel(const void* __restrict__ W, uint32_t* __restrict__ X,
                                                                  int64_t H, int64_t I, int64_t total4) {
  const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;  // over [E, 128, 2, 2H / 512, I / 4]
  if (idx >= total4) return;
  const int64_t nH = H / 256, I4 = I / 4;
  const int64_t i = (idx % I4) * 4, t = (idx / I4) % nH, gu = (idx / (I4 * nH)) % 2, p = (idx / (I4 * nH * 2)) % 128,
                e = idx / (I4 * nH * 2 * 128);
  const int64_t h = t * 256 + p * 2;
  const uint2 r0 = four_as_bf16<W8>(W, ((e * H + h) * 2 + gu) * I + i);
  const uint2 r1 = four_as_bf16<W8>(W, ((e * H + h + 1) * 2 + gu) * I + i);
  *(uint4*)(X + idx * 4) = pairs_of_4(r0, r1);
}
template <bool W8>
__global__ __launch_bounds__(256) void relayout_down_x4_bf16_kernel(const void* __restrict__ W,
                                                                    uint32_t* __restrict__ X, int64_t H, int64_t I,
                                                                    int64_t I_pad, int64_t pI, int64_t nI,
                                                                    int64_t total4) {
  const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;  // over [E, pI, nI, H / 4], pI and nI those of 2I bytes
  if (idx >= total4) return;
  const int64_t H4 = H / 4;
  const int64_t h = (idx % H4) * 4, t = (idx / H4) % nI, p = (idx / (H4 * nI)) % pI, e = idx / (H4 * nI * pI);
  const int64_t i0 = t * 256 + p * 2;
  const uint2 zero = make_uint2(0u, 0u);
  const uint2 r0 = (i0 < I) ? four_as_bf16<W8>(W, (e * I_pad + i0) * H + h) : zero;
  const uint2 r1 = (i0 + 1 < I) ? four_as_bf16<W8>(W, (e * I_pad + i0 + 1) * H + h) : zero;
  *(uint4*)(X + idx * 4) = pairs_of_4(r0, r1);
}
int launch_relayout_x4_bf16(const void* gate_up, const void* down, int w8, uint8_t* dst, int which, int64_t E, int64_t H,
                            int64_t I, int64_t I_pad, hipStream_t s) {
  const uintptr_t src_align = w8 ? 3 : 7;
  if ((((uintptr_t)dst) & 15) != 0 || (((uintptr_t)gate_up) & src_align) != 0 || (((uintptr_t)down) & src_align) != 0 ||
      H % 256 != 0 || I % 4 != 0)
    return MOE_E_BAD_ARG;
  if (which == 0) {
    const int64_t total = E * 128 * 2 * (H / 256) * (I / 4);
    if ((total + 255) / 256 >= (int64_t)1 << 31) return MOE_E_BAD_SHAPE;
    if (w8)
      hipLaunchKernelGGL(relayout_gu_x4_bf16_kernel<true>, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, s, gate_up,
                         (uint32_t*)dst, H, I, total);
    else
      hipLaunchKernelGGL(relayout_gu_x4_bf16_kernel<false>, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, s, gate_up,
                         (uint32_t*)dst, H, I, total);
  } else {
    const int64_t Ib = 2 * I, nI = (Ib + 511) / 512, pI = Ib > 512 ? 128 : Ib / 4;
    const int64_t total = E * pI * nI * (H / 4);
    if ((total + 255) / 256 >= (int64_t)1 << 31) return MOE_E_BAD_SHAPE;
    if (w8)
      hipLaunchKernelGGL(relayout_down_x4_bf16_kernel<true>, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, s, down,
                         (uint32_t*)dst, H, I, I_pad, pI, nI, total);
    else
      hipLaunchKernelGGL(relayout_down_x4_bf16_kernel<false>, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, s, down,
                         (uint32_t*)dst, H, I, I_pad, pI, nI, total);
  }
  MOE_CHECK_LAUNCH();
  return MOE_OK;
}

template <int KIND, int STAGE>
static int launch_gemm(const GemmArgs& g, unsigned gx, unsigned gy, hipStream_t s) {
  if (gx == 0 || gy == 0) return MOE_OK;
  hipLaunchKernelGGL((bwmm_kernel<KIND, STAGE>), dim3(gx, gy), dim3(GT), 0, s, g);
  MOE_CHECK_LAUNCH();
  return MOE_OK;
}

int launch_gemm_stage(int kind, int stage, const GemmArgs& g, unsigned gx, unsigned gy, hipStream_t s) {
  if (kind == MOE_KIND_BF16) return stage == 1 ? launch_gemm<MOE_KIND_BF16, 1>(g, gx, gy, s) : launch_gemm<MOE_KIND_BF16, 2>(g, gx, gy, s);
  if (kind == MOE_KIND_FP8_ROW)
    return stage == 1 ? launch_gemm<MOE_KIND_FP8_ROW, 1>(g, gx, gy, s) : launch_gemm<MOE_KIND_FP8_ROW, 2>(g, gx, gy, s);
  return stage == 1 ? launch_gemm<MOE_KIND_MXFP8, 1>(g, gx, gy, s) : launch_gemm<MOE_KIND_MXFP8, 2>(g, gx, gy, s);
}

int launch_row_requant(const float* Y, uint8_t* Yq, float* ys, const Bookkeeping& k, int64_t N, int64_t B, int64_t I,
                       int64_t Iw, hipStream_t s) {
  hipLaunchKernelGGL(row_requant_kernel, dim3((unsigned)(N * B)), dim3(256), 0, s, Y, Yq, ys, k.n_active, k.valid_rows,
                     B, I, Iw);
  MOE_CHECK_LAUNCH();
  return MOE_OK;
}

}  // namespace moe
