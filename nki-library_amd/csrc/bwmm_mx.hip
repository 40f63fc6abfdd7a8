// MX (MXFP8 / MXFP4 weights, MXFP8 activations) blockwise expert GEMMs for gfx950, large-tile version.
//
// A 256-thread workgroup (4 waves, one per SIMD) owns an "expert chunk" of up to 320 consecutive
// slots of one expert and 256 output columns:
//   gate/up: 32 intermediate partitions p x 4 q, for gate and for up; wave w owns q = w
//   down:    256 hidden columns; wave w owns 64 of them
// so every weight byte that enters the CU is used by all rows of the chunk, and both operands enter
// the CU exactly once per workgroup (smaller or split tiles were measured: 128-row workgroups double
// the traffic into the CU and, because sibling workgroups drift apart by more K slices than the L2
// holds, the traffic over the fabric as well).  A wave accumulates rows x 64 columns: 16 x 4 MFMA
// tiles in the 256 accumulation registers, plus 4 x 4 tiles in ordinary registers for chunks of
// 257..320 rows.
//
// With one wave per SIMD nothing overlaps unless the instruction stream says so, so the K loop is
// written as a fixed sequence of instructions (MFMAs, loads, waits) around which the compiler only
// allocates registers:
//   * the loads of slice ks+D (D = 3, or 2 for 320-row chunks) are issued one by one between the
//     MFMAs of slice ks (a burst of loads blocks the wave at the issue stage while the matrix pipe
//     drains);
//   * expert weights (B operand) go global -> registers, never through LDS.  In the reference
//     layout a weight column's K runs over partitions p (4 K values per x4 element), and lane
//     group g of v_mfma_scale_f32_16x16x128_f8f6f4 needs K bytes [16g,16g+16) and [64+16g,
//     64+16g+16) of the 128-byte K slice, i.e. partitions 4g..4g+3 and 16+4g..16+4g+3 of the 32
//     partitions of the slice (4-bit weights: K 32g..32g+31 = partitions 8g..8g+7): eight loads
//     per lane, each fetching 4 adjacent columns = 4 MFMA column tiles at once.  The loads land in
//     one of D "raw" register sets; a set is transposed into MFMA operand order at the top of the
//     slice that uses it;
//   * activations (A operand, rows gathered through token_position_to_id) go global -> LDS
//     directly into a ring of D+1 stages of 256 (320) rows x 128 K-bytes, read by all four waves;
//     the fragments of the next two row tiles are read while the current two multiply;
//   * E8M0 scales ride along: A scales sit in LDS as [g][row%16][row/16] so that one 16-byte read
//     gives a lane the scales of 16 row tiles (selected with op_sel); B scales are 4 bytes per lane
//     per K slice straight from global.
// The gate/up epilogue computes act(gate)*up in registers (a pair of lanes holds gate and up of the
// same elements and exchanges them) and passes the products through LDS so that the MX
// re-quantisation sees the reference's blocks (8 partitions x 4 q) and writes K-contiguous rows for
// the down GEMM.
//
// Reference semantics: test/integration/nkilib/core/mlp/test_mlp_common.py:550-682 (layouts,
// re-quantisation), test/integration/nkilib/core/moe/moe_cte/test_utils.py:474-735 (block loop).
#include <type_traits>

#include "bwmm.hpp"

namespace moe {

constexpr int MXT = 256;                       // threads
constexpr int MX_ROWS_MAX = CHUNK_ROWS_MAX;    // rows of the largest chunk (320)
constexpr int MXROW = 128;                     // LDS pitch of one staged row; 16-byte chunk ch of row r sits in
                                               // slot ch ^ (r & 7), which makes the fragment reads (16 rows x 4
                                               // chunks per instruction) and the staging writes conflict free
constexpr int MX_EP = 128 + 8;                 // epilogue exchange: floats per row ([q][32 partitions] + pad)
// Per variant (NMT row tiles): how many slices the loads run ahead, the ring of activation stages, and
// the bytes of one stage.  Chunks of up to 256 rows: 3 slices ahead, 4 stages of 256 rows.  Chunks of
// 257..320 rows (an expert's usual load plus a small excess, which would otherwise cost a second pass
// over the expert's weights): 2 slices ahead, 3 stages of 320 rows -- the 64 extra accumulators
// live in ordinary registers, which leaves room for two raw weight sets, not three.
template <int NMT>
struct MxCfg {
  static constexpr int D = NMT > 16 ? 2 : 3;          // slices between a load and its use
  static constexpr int RING = D + 1;                  // activation stages
  static constexpr int ROWS = NMT > 16 ? 320 : 256;   // rows of a stage
  static constexpr int SA = ROWS * MXROW;             // bytes of a stage's rows
  static constexpr int SSP = NMT > 16 ? 32 : 16;      // scale bytes per (K block, row within tile): one per row tile
  static constexpr int SS = 64 * SSP;                 // bytes of a stage's scales, [g][c][mt]
  static constexpr int LDS = RING * (SA + SS);
};
constexpr int MX_LDS_LOOP = MxCfg<16>::LDS > MxCfg<20>::LDS ? MxCfg<16>::LDS : MxCfg<20>::LDS;
constexpr int MX_LDS_EPI = 64 * MX_EP * 4;
constexpr int MX_LDS = MX_LDS_EPI > MX_LDS_LOOP ? MX_LDS_EPI : MX_LDS_LOOP;

template <int I, int N, class F>
__device__ __forceinline__ void static_for(F&& f) {
  if constexpr (I < N) {
    f(std::integral_constant<int, I>{});
    static_for<I + 1, N>(f);
  }
}

template <class Operand>
struct BFrag {
  Operand f[4];  // four column tiles (8 registers each for 8-bit weights, 4 for 4-bit ones)
  int sc;        // their E8M0 scale bytes (byte t = tile t)
};

__device__ __forceinline__ v8i frag_from_lds(const uint8_t* plo, const uint8_t* phi) {
  const v4i lo = *(const v4i*)plo;
  const v4i hi = *(const v4i*)phi;
  v8i r;
  r[0] = lo[0]; r[1] = lo[1]; r[2] = lo[2]; r[3] = lo[3];
  r[4] = hi[0]; r[5] = hi[1]; r[6] = hi[2]; r[7] = hi[3];
  return r;
}

// The accumulators live in fixed accumulation registers that only the statements below name: tile
// (mt, nt) of a wave's 16 x 4 tiles is a[16 mt + 4 nt .. + 3].  They are not C++ values, so the
// compiler never moves, copies or spills them (it would do so without the wait that a read of an
// MFMA result needs: it does not know these statements as MFMAs).  Every accumulation register is
// declared clobbered at both ends of each K slice, so the compiler keeps nothing of its own there.
#define MX_A10(p) "a" #p "0", "a" #p "1", "a" #p "2", "a" #p "3", "a" #p "4", "a" #p "5", "a" #p "6", "a" #p "7", "a" #p "8", "a" #p "9"
#define MX_ALL_ACC                                                                                               \
  "a0", "a1", "a2", "a3", "a4", "a5", "a6", "a7", "a8", "a9", MX_A10(1), MX_A10(2), MX_A10(3), MX_A10(4),        \
      MX_A10(5), MX_A10(6), MX_A10(7), MX_A10(8), MX_A10(9), MX_A10(10), MX_A10(11), MX_A10(12), MX_A10(13),     \
      MX_A10(14), MX_A10(15), MX_A10(16), MX_A10(17), MX_A10(18), MX_A10(19), MX_A10(20), MX_A10(21), MX_A10(22), \
      MX_A10(23), MX_A10(24), "a250", "a251", "a252", "a253", "a254", "a255"
__device__ __forceinline__ void acc_fence() { asm volatile("" ::: MX_ALL_ACC); }
template <int I>
__device__ __forceinline__ void acc_zero() {
  asm volatile("v_accvgpr_write_b32 a[%0], 0" : : "n"(I));
}
template <int I>
__device__ __forceinline__ float acc_get() {
  float x;
  asm volatile("v_accvgpr_read_b32 %0, a[%1]" : "=v"(x) : "n"(I));
  return x;
}
// One MFMA of row-tile fragment `af` (scale byte OA of `sa`) with column tile NT of `b`, written as
// an instruction: statements of this kind keep their order, so what the source puts between two
// MFMAs (a load, an LDS read) is issued between them and runs in the shadow of the first -- with one
// wave per SIMD nothing else hides it.  op_sel / op_sel_hi carry bit 0 / bit 1 of the two scale
// byte selectors.
// WFMT: element format of the weights (B operand): 0 = e4m3, 1 = e5m2 (blgp:1), 2 = e2m1 (blgp:4; 4-bit
// elements: the operand is four registers, lane group g holding K 32g .. 32g+31, eight to a register).
#define MX_MFMA_ASM(FMT_, SEL_, SELHI_)                                                                          \
  asm volatile("v_mfma_scale_f32_16x16x128_f8f6f4 a[%0:%1], %2, %3, a[%0:%1], %4, %5 op_sel:" SEL_ " op_sel_hi:" SELHI_ FMT_ \
               : : "n"(ACC), "n"(ACC + 3), "v"(af), "v"(bf), "v"(sa), "v"(sb))
#define MX_MFMA_CASE(OA_, OB_, SEL_, SELHI_)               \
  if constexpr (OA == OA_ && OB == OB_) {                  \
    if constexpr (WFMT == 0) MX_MFMA_ASM("", SEL_, SELHI_); \
    else if constexpr (WFMT == 1) MX_MFMA_ASM(" blgp:1", SEL_, SELHI_); \
    else MX_MFMA_ASM(" blgp:4", SEL_, SELHI_);             \
  }
template <int ACC, int OA, int OB, int WFMT, class BOp>
__device__ __forceinline__ void mfma_asm(const v8i& af, const BOp& bf, int sa, int sb) {
  MX_MFMA_CASE(0, 0, "[0,0,0]", "[0,0,0]");
  MX_MFMA_CASE(1, 0, "[1,0,0]", "[0,0,0]");
  MX_MFMA_CASE(2, 0, "[0,0,0]", "[1,0,0]");
  MX_MFMA_CASE(3, 0, "[1,0,0]", "[1,0,0]");
  MX_MFMA_CASE(0, 1, "[0,1,0]", "[0,0,0]");
  MX_MFMA_CASE(1, 1, "[1,1,0]", "[0,0,0]");
  MX_MFMA_CASE(2, 1, "[0,1,0]", "[1,0,0]");
  MX_MFMA_CASE(3, 1, "[1,1,0]", "[1,0,0]");
  MX_MFMA_CASE(0, 2, "[0,0,0]", "[0,1,0]");
  MX_MFMA_CASE(1, 2, "[1,0,0]", "[0,1,0]");
  MX_MFMA_CASE(2, 2, "[0,0,0]", "[1,1,0]");
  MX_MFMA_CASE(3, 2, "[1,0,0]", "[1,1,0]");
  MX_MFMA_CASE(0, 3, "[0,1,0]", "[0,1,0]");
  MX_MFMA_CASE(1, 3, "[1,1,0]", "[0,1,0]");
  MX_MFMA_CASE(2, 3, "[0,1,0]", "[1,1,0]");
  MX_MFMA_CASE(3, 3, "[1,1,0]", "[1,1,0]");
}
#undef MX_MFMA_CASE
#undef MX_MFMA_ASM
// The same with the accumulator tile in ordinary registers (row tiles 16..19 of a 320-row chunk).
#define MX_MFMA_ASM(FMT_, SEL_, SELHI_)                                                                        \
  asm volatile("v_mfma_scale_f32_16x16x128_f8f6f4 %0, %1, %2, %0, %3, %4 op_sel:" SEL_ " op_sel_hi:" SELHI_ FMT_ \
               : "+v"(c) : "v"(af), "v"(bf), "v"(sa), "v"(sb))
#define MX_MFMA_CASE(OA_, OB_, SEL_, SELHI_)               \
  if constexpr (OA == OA_ && OB == OB_) {                  \
    if constexpr (WFMT == 0) MX_MFMA_ASM("", SEL_, SELHI_); \
    else if constexpr (WFMT == 1) MX_MFMA_ASM(" blgp:1", SEL_, SELHI_); \
    else MX_MFMA_ASM(" blgp:4", SEL_, SELHI_);             \
  }
template <int OA, int OB, int WFMT, class BOp>
__device__ __forceinline__ void mfma_asm_v(v4f& c, const v8i& af, const BOp& bf, int sa, int sb) {
  MX_MFMA_CASE(0, 0, "[0,0,0]", "[0,0,0]");
  MX_MFMA_CASE(1, 0, "[1,0,0]", "[0,0,0]");
  MX_MFMA_CASE(2, 0, "[0,0,0]", "[1,0,0]");
  MX_MFMA_CASE(3, 0, "[1,0,0]", "[1,0,0]");
  MX_MFMA_CASE(0, 1, "[0,1,0]", "[0,0,0]");
  MX_MFMA_CASE(1, 1, "[1,1,0]", "[0,0,0]");
  MX_MFMA_CASE(2, 1, "[0,1,0]", "[1,0,0]");
  MX_MFMA_CASE(3, 1, "[1,1,0]", "[1,0,0]");
  MX_MFMA_CASE(0, 2, "[0,0,0]", "[0,1,0]");
  MX_MFMA_CASE(1, 2, "[1,0,0]", "[0,1,0]");
  MX_MFMA_CASE(2, 2, "[0,0,0]", "[1,1,0]");
  MX_MFMA_CASE(3, 2, "[1,0,0]", "[1,1,0]");
  MX_MFMA_CASE(0, 3, "[0,1,0]", "[0,1,0]");
  MX_MFMA_CASE(1, 3, "[1,1,0]", "[0,1,0]");
  MX_MFMA_CASE(2, 3, "[0,1,0]", "[1,1,0]");
  MX_MFMA_CASE(3, 3, "[1,1,0]", "[1,1,0]");
}
#undef MX_MFMA_CASE
#undef MX_MFMA_ASM

// Raw buffer descriptor over [p, p + bytes): loads take a per-lane 32-bit byte offset (VGPR) plus a
// wave-uniform 32-bit byte offset (SGPR), which is exactly the shape of every address in this
// kernel, so no 64-bit per-lane pointer is ever formed.
// (The descriptor and the uniform offsets are passed through readfirstlane: 64-bit address
// arithmetic on uniform values is done by the vector ALU, and without the hint the compiler wraps
// every load in a loop that checks whether all lanes agree on the descriptor.)
__device__ __forceinline__ int uni(int v) { return __builtin_amdgcn_readfirstlane(v); }
__device__ __forceinline__ int uni(int64_t v) { return __builtin_amdgcn_readfirstlane((int)v); }
__device__ __forceinline__ v4i make_rsrc(const void* p, uint32_t bytes) {
  const uint64_t addr = (uint64_t)p;
  v4i d;
  d[0] = uni((int)(uint32_t)addr);
  d[1] = uni((int)(uint32_t)(addr >> 32)) & 0xffff;  // stride 0: raw buffer
  d[2] = uni((int)bytes);
  d[3] = 0x00020000;
  return d;
}
// The K loop's loads are written as instructions, not builtins: the compiler orders the results of
// its own loads with a counter that completes in order, and places those waits as if every load it
// can see on any path had just been issued -- which with two alternating weight sets means waiting
// for the set that was only just requested.  Loads the compiler cannot see get no waits from it;
// the waits are placed by hand where the data is first used (vm_wait).  The destination is an
// in/out operand so that the load updates the variable's register in place.
// NT: non-temporal, for data that nobody will ask the L2 for again.
template <bool NT>
__device__ __forceinline__ void ld_b128(v4i& d, uint32_t voff, const v4i& rsrc, int soff) {
  if constexpr (NT)
    asm volatile("buffer_load_dwordx4 %0, %1, %2, %3 offen nt" : "+v"(d) : "v"(voff), "s"(rsrc), "s"(soff) : "memory");
  else
    asm volatile("buffer_load_dwordx4 %0, %1, %2, %3 offen" : "+v"(d) : "v"(voff), "s"(rsrc), "s"(soff) : "memory");
}
__device__ __forceinline__ void st_b64(const v2i& d, uint32_t voff, const v4i& rsrc, int soff) {
  asm volatile("buffer_store_dwordx2 %0, %1, %2, %3 offen nt" : : "v"(d), "v"(voff), "s"(rsrc), "s"(soff) : "memory");
}
// 16 bytes per lane straight into LDS at lds + 16 * lane (no destination registers).  The instruction takes its
// LDS base from M0, which is set in the same statement.  M0 is declared clobbered: the compiler warns that it
// does not save reserved registers around a statement, which is what is wanted here -- on this target it never
// carries a value in M0 from one instruction to the next (it writes M0 itself immediately before each instruction
// of its own that reads it), so there is nothing to save.
__device__ __forceinline__ void ld_lds_b128(uint32_t lds, uint32_t voff, const v4i& rsrc, int soff) {
  asm volatile("s_mov_b32 m0, %0\n\tbuffer_load_dwordx4 %1, %2, %3 offen lds"
               : : "s"(lds), "v"(voff), "s"(rsrc), "s"(soff) : "memory", "m0");
}
template <bool NT>
__device__ __forceinline__ void ld_b64(v2i& d, uint32_t voff, const v4i& rsrc, int soff) {
  if constexpr (NT)
    asm volatile("buffer_load_dwordx2 %0, %1, %2, %3 offen nt" : "+v"(d) : "v"(voff), "s"(rsrc), "s"(soff) : "memory");
  else
    asm volatile("buffer_load_dwordx2 %0, %1, %2, %3 offen" : "+v"(d) : "v"(voff), "s"(rsrc), "s"(soff) : "memory");
}
typedef int v3i __attribute__((ext_vector_type(3)));
__device__ __forceinline__ void ld_dwords(v3i& d, uint32_t voff, const v4i& rsrc, int soff) {
  asm volatile("buffer_load_dwordx3 %0, %1, %2, %3 offen" : "+v"(d) : "v"(voff), "s"(rsrc), "s"(soff) : "memory");
}
__device__ __forceinline__ void ld_dwords(v2i& d, uint32_t voff, const v4i& rsrc, int soff) {
  asm volatile("buffer_load_dwordx2 %0, %1, %2, %3 offen" : "+v"(d) : "v"(voff), "s"(rsrc), "s"(soff) : "memory");
}
__device__ __forceinline__ void ld_b32(int& d, uint32_t voff, const v4i& rsrc, int soff) {
  asm volatile("buffer_load_dword %0, %1, %2, %3 offen" : "+v"(d) : "v"(voff), "s"(rsrc), "s"(soff) : "memory");
}

// NMT = number of 16-row tiles this instantiation multiplies (the chunk has at most NMT*16 rows).
// Keeping it a compile-time constant keeps the K loop free of branches around the MFMAs.
// LASTUSE: this chunk is the last one of its expert, so its weights are streamed past the L2 (which
// then keeps the activation tiles that the sibling workgroups share); an earlier chunk loads them
// normally, for the chunk after it to find.
template <int STAGE, int NMT, bool LASTUSE, int WFMT>
__device__ __forceinline__ void mx_gemm_body(const MxArgs& a, uint8_t* smem, int* s_tok, float* s_aff, int nrows, int e,
                                             int64_t slot0, int xt) {
  using Cfg = MxCfg<NMT>;
  constexpr int D = Cfg::D, RING = Cfg::RING, SA = Cfg::SA, SS = Cfg::SS, SSP = Cfg::SSP;
  constexpr bool BIG = NMT > 16;  // row tiles 16.. accumulate in ordinary registers
  uint8_t* sA = smem;
  uint8_t* sS = smem + RING * SA;
  // ring arithmetic: x in [0, 2 RING)
  auto wrapst = [](int x) { return (RING == 4) ? (x & 3) : ((x >= RING) ? x - RING : x); };

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int w = __builtin_amdgcn_readfirstlane(tid >> 6);  // wave index, kept scalar
  const int c = lane & 15, g = lane >> 4;
  const int64_t nH = a.H / 512;

  // ---- column tile ---------------------------------------------------------------------------
  int tI = 0, p0 = 0, Pt = 128;
  int64_t h0 = 0;
  if (STAGE == 1) {
    tI = xt >> 2;
    p0 = (xt & 3) * 32;
    const int64_t rows_t = (a.I - (int64_t)tI * 512 < 512) ? (a.I - (int64_t)tI * 512) : 512;
    Pt = (int)(rows_t / 4);
    if (p0 >= Pt) return;  // whole workgroup: Pt is a multiple of 32 on this path
  } else {
    h0 = (int64_t)xt * 256;
  }
  const int q = w;

  // ---- rows: token ids, affinities ---------------------------------------------------------------
  for (int r = tid; r < NMT * 16; r += MXT) {
    int id = -1;
    if (r < nrows) {
      id = a.tp2id[slot0 + r];
      if (id < 0 || id >= a.n_real) id = -1;
    }
    s_tok[r] = id;
    if (STAGE == 2) {
      float af = 0.f;
      if (id >= 0 && a.aff)
        af = (a.aff_dtype == MOE_DT_BF16) ? bf16_bits_to_f32(((const uint16_t*)a.aff)[(int64_t)id * a.E + e])
                                          : ((const float*)a.aff)[(int64_t)id * a.E + e];
      s_aff[r] = af;
    }
  }
  __syncthreads();

  // A staging: thread covers rows (tid>>3) + 32 j; its load goes straight to LDS slot tid&7 of that
  // row and fetches the 16-byte chunk (tid&7) ^ (row&7) that belongs there
  const int arow0 = tid >> 3, ach = tid & 7;
  constexpr int NAJ = NMT / 2;  // 32-row groups that hold rows of the NMT tiles
  // Per-lane 32-bit byte offsets (row * stride + chunk); the K offset is wave-uniform and is added
  // to the scalar base, so a load needs one VGPR of address.  Rows without a token (padding
  // slots, rows past the end of the chunk) read some valid row instead of being zeroed: rows are
  // independent in a GEMM and the results of such rows are never written out, so what they hold
  // does not matter -- and the loads stay free of branches.
  uint32_t a_voff[NAJ];
#pragma unroll
  for (int j = 0; j < NAJ; ++j) {
    const int row = arow0 + 32 * j;
    uint32_t r;
    if (STAGE == 1) {
      const int tok = s_tok[row];
      r = (tok >= 0) ? (uint32_t)tok : 0u;
    } else {
      r = (uint32_t)(slot0 + ((row < nrows) ? row : (nrows - 1)));
    }
    a_voff[j] = r * (uint32_t)a.a_stride + (uint32_t)((ach ^ (arow0 & 7)) * 16);
  }
  // A scales: thread covers row tid (and, in a chunk of more than 256 rows, row 256 + tid % 64: every
  // wave issues that load so that all waves count the same loads, the first wave's is used)
  auto scale_row_off = [&](int row) {
    if (STAGE == 1) {
      const int tok = s_tok[row];
      return ((tok >= 0) ? (uint32_t)tok : 0u) * (uint32_t)a.a_scale_stride;
    }
    return (uint32_t)(slot0 + ((row < nrows) ? row : (nrows - 1))) * (uint32_t)a.a_scale_stride;
  };
  const uint32_t as_voff = scale_row_off(tid);
  const uint32_t as_voff2 = BIG ? scale_row_off(256 + (tid & 63)) : 0u;
  // where the scales of row 256 + tid go: the other waves' copies land in a row tile that does not
  // exist (no branch inside the K loop: values that cross one stop being known as uniform)
  const int row_hi = (tid < 64) ? 256 + tid : 31 * 16 + (tid & 15);

  // ---- K schedule -----------------------------------------------------------------------------------
  // stage 1: ks -> (H tile ks>>2, partition group ks&3), all slices full.
  // stage 2: slices of intermediate tile t are the first Pt(t)/32 partition groups; only the last
  // tile can be short and its slices come last, so ks -> (ks>>2, ks&3) holds for both.
  int nks;
  if (STAGE == 1) {
    nks = (int)(a.H / 128);
  } else {
    const int64_t tail = a.I % 512;
    nks = (int)((a.I / 512) * 4 + (tail / 128));
  }

  // ---- B operand addressing ---------------------------------------------------------------------------
  // byte address inside the expert's weights = uniform part (gate/up, K tile, partition
  // 32*pb + {r | 16 + r}, first column of the wave) + per-lane part (partition 4g, lane's columns).
  int64_t w_pstride, w_tstride;  // element strides (4-byte weights; scales use the same counts in bytes)
  v4i rw_, rs_;
  uint32_t w_voff, s_voff;
  int64_t colu;
  // A lane loads 16 bytes = 4 adjacent columns of one K row: column 4*cl + t belongs to column tile
  // t.  In the gate/up stage the wave's 32 gate columns take lanes c = 0..7 of each group and its 32
  // up columns lanes c = 8..15, so every column tile is half gate, half up, and one load instruction
  // fetches 128 contiguous bytes of gate and of up for 4 K rows.  (8-byte loads, one tile pair per
  // load, cost the memory pipeline as much per instruction as 16-byte ones.)
  const int hcol = (STAGE == 1) ? (c >> 3) : 0, cl = (STAGE == 1) ? (c & 7) : c;
  // 4-bit weights (x4: four K values in a 2-byte element): lane group g needs K 32g .. 32g+31 of the
  // slice = partitions 8g .. 8g+7, one 8-byte load (4 columns) per partition; 8-bit weights (4-byte
  // elements): partitions 4g .. 4g+3 and 16+4g .. 16+4g+3, one 16-byte load each.
  constexpr bool FP4 = WFMT == 2;
  constexpr int ES = FP4 ? 2 : 4;      // bytes of a weight element
  constexpr int GROWS = FP4 ? 8 : 4;   // partition rows between the lane groups' first rows
  const uint8_t* Wb = (const uint8_t*)a.W;
  if (STAGE == 1) {
    w_pstride = 2 * nH * a.I;
    w_tstride = a.I;
    colu = (int64_t)tI * 512 + (int64_t)q * Pt + p0;
    rw_ = make_rsrc(Wb + (int64_t)e * 128 * w_pstride * ES, (uint32_t)(128 * w_pstride * ES));
    rs_ = make_rsrc(a.W_scale + (int64_t)e * 16 * w_pstride, (uint32_t)(16 * w_pstride));
    w_voff = (uint32_t)((GROWS * g * w_pstride + hcol * nH * a.I + 4 * cl) * ES);
    s_voff = (uint32_t)(g * w_pstride + hcol * nH * a.I + 4 * cl);
  } else {
    w_pstride = (int64_t)a.nI * a.H;
    w_tstride = a.H;
    colu = h0 + 64 * q;
    const int64_t sp = (a.pI + 7) / 8;
    rw_ = make_rsrc(Wb + (int64_t)e * a.pI * w_pstride * ES, (uint32_t)(a.pI * w_pstride * ES));
    rs_ = make_rsrc(a.W_scale + (int64_t)e * sp * w_pstride, (uint32_t)(sp * w_pstride));
    w_voff = (uint32_t)((GROWS * g * w_pstride + 4 * c) * ES);
    s_voff = (uint32_t)(g * w_pstride + 4 * c);
  }

  // A K slice's loads, numbered in issue order:
  //   0 .. NAJ-1            activation rows (16 bytes per lane each, straight into the LDS ring)
  //   NAJ .. NAJ+NSC-1      activation scales of D slices (4 D bytes per lane, into registers), only in the
  //                         first slice of every D
  //   then NBL              weights (16 bytes per lane each, into a raw register set)
  //   then 1                weight scales
  constexpr int NBL = 8;
  constexpr int NSC = BIG ? 2 : 1;
  constexpr int NLB = NBL + 1;              // weight loads of a slice
  constexpr int N1 = NAJ + NLB;             // loads of a slice that carries no activation scales
  constexpr int N0 = N1 + NSC;              // loads of one that does
  typedef typename std::conditional<D == 3, v3i, v2i>::type ScaleRegs;
  typedef typename std::conditional<FP4, v2i, v4i>::type RawLoad;
  typedef typename std::conditional<FP4, v4i, v8i>::type BOperand;
  struct BRaw {
    RawLoad d[NBL];
    int sc;
  };
  const v4i ra_ = make_rsrc(a.A, 0xffffffffu), ras_ = make_rsrc(a.A_scale, (uint32_t)(a.a_rows * a.a_scale_stride));
  // Scalar byte offset of a weight load = (offset of its row and column within the slice, fixed per
  // load and kept in scalar registers) + (offset of the slice, computed once per slice): one scalar
  // add per load.  Address arithmetic done per load costs more issue cycles than the MFMAs between
  // two loads take.
  int w_soff[NBL];
#pragma unroll
  for (int i = 0; i < NBL; ++i) {
    const int pr = FP4 ? i : ((i < 4) ? i : (16 + i - 4));
    w_soff[i] = uni(((int64_t)pr * w_pstride + colu) * ES);
  }
  const int s_soff = uni(colu);
  // Everything a slice's loads share: descriptors (of zero records past the end: such a load is out
  // of range, fetches nothing and returns zeros, so the K loop needs no conditions around its loads)
  // and the slice's scalar offsets.
  struct SliceAddr {
    v4i ra, ras, rw, rs;
    int a_off, as_off, w_off, s_off;
    uint32_t lds_a;  // LDS address of the ring stage that receives this slice's activations
  };
  const uint32_t lds_ring = (uint32_t)(uintptr_t)sA;
  auto slice_addr = [&](int ks, int st) {
    SliceAddr r;
    r.lds_a = uni((int)(lds_ring + (uint32_t)st * SA));
    const int live = (ks < nks) ? -1 : 0;
    auto sel = [&](const v4i& d) {
      v4i x;
      x[0] = uni(d[0]);
      x[1] = uni(d[1]);
      x[2] = uni(d[2] & live);
      x[3] = uni(d[3]);
      return x;
    };
    r.ra = sel(ra_); r.ras = sel(ras_); r.rw = sel(rw_); r.rs = sel(rs_);
    const int kt = ks >> 2, pb = ks & 3;
    r.a_off = ks * 128;
    r.as_off = ks * 4;
    r.w_off = uni(((int64_t)(pb * 32) * w_pstride + (int64_t)kt * w_tstride) * ES);
    r.s_off = uni((int64_t)(pb * 4) * w_pstride + (int64_t)kt * w_tstride);
    return r;
  };
  auto issue_load = [&](auto idx_, const SliceAddr& sa, BRaw& b, ScaleRegs& sc0, ScaleRegs& sc1, auto with_scales_) {
    constexpr int idx = decltype(idx_)::value;
    if constexpr (idx < NAJ) {
      // the wave's 64 lanes fill 8 rows x 128 bytes = 1 KB of the ring stage, in lane order
      ld_lds_b128(sa.lds_a + (uint32_t)((w * 8 + 32 * idx) * MXROW), a_voff[idx], sa.ra, sa.a_off);
    } else if constexpr (idx < NAJ + NSC) {
      // the four scale bytes (K blocks) of a row, for this slice and the D-1 after it: a lane's
      // dwords sit in different cache lines, so this load costs the memory pipeline as many
      // requests as all the activation rows of a slice together -- hence one in D slices
      if constexpr (decltype(with_scales_)::value) {
        if constexpr (idx == NAJ) ld_dwords(sc0, as_voff, sa.ras, sa.as_off);
        else ld_dwords(sc1, as_voff2, sa.ras, sa.as_off);
      }
    } else if constexpr (idx < NAJ + NSC + NBL) {
      constexpr int i = idx - NAJ - NSC;
      if constexpr (FP4) ld_b64<LASTUSE>(b.d[i], w_voff, sa.rw, w_soff[i] + sa.w_off);
      else ld_b128<LASTUSE>(b.d[i], w_voff, sa.rw, w_soff[i] + sa.w_off);
    } else {
      ld_b32(b.sc, s_voff, sa.rs, s_soff + sa.s_off);
    }
  };
  // The MFMA wants a lane's scale byte to be that of row 16*mt + c and K block g, one byte per row
  // tile: [g][c][mt], so that one 16-byte read gives a lane the scales of all 16 row tiles.  A
  // thread loads the scale bytes of row tid and puts them in place.
  auto scales_to_operand_order = [&](int st, uint32_t raw, int row) {
    uint8_t* sd = sS + st * SS;
    const int mt = row >> 4, cc = row & 15;
#pragma unroll
    for (int gg = 0; gg < 4; ++gg) sd[(gg * 16 + cc) * SSP + mt] = (uint8_t)((raw >> (8 * gg)) & 0xffu);
  };

  acc_fence();
  static_for<0, (BIG ? 16 : NMT) * 16>([&](auto i_) { acc_zero<decltype(i_)::value>(); });
  v4f accv[4][4];  // row tiles 16..19
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) accv[i][j] = (v4f){0.f, 0.f, 0.f, 0.f};

  // ---- K loop ---------------------------------------------------------------------------------------
  // Loads run D slices ahead of the MFMAs (what the memory system delivers is the amount in flight
  // divided by its latency, and one wave per SIMD has nobody to take over while it waits): during
  // slice ks the loads of slice ks+D are issued, one after every second or third MFMA, the
  // activations into ring stage (ks+D) % RING (last read in slice ks-1, which every wave left before
  // the barrier that ended it), the weights into raw register set ks % D, which was transposed into
  // MFMA operand order at the top of this slice.  A wave's loads complete in issue order, so a wait
  // names how many of the most recent ones may still be out.  At the top of slice ks the weights of
  // slice ks must be in and, next in line, the activations of slice ks+1 (issued since: the weights
  // of slice ks+1 and all of the slices after it); the barrier at the end of the slice publishes
  // them to the other waves.  The activation scales of D slices arrive together in the first slice
  // of every D and are re-ordered into the stages of the next D slices during the last.  The loop
  // body is written out D times so that the raw set of a slice is a compile-time choice.
  const int rd_lo = c * MXROW + ((g ^ (c & 7)) * 16), rd_hi = c * MXROW + (((g + 4) ^ (c & 7)) * 16);
  constexpr int NG = NMT / 2;
  BRaw br[D];
  ScaleRegs asr = 0, asr2 = 0;  // activation scales as loaded: row tid, row 256 + tid % 64
  static_for<0, D>([&](auto u_) {
    constexpr int u = decltype(u_)::value;
#pragma unroll
    for (int j = 0; j < NBL; ++j) br[u].d[j] = 0;
    br[u].sc = 0;
  });
  auto slice = [&](auto u_, int ks, int st) {
    constexpr int U = decltype(u_)::value;
    BRaw& braw = br[U];
    acc_fence();
    const uint8_t* plo = sA + st * SA + rd_lo;
    const uint8_t* phi = sA + st * SA + rd_hi;
    const v4i asc = *(const v4i*)(sS + st * SS + (g * 16 + c) * SSP);
    int asc_hi = 0;
    if constexpr (BIG) asc_hi = *(const int*)(sS + st * SS + (g * 16 + c) * SSP + 16);
    // first fragments of this slice: in flight while the weights are transposed
    v8i af[2][2];
    af[0][0] = frag_from_lds(plo, phi);
    af[0][1] = frag_from_lds(plo + 16 * MXROW, phi + 16 * MXROW);
    asm volatile("" ::: "memory");
    asm volatile("s_waitcnt vmcnt(%0)" : : "n"(NLB + (D - 2) * N1) : "memory");
    if constexpr (U == D - 1) {  // activation scales of slices ks+1 .. ks+D
      asm volatile("" : "+v"(asr));
      if constexpr (BIG) asm volatile("" : "+v"(asr2));
    }
    // (the wait names no register: an in/out operand may be copied into place ahead of its
    // statement, i.e. read while its load is still in flight; the registers are tied to this point
    // by statements of their own)
#pragma unroll
    for (int j = 0; j < NBL; ++j) asm volatile("" : "+v"(braw.d[j]));
    asm volatile("" : "+v"(braw.sc));
    // one load gives a lane the same K row (partition) of 4 column tiles; an MFMA wants the K rows of
    // one tile in consecutive registers (8-bit: one register per partition; 4-bit: two partitions,
    // 16 bits each, per register)
    BFrag<BOperand> b;
    if constexpr (FP4) {
#pragma unroll
      for (int r = 0; r < 4; ++r) {
#pragma unroll
        for (int t = 0; t < 4; ++t) {
          const uint32_t lo = (uint32_t)braw.d[2 * r][t >> 1], hi = (uint32_t)braw.d[2 * r + 1][t >> 1];
          // low halves (even tile) or high halves (odd tile) of the two partitions' dwords
          b.f[t][r] = (int)__builtin_amdgcn_perm(hi, lo, (t & 1) ? 0x07060302u : 0x05040100u);
        }
      }
    } else {
#pragma unroll
      for (int r = 0; r < 8; ++r) {
        b.f[0][r] = braw.d[r][0];
        b.f[1][r] = braw.d[r][1];
        b.f[2][r] = braw.d[r][2];
        b.f[3][r] = braw.d[r][3];
      }
    }
    b.sc = braw.sc;
    asm volatile("s_nop 1" : "+v"(b.f[0]), "+v"(b.f[1]), "+v"(b.f[2]), "+v"(b.f[3]), "+v"(b.sc));
    SliceAddr sad;
    static_for<0, NG>([&](auto gi_) {
      constexpr int gi = decltype(gi_)::value;
      constexpr int cur = gi & 1, nxt = cur ^ 1;
      if constexpr (gi + 1 < NG) {
        af[nxt][0] = frag_from_lds(plo + (2 * gi + 2) * 16 * MXROW, phi + (2 * gi + 2) * 16 * MXROW);
        af[nxt][1] = frag_from_lds(plo + (2 * gi + 3) * 16 * MXROW, phi + (2 * gi + 3) * 16 * MXROW);
      }
      // Fixed point between "next group's reads issued" and "this group's MFMAs": the reads above
      // cannot sink below it (memory clobber) and the MFMAs below cannot rise above it (they use the
      // fragments it returns), so the two fragment sets stay live together and the LDS latency of
      // the next group is covered by this group's eight MFMAs.
      asm volatile("" : "+v"(af[cur][0]), "+v"(af[cur][1]) : : "memory");
      static_for<0, 8>([&](auto j_) {
        constexpr int j = decltype(j_)::value;
        constexpr int mt = 2 * gi + j / 4, nt = j % 4;
        constexpr int m = gi * 8 + j;  // MFMA number within the slice
        if constexpr (mt < 16)
          mfma_asm<16 * mt + 4 * nt, mt % 4, nt, WFMT>(af[cur][j / 4], b.f[nt], asc[mt / 4], b.sc);
        else
          mfma_asm_v<mt % 4, nt, WFMT>(accv[mt - 16][nt], af[cur][j / 4], b.f[nt], asc_hi, b.sc);
        if constexpr (m == 0) {
          // the scalar arithmetic for the addresses of slice ks+D starts here, behind the first
          // MFMA, instead of ahead of it
          int ksd = ks + D;
          asm volatile("" : "+s"(ksd));
          sad = slice_addr(ksd, wrapst(st + D));
        }
        if constexpr (U == D - 1 && m >= 3 && m < 3 + D) {
          scales_to_operand_order(wrapst(st + m - 2), (uint32_t)asr[m - 3], tid);
          if constexpr (BIG) scales_to_operand_order(wrapst(st + m - 2), (uint32_t)asr2[m - 3], row_hi);
        }
        static_for<m * N0 / (8 * NG), (m + 1) * N0 / (8 * NG)>(
            [&](auto i_) { issue_load(i_, sad, braw, asr, asr2, std::integral_constant<bool, U == 0>{}); });
      });
    });
    // (accumulators in ordinary registers are C++ values: should the compiler copy one where paths
    // join, the MFMA that wrote it has left the pipe)
    if constexpr (BIG) asm volatile("s_nop 15");
    acc_fence();
    __syncthreads();
  };

  // prologue: the first D slices are requested at once; slice 0 needs its activations
  static_for<0, D>([&](auto u_) {
    constexpr int u = decltype(u_)::value;
    const SliceAddr sa = slice_addr(u, u);
    static_for<0, N0>([&](auto i_) { issue_load(i_, sa, br[u], asr, asr2, std::integral_constant<bool, u == 0>{}); });
  });
  asm volatile("s_waitcnt vmcnt(%0)" : : "n"(NLB + (D - 1) * N1) : "memory");
  asm volatile("" : "+v"(asr));
  if constexpr (BIG) asm volatile("" : "+v"(asr2));
#pragma unroll
  for (int j = 0; j < D; ++j) {
    scales_to_operand_order(j, (uint32_t)asr[j], tid);
    if constexpr (BIG) scales_to_operand_order(j, (uint32_t)asr2[j], row_hi);
  }
  __syncthreads();
  int st = 0;
  int ks = 0;
#pragma clang loop unroll(disable)
  for (; ks + D <= nks; ks += D) {
    static_for<0, D>([&](auto u_) { slice(u_, ks + decltype(u_)::value, wrapst(st + decltype(u_)::value)); });
    st = wrapst(st + D);
  }
  static_for<0, D - 1>([&](auto u_) {
    if (ks + decltype(u_)::value < nks) slice(u_, ks + decltype(u_)::value, wrapst(st + decltype(u_)::value));
  });
  // the last MFMAs are still in the pipe, and nothing but the distance in instructions separates
  // them from the first read of an accumulator
  asm volatile("s_waitcnt vmcnt(0)\n\ts_nop 15\n\ts_nop 15" ::: "memory");
  // The loads of the slices past the end are never used, but they do arrive (as zeros): the registers
  // they were aimed at stay reserved until the wait above has passed.
#pragma unroll
  for (int u = 0; u < D; ++u) {
#pragma unroll
    for (int j = 0; j < NBL; ++j) asm volatile("" : : "v"(br[u].d[j]));
    asm volatile("" : : "v"(br[u].sc));
  }
  asm volatile("" : : "v"(asr), "v"(asr2));

  // ---- epilogue ---------------------------------------------------------------------------------------------
  if (STAGE == 1) {
    // act(gate + bias) * (up + bias) in registers, then through LDS, 64 rows at a time, as
    // [row][q][32 partitions] fp32; then one thread per MX block (8 partitions x 4 q) quantises and
    // writes 32 K-contiguous bytes plus the scale byte.
    float* E = (float*)smem;
    // the lane's four partitions within the workgroup's 32: 4*cl + t
    float bg[4] = {0.f, 0.f, 0.f, 0.f}, bu[4] = {0.f, 0.f, 0.f, 0.f};
    if (a.bias) {
#pragma unroll
      for (int t = 0; t < 4; ++t) {
        const int64_t p = p0 + 4 * cl + t;
        const int64_t ig = ((((int64_t)e * a.pI + p) * 2 + 0) * a.nI + tI) * 4 + q;
        const int64_t iu = ((((int64_t)e * a.pI + p) * 2 + 1) * a.nI + tI) * 4 + q;
        if (a.bias_dtype == MOE_DT_BF16) {
          bg[t] = bf16_bits_to_f32(((const uint16_t*)a.bias)[ig]);
          bu[t] = bf16_bits_to_f32(((const uint16_t*)a.bias)[iu]);
        } else {
          bg[t] = ((const float*)a.bias)[ig];
          bu[t] = ((const float*)a.bias)[iu];
        }
      }
    }
    const int pl0 = 4 * cl;
    constexpr int NPS = NMT / 4;
    // Clamps as unconditional min/max against +-inf, and the activation kind as a compile-time
    // constant of the pass: a lane evaluates 128 elements here, and per-element decisions made this
    // code longer (and slower) than the K loop.
    const float inf = __builtin_inff();
    const float g_lo = (a.clamp_mask & MOE_CLAMP_GATE_LO) ? a.clamp[1] : -inf;
    const float g_hi = (a.clamp_mask & MOE_CLAMP_GATE_HI) ? a.clamp[0] : inf;
    const float u_lo = (a.clamp_mask & MOE_CLAMP_UP_LO) ? a.clamp[3] : -inf;
    const float u_hi = (a.clamp_mask & MOE_CLAMP_UP_HI) ? a.clamp[2] : inf;
    auto passes = [&](auto act_) {
    constexpr int ACT = decltype(act_)::value;
    static_for<0, NPS>([&](auto ps_) {
      constexpr int ps = decltype(ps_)::value;
      if (ps * 64 < nrows) {
        __syncthreads();
        static_for<0, 4>([&](auto m_) {
          constexpr int ml = decltype(m_)::value;
          constexpr int mt = ps * 4 + ml;
          // Lane c < 8 holds gate, lane c + 8 up, of the same four partitions and the same four rows.
          // The pair splits the rows: the gate lane finishes rows 0,1 of its four, the up lane rows
          // 2,3; each hands the other the two values it needs (a rotation by 8 within the 16 lanes).
          float av[4][4];  // [column tile][row]
          static_for<0, 16>([&](auto i_) {
            constexpr int i = decltype(i_)::value;
            if constexpr (mt < 16) av[i / 4][i % 4] = acc_get<16 * mt + i>();
            else av[i / 4][i % 4] = accv[mt - 16][i / 4][i % 4];
          });
          float y[2][4];
#pragma unroll
          for (int t = 0; t < 4; ++t) {
#pragma unroll
            for (int k = 0; k < 2; ++k) {
              const float lo = av[t][k], hi = av[t][2 + k];
              const float mine = hcol ? hi : lo;
              const float send = hcol ? lo : hi;
              const float recv = __builtin_bit_cast(
                  float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, send), 0x128 /* row_ror:8 */, 0xf, 0xf, false));
              const float gv = hcol ? recv : mine, uv = hcol ? mine : recv;
              const float gg = fminf(fmaxf(gv + bg[t], g_lo), g_hi);
              const float uu = fminf(fmaxf(uv + bu[t], u_lo), u_hi);
              y[k][t] = act_apply(gg, ACT) * uu;
            }
          }
#pragma unroll
          for (int k = 0; k < 2; ++k) {
            const int rl = ml * 16 + 4 * g + 2 * hcol + k;
            *(float4*)(E + rl * MX_EP + q * 32 + pl0) = make_float4(y[k][0], y[k][1], y[k][2], y[k][3]);
          }
        });
        __syncthreads();
        // thread (rl = tid/4, j = tid%4): MX block of chunk row ps*64 + rl, partitions 8j .. 8j+7 of the 32 (x 4 q)
        const int rl = tid >> 2, j = tid & 3;
        const int row = ps * 64 + rl;
        if (row < nrows) {
          const float* src = E + rl * MX_EP + 8 * j;
          float yv[4][8];
          float am = 0.f;
#pragma unroll
          for (int qq = 0; qq < 4; ++qq) {
            const float4 lo = *(const float4*)(src + qq * 32), hi = *(const float4*)(src + qq * 32 + 4);
            yv[qq][0] = lo.x; yv[qq][1] = lo.y; yv[qq][2] = lo.z; yv[qq][3] = lo.w;
            yv[qq][4] = hi.x; yv[qq][5] = hi.y; yv[qq][6] = hi.z; yv[qq][7] = hi.w;
#pragma unroll
            for (int k = 0; k < 8; ++k) am = fmaxf(am, fabsf(yv[qq][k]));
          }
          const uint32_t sb = mx_scale_byte(am);
          const float is = mx_inv_scale(sb);
          uint32_t d[8];
#pragma unroll
          for (int k = 0; k < 8; ++k)
            d[k] = pack4_e4m3(clip448(yv[0][k] * is), clip448(yv[1][k] * is), clip448(yv[2][k] * is), clip448(yv[3][k] * is));
          const int64_t slot = slot0 + row;
          const int pw = p0 + 8 * j;  // first partition of the block within the intermediate tile
          uint4* o = (uint4*)(a.Yq + slot * a.y_stride + tI * 512 + pw * 4);
          o[0] = make_uint4(d[0], d[1], d[2], d[3]);
          o[1] = make_uint4(d[4], d[5], d[6], d[7]);
          a.Ys[slot * a.ys_stride + tI * 16 + (pw >> 3)] = (uint8_t)sb;
        }
      }
    });
    };
    switch (a.act_fn) {
      case MOE_ACT_SILU: passes(std::integral_constant<int, MOE_ACT_SILU>{}); break;
      case MOE_ACT_GELU: passes(std::integral_constant<int, MOE_ACT_GELU>{}); break;
      case MOE_ACT_GELU_TANH: passes(std::integral_constant<int, MOE_ACT_GELU_TANH>{}); break;
      default: passes(std::integral_constant<int, MOE_ACT_SWISH>{}); break;
    }
  } else {
    const int64_t col0 = h0 + 64 * q + 4 * c;
    float bd[4] = {0.f, 0.f, 0.f, 0.f};
    if (a.bias) {
#pragma unroll
      for (int t = 0; t < 4; ++t) {
        const int64_t ib = (int64_t)e * a.H + col0 + t;
        bd[t] = (a.bias_dtype == MOE_DT_BF16) ? bf16_bits_to_f32(((const uint16_t*)a.bias)[ib]) : ((const float*)a.bias)[ib];
      }
    }
    const bool post = a.scaling_mode == MOE_SCALE_POST;
    // Rows go out through a descriptor that ends after the chunk's last row, so rows past the end
    // are dropped by the range check and the stores need no branches.  (Rows of padding slots
    // inside the chunk are written too: nothing reads the contributions of such slots.)
    const v4i rd = make_rsrc(a.D + slot0 * a.H, (uint32_t)((int64_t)nrows * a.H * 2));
    const uint32_t d_voff = (uint32_t)((4 * g * a.H + col0) * 2);
    const int rowb = uni(a.H * 2);
    typedef __bf16 v2bf __attribute__((ext_vector_type(2)));
    typedef float v2f __attribute__((ext_vector_type(2)));
    // the affinities of the lane's rows (4 consecutive rows per row tile), all requested before the
    // first is used: a read per store, waited for on the spot, made the LDS latency the epilogue's pace
    v4f aff4[NMT];
#pragma unroll
    for (int mt = 0; mt < NMT; ++mt) {
      aff4[mt] = *(const v4f*)(s_aff + mt * 16 + 4 * g);
      if (!post) aff4[mt] = (v4f){1.f, 1.f, 1.f, 1.f};
    }
    static_for<0, NMT>([&](auto mt_) {
      constexpr int mt = decltype(mt_)::value;
      float av[4][4];  // [column tile][row]
      static_for<0, 16>([&](auto i_) {
        constexpr int i = decltype(i_)::value;
        if constexpr (mt < 16) av[i / 4][i % 4] = acc_get<16 * mt + i>();
        else av[i / 4][i % 4] = accv[mt - 16][i / 4][i % 4];
      });
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const float af = aff4[mt][r];
        v2i o;
#pragma unroll
        for (int t = 0; t < 4; t += 2) {
          const v2f d = {(av[t][r] + bd[t]) * af, (av[t + 1][r] + bd[t + 1]) * af};
          o[t >> 1] = __builtin_bit_cast(int, __builtin_convertvector(d, v2bf));
        }
        st_b64(o, d_voff, rd, (mt * 16 + r) * rowb);
      }
    });
  }
}

// One translation unit per (stage, weight format): the build compiles this file once for each with
// MX_INST_STAGE / MX_INST_WFMT defined, and once without them for the dispatcher below.
#if defined(MX_INST_STAGE)
template <int STAGE, int WFMT>
__global__ __launch_bounds__(MXT) __attribute__((amdgpu_waves_per_eu(1, 1))) void mx_gemm_kernel(const MxArgs a) {
  extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
  __shared__ int s_tok[MX_ROWS_MAX];
  __shared__ __attribute__((aligned(16))) float s_aff[MX_ROWS_MAX];
  // Workgroups are handed to the 8 XCDs round-robin by linear index, and each XCD has its own L2.
  // XCD x therefore takes the x-th contiguous eighth of the chunk list (chunks are ordered by
  // expert), and walks it chunk by chunk with the column tiles innermost: the workgroups that share
  // an activation tile, and the chunks that share an expert's weights, then run at the same time
  // behind the same L2, so each operand crosses the fabric about once.
  const int n_chunks = __builtin_amdgcn_readfirstlane(*a.n_chunks);
  const int per_xcd = (n_chunks + 7) >> 3;
  const int xcd = blockIdx.x & 7, j = blockIdx.x >> 3;
  const int local = j / a.col_tiles, xt = j - local * a.col_tiles;
  const int chunk = xcd * per_xcd + local;
  if (local >= per_xcd || chunk >= n_chunks) return;
  // values read from memory at a uniform address are uniform; say so, so that everything derived
  // from them (buffer descriptors, scalar offsets) stays in scalar registers
  const int nrows = __builtin_amdgcn_readfirstlane(a.chunk_rows[chunk]);
  const int e = __builtin_amdgcn_readfirstlane(a.chunk_expert[chunk]);
  const int64_t slot0 = __builtin_amdgcn_readfirstlane(a.chunk_slot[chunk]);
  const bool last = (chunk + 1 >= n_chunks) || (__builtin_amdgcn_readfirstlane(a.chunk_expert[chunk + 1]) != e);
  if (last) {
    if (nrows <= 64) mx_gemm_body<STAGE, 4, true, WFMT>(a, smem, s_tok, s_aff, nrows, e, slot0, xt);
    else if (nrows <= 128) mx_gemm_body<STAGE, 8, true, WFMT>(a, smem, s_tok, s_aff, nrows, e, slot0, xt);
    else if (nrows <= 256) mx_gemm_body<STAGE, 16, true, WFMT>(a, smem, s_tok, s_aff, nrows, e, slot0, xt);
    else mx_gemm_body<STAGE, 20, true, WFMT>(a, smem, s_tok, s_aff, nrows, e, slot0, xt);
  } else {
    if (nrows <= 64) mx_gemm_body<STAGE, 4, false, WFMT>(a, smem, s_tok, s_aff, nrows, e, slot0, xt);
    else if (nrows <= 128) mx_gemm_body<STAGE, 8, false, WFMT>(a, smem, s_tok, s_aff, nrows, e, slot0, xt);
    else if (nrows <= 256) mx_gemm_body<STAGE, 16, false, WFMT>(a, smem, s_tok, s_aff, nrows, e, slot0, xt);
    else mx_gemm_body<STAGE, 20, false, WFMT>(a, smem, s_tok, s_aff, nrows, e, slot0, xt);
  }
}

#define MX_CAT_(a, b, c, d) a##b##c##d
#define MX_CAT(a, b, c, d) MX_CAT_(a, b, c, d)
int MX_CAT(launch_mx_gemm_s, MX_INST_STAGE, _f, MX_INST_WFMT)(const MxArgs& m, unsigned grid, hipStream_t s) {
  const hipError_t err = hipFuncSetAttribute((const void*)mx_gemm_kernel<MX_INST_STAGE, MX_INST_WFMT>,
                                             hipFuncAttributeMaxDynamicSharedMemorySize, MX_LDS);
  if (err != hipSuccess) return MOE_E_LAUNCH;
  hipLaunchKernelGGL((mx_gemm_kernel<MX_INST_STAGE, MX_INST_WFMT>), dim3(grid), dim3(MXT), MX_LDS, s, m);
  MOE_CHECK_LAUNCH();
  return MOE_OK;
}

#else  // dispatcher

int launch_mx_gemm_s1_f0(const MxArgs& m, unsigned grid, hipStream_t s);
int launch_mx_gemm_s2_f0(const MxArgs& m, unsigned grid, hipStream_t s);
int launch_mx_gemm_s1_f1(const MxArgs& m, unsigned grid, hipStream_t s);
int launch_mx_gemm_s2_f1(const MxArgs& m, unsigned grid, hipStream_t s);
int launch_mx_gemm_s1_f2(const MxArgs& m, unsigned grid, hipStream_t s);
int launch_mx_gemm_s2_f2(const MxArgs& m, unsigned grid, hipStream_t s);

int launch_mx_gemm(int stage, const MxArgs& m0, unsigned gx, unsigned gy, hipStream_t s) {
  if (gx == 0 || gy == 0) return MOE_OK;
  MxArgs m = m0;
  m.col_tiles = (int32_t)gx;
  const unsigned grid = 8u * ((gy + 7u) / 8u) * gx;  // gy = upper bound on the number of chunks
  switch (m.wfmt) {
    case MX_WFMT_E4M3: return stage == 1 ? launch_mx_gemm_s1_f0(m, grid, s) : launch_mx_gemm_s2_f0(m, grid, s);
    case MX_WFMT_E5M2: return stage == 1 ? launch_mx_gemm_s1_f1(m, grid, s) : launch_mx_gemm_s2_f1(m, grid, s);
    case MX_WFMT_E2M1: return stage == 1 ? launch_mx_gemm_s1_f2(m, grid, s) : launch_mx_gemm_s2_f2(m, grid, s);
    default: return MOE_E_BAD_ARG;
  }
}

#endif

}  // namespace moe
