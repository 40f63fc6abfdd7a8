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
// MX_WFMT_BF16: the 128 K bytes are 64 bf16 values; the first four registers of both fragments (K bytes [16g, 16g+16)
// of the slice = elements 8g .. 8g+7 of its first 32) and the last four (the same of its second 32) are the operands
// of two 32-deep bf16 MFMAs, which take the time of the one 128-deep 8-bit MFMA.  No scales.
__device__ __forceinline__ v4i lo4(const v8i& x) { return (v4i){x[0], x[1], x[2], x[3]}; }
__device__ __forceinline__ v4i hi4(const v8i& x) { return (v4i){x[4], x[5], x[6], x[7]}; }
__device__ __forceinline__ v4i lo4(const v4i& x) { return x; }  // (4-bit operands: never instantiated for bf16)
__device__ __forceinline__ v4i hi4(const v4i& x) { return x; }
template <int ACC, int OA, int OB, int WFMT, class BOp>
__device__ __forceinline__ void mfma_asm(const v8i& af, const BOp& bf, int sa, int sb) {
  if constexpr (WFMT == MX_WFMT_BF16) {
    asm volatile("v_mfma_f32_16x16x32_bf16 a[%0:%1], %2, %3, a[%0:%1]\n\tv_mfma_f32_16x16x32_bf16 a[%0:%1], %4, %5, a[%0:%1]"
                 : : "n"(ACC), "n"(ACC + 3), "v"(lo4(af)), "v"(lo4(bf)), "v"(hi4(af)), "v"(hi4(bf)));
  } else {
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
  if constexpr (WFMT == MX_WFMT_BF16) {
    asm volatile("v_mfma_f32_16x16x32_bf16 %0, %1, %2, %0\n\tv_mfma_f32_16x16x32_bf16 %0, %3, %4, %0"
                 : "+v"(c) : "v"(lo4(af)), "v"(lo4(bf)), "v"(hi4(af)), "v"(hi4(bf)));
  } else {
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
}
#undef MX_MFMA_CASE
#undef MX_MFMA_ASM

// A vector memory instruction that reads a scalar register (descriptor, scalar offset) needs five wait states
// after a vector ALU instruction that wrote that register (v_readfirstlane, v_readlane: the compiler reloads
// spilled scalars with the latter right where they are used).  The compiler keeps that distance for instructions
// of its own; for the instructions written out in this file it cannot (it does not see which operands an inline
// statement reads when), so each of them carries the wait states itself.  They are issue slots in the shadow of
// the MFMAs between which the loads sit.
#define MX_SGPR_WAIT "s_nop 4\n\t"

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
    asm volatile(MX_SGPR_WAIT "buffer_load_dwordx4 %0, %1, %2, %3 offen nt" : "+v"(d) : "v"(voff), "s"(rsrc), "s"(soff) : "memory");
  else
    asm volatile(MX_SGPR_WAIT "buffer_load_dwordx4 %0, %1, %2, %3 offen" : "+v"(d) : "v"(voff), "s"(rsrc), "s"(soff) : "memory");
}
__device__ __forceinline__ void st_b64(const v2i& d, uint32_t voff, const v4i& rsrc, int soff) {
  asm volatile(MX_SGPR_WAIT "buffer_store_dwordx2 %0, %1, %2, %3 offen nt" : : "v"(d), "v"(voff), "s"(rsrc), "s"(soff) : "memory");
}
__device__ __forceinline__ void st_b128(const v4i& d, uint32_t voff, const v4i& rsrc, int soff) {
  asm volatile(MX_SGPR_WAIT "buffer_store_dwordx4 %0, %1, %2, %3 offen nt" : : "v"(d), "v"(voff), "s"(rsrc), "s"(soff) : "memory");
}
// 16 bytes per lane straight into LDS at lds + 16 * lane (no destination registers).  The instruction takes its
// LDS base from M0, which is set in the same statement.  M0 is declared clobbered: the compiler warns that it
// does not save reserved registers around a statement, which is what is wanted here -- on this target it never
// carries a value in M0 from one instruction to the next (it writes M0 itself immediately before each instruction
// of its own that reads it), so there is nothing to save.
__device__ __forceinline__ void ld_lds_b128(uint32_t lds, uint32_t voff, const v4i& rsrc, int soff) {
  asm volatile(MX_SGPR_WAIT "s_mov_b32 m0, %0\n\tbuffer_load_dwordx4 %1, %2, %3 offen lds"
               : : "s"(lds), "v"(voff), "s"(rsrc), "s"(soff) : "memory", "m0");
}
template <bool NT>
__device__ __forceinline__ void ld_b64(v2i& d, uint32_t voff, const v4i& rsrc, int soff) {
  if constexpr (NT)
    asm volatile(MX_SGPR_WAIT "buffer_load_dwordx2 %0, %1, %2, %3 offen nt" : "+v"(d) : "v"(voff), "s"(rsrc), "s"(soff) : "memory");
  else
    asm volatile(MX_SGPR_WAIT "buffer_load_dwordx2 %0, %1, %2, %3 offen" : "+v"(d) : "v"(voff), "s"(rsrc), "s"(soff) : "memory");
}
typedef int v3i __attribute__((ext_vector_type(3)));
__device__ __forceinline__ void ld_dwords(v3i& d, uint32_t voff, const v4i& rsrc, int soff) {
  asm volatile(MX_SGPR_WAIT "buffer_load_dwordx3 %0, %1, %2, %3 offen" : "+v"(d) : "v"(voff), "s"(rsrc), "s"(soff) : "memory");
}
__device__ __forceinline__ void ld_dwords(v2i& d, uint32_t voff, const v4i& rsrc, int soff) {
  asm volatile(MX_SGPR_WAIT "buffer_load_dwordx2 %0, %1, %2, %3 offen" : "+v"(d) : "v"(voff), "s"(rsrc), "s"(soff) : "memory");
}
__device__ __forceinline__ void ld_b32(int& d, uint32_t voff, const v4i& rsrc, int soff) {
  asm volatile(MX_SGPR_WAIT "buffer_load_dword %0, %1, %2, %3 offen" : "+v"(d) : "v"(voff), "s"(rsrc), "s"(soff) : "memory");
}

// A workgroup barrier that orders LDS traffic only.  (__syncthreads also makes the workgroup's global stores
// visible, for which the compiler waits until every vector memory operation has completed -- the loads in flight
// for the next tile included.)
__device__ __forceinline__ void lds_barrier() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }

// NMT = number of 16-row tiles this instantiation multiplies (the chunks it takes have at most NMT*16 rows).
// Keeping it a compile-time constant keeps the K loop free of branches around the MFMAs.
// LASTUSE: the chunks are the last ones of their experts, so their weights are streamed past the L2 (which
// then keeps the activation tiles that the sibling workgroups share); an earlier chunk loads them
// normally, for the chunk after it to find.
//
// A workgroup stays on its CU and walks a list of tiles of one class (items L, L + Lstep, ... below endL of its
// XCD's queue; an item is a chunk and one of its column tiles).  Between two tiles nothing is left to the
// hardware's workgroup dispatch: as soon as the K loop of a tile has ended, the loads of the first D slices of the
// next tile are issued, and only then does the tile's epilogue run -- the memory pipeline works through those
// loads while the epilogue computes, and the next K loop starts on data that has arrived.  What the next tile
// needs before its loads can be issued (token ids, affinities, bias) is read one tile earlier the same way:
// requested before an epilogue, put in place after it.
template <int STAGE, int NMT, bool LASTUSE, int WFMT>
__device__ __forceinline__ int mx_gemm_tiles(const MxArgs& a, uint8_t* smem, int (*s_tok)[MX_ROWS_MAX],
                                             float (*s_aff)[MX_ROWS_MAX], float (*s_bias)[MXT],
                                             float (*s_rs)[MX_ROWS_MAX], float (*s_wsc)[MXT], int L, const int startL,
                                             const int endL, const int Lstep, const int qbase, const int interleave) {
  using Cfg = MxCfg<NMT>;
  // ROW8: the fp8-row kind.  Same K loop on e4m3 operands with block scales of 2^0; what differs is the epilogue
  // (per-channel weight scale x per-row activation scale ahead of the bias, bias and scales indexed by natural
  // column, gate/up results written as fp32 rows for the per-row re-quantisation pass) and two more row / column
  // tables (s_rs, s_wsc: null for the MX formats).
  // BF16: the bf16 kind.  The same again, on bf16 operands (see mfma_asm) with no scales at all: row "scales" are 1
  // (0 for a slot without a token), column scales 1 unless per-channel scales of widened fp8 weights are given, and
  // the gate/up results go out as bf16 rows in natural column order, which the down stage reads as they are.
  constexpr bool BF16 = WFMT == MX_WFMT_BF16;
  constexpr bool ROW8 = WFMT == MX_WFMT_ROW8 || BF16;
  constexpr int MFMT = BF16 ? MX_WFMT_BF16 : ROW8 ? MX_WFMT_E4M3 : WFMT;  // element format of the MFMA's B operand
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
  const int q = w;

  // ---- tiles ------------------------------------------------------------------------------------
  // Everything that says which tile: uniform values, kept in scalar registers.  A tile's queue entry (two words)
  // is read through the scalar cache where it is needed, with an instruction of this file's own: a plain load is a
  // vector load to the compiler (it cannot know that no store aliases the queue), and a vector load in the wrong
  // place waits for every load in flight.
  struct Tile {
    int nrows, e, slot0, xt;
  };
  typedef int v2i_t __attribute__((ext_vector_type(2)));
  // Item l of the class -> (chunk position, column tile).  G = `interleave` chunks at a time (chosen with the queues): within a
  // group of G queue positions the chunk varies fastest, so that workgroups with neighbouring items work on the
  // same column tile of different chunks (of one expert: they share the weight tile); G = 1 is column tiles
  // innermost.  The last group of a class may hold fewer than G chunks.
  // (items are numbered through the XCD's whole queue; the class's own run from startL to endL)
  const int pos0 = startL / a.col_tiles, npos = (endL - startL) / a.col_tiles;
  auto tile_at = [&](int l) {
    int pos, xt;
    if (interleave == 1) {
      pos = l / a.col_tiles;
      xt = l - pos * a.col_tiles;
    } else {
      const int per_group = interleave * a.col_tiles;
      const int lr = l - startL;
      const int grp = lr / per_group, j = lr - grp * per_group;
      const int base = grp * interleave;
      const int G = (npos - base < interleave) ? npos - base : interleave;
      xt = j / G;
      pos = pos0 + base + (j - xt * G);
    }
    v2i_t raw;
    asm volatile(MX_SGPR_WAIT "s_load_dwordx2 %0, %1, %2\n\ts_waitcnt lgkmcnt(0)"
                 : "=s"(raw) : "s"(a.q_chunk), "s"((qbase + pos) * 8) : "memory");
    Tile t;
    t.xt = xt;
    t.slot0 = raw[0];
    t.nrows = raw[1] & 0xffff;
    t.e = raw[1] >> 16;
    return t;
  };
  // gate/up: column tiles are numbered over the existing ones, 4 per full intermediate tile, then those of a
  // short last tile (whose partitions per q are a multiple of 32 on this path): intermediate tile, first
  // partition, partitions per q.  down: first hidden column.
  auto tile_tI = [&](const Tile& t) { return t.xt >> 2; };
  auto tile_p0 = [&](const Tile& t) { return (t.xt & 3) * 32; };
  auto tile_Pt = [&](const Tile& t) {
    const int64_t rows_t = (a.I - (int64_t)(t.xt >> 2) * 512 < 512) ? (a.I - (int64_t)(t.xt >> 2) * 512) : 512;
    return (int)(rows_t / 4);
  };
  auto tile_h0 = [&](const Tile& t) { return (int64_t)t.xt * 256; };
  // Rows: a thread looks after rows tid and 256 + tid of the chunk (token id, affinity), and after one of the
  // tile's 256 bias values.  Each of these is fetched in two steps: `*_raw` issues loads (always from a valid
  // address, no branch), `*_put` turns what arrived into the value and stores it in LDS.  Between the two lies an
  // epilogue with a tile's first loads in flight.  The loads are instructions of this file's own, like those of
  // the K loop: the compiler waits for a load of its own wherever it first touches the result or reuses the
  // register, and such a wait would hold the epilogue until everything issued before it has arrived.
  constexpr bool ROWS2 = NMT * 16 > 256;
  auto ids_raw = [&](const Tile& t, int (&raw)[2]) {
    const v4i rd = make_rsrc(a.tp2id, 0xffffffffu);
#pragma unroll
    for (int j = 0; j < (ROWS2 ? 2 : 1); ++j) {
      const int r = tid + 256 * j;
      ld_b32(raw[j], (uint32_t)(t.slot0 + ((r < t.nrows) ? r : t.nrows - 1)) * 4u, rd, 0);
    }
  };
  auto ids_put = [&](int buf, int nrows, const int (&raw)[2]) {
#pragma unroll
    for (int j = 0; j < (ROWS2 ? 2 : 1); ++j) {
      const int r = tid + 256 * j;
      if (r < Cfg::ROWS) s_tok[buf][r] = (r < nrows && raw[j] >= 0 && raw[j] < a.n_real) ? raw[j] : -1;
    }
  };
  // (No branch may surround such a load: where two paths that load into the same variable meet, the compiler
  // copies the register right behind the load instruction, i.e. before the data has arrived.  So there is one
  // load instruction for both element types -- the aligned word that holds the element, the half picked later --
  // and a table that is absent is replaced by an address that is valid.)
  auto elem_offset = [&](uint32_t idx, bool two_byte) { return two_byte ? ((idx << 1) & ~3u) : (idx << 2); };
  auto elem_value = [&](int word, uint32_t idx, bool two_byte) {
    return two_byte ? bf16_bits_to_f32((uint16_t)((uint32_t)word >> ((idx & 1u) * 16u))) : __builtin_bit_cast(float, word);
  };
  auto aff_index = [&](int e, int buf, int r) {
    const int id = s_tok[buf][(r < NMT * 16) ? r : 0];
    return (uint32_t)((id >= 0) ? id : 0) * (uint32_t)a.E + (uint32_t)e;
  };
  auto aff_raw = [&](const Tile& t, int buf, int (&raw)[2]) {
    const v4i rd = make_rsrc(a.aff ? a.aff : (const void*)a.tp2id, 0xffffffffu);
#pragma unroll
    for (int j = 0; j < (ROWS2 ? 2 : 1); ++j) {
      const uint32_t off = a.aff ? elem_offset(aff_index(t.e, buf, tid + 256 * j), a.aff_dtype == MOE_DT_BF16) : 0u;
      ld_b32(raw[j], off, rd, 0);
    }
  };
  auto aff_put = [&](int e, int buf, const int (&raw)[2]) {
#pragma unroll
    for (int j = 0; j < (ROWS2 ? 2 : 1); ++j) {
      const int r = tid + 256 * j;
      if (r < NMT * 16) {
        float v = 0.f;
        if (a.aff && s_tok[buf][r] >= 0) v = elem_value(raw[j], aff_index(e, buf, r), a.aff_dtype == MOE_DT_BF16);
        s_aff[buf][r] = v;
      }
    }
  };
  // gate/up: bias value (gu*4 + q)*32 + pl belongs to partition p0 + pl; down: value j to column h0 + j.
  const int hcol = (STAGE == 1) ? (c >> 3) : 0, cl = (STAGE == 1) ? (c & 7) : c;
  // the natural column of the thread's table entry: gate/up (gu = tid/128, q = tid/32 % 4, pl = tid % 32) ->
  // gu * I + tile*512 + q*Pt + p0 + pl; down -> h0 + tid
  auto natural_col = [&](const Tile& t) {
    if (STAGE == 1)
      return (uint32_t)(tid >> 7) * (uint32_t)a.I + (uint32_t)tile_tI(t) * 512u +
             (uint32_t)((tid >> 5) & 3) * (uint32_t)tile_Pt(t) + (uint32_t)(tile_p0(t) + (tid & 31));
    return (uint32_t)tile_h0(t) + (uint32_t)tid;
  };
  const uint32_t ncols = (STAGE == 1) ? 2u * (uint32_t)a.I : (uint32_t)a.H;  // table entries per expert
  auto bias_index = [&](const Tile& t) {
    if (ROW8) return (uint32_t)t.e * ncols + natural_col(t);
    if (STAGE == 1) {
      const uint32_t p = (uint32_t)(tile_p0(t) + (tid & 31));
      return ((((uint32_t)t.e * (uint32_t)a.pI + p) * 2u + (uint32_t)(tid >> 7)) * (uint32_t)a.nI + (uint32_t)tile_tI(t)) * 4u +
             (uint32_t)((tid >> 5) & 3);
    }
    return (uint32_t)t.e * (uint32_t)a.H + (uint32_t)tile_h0(t) + (uint32_t)tid;
  };
  auto bias_raw = [&](const Tile& t, int& raw) {
    const v4i rd = make_rsrc(a.bias ? a.bias : (const void*)a.tp2id, 0xffffffffu);
    ld_b32(raw, a.bias ? elem_offset(bias_index(t), a.bias_dtype == MOE_DT_BF16) : 0u, rd, 0);
  };
  auto bias_put = [&](const Tile& t, int buf, int raw) {
    s_bias[buf][tid] = a.bias ? elem_value(raw, bias_index(t), a.bias_dtype == MOE_DT_BF16) : 0.f;
  };
  // ROW8: the weights' per-channel scale of the thread's column (fp32), and the activation rows' scales: gate/up,
  // the fp32 behind the H codes of the token's record, times the affinity under PRE_SCALE (the affinity scales
  // the token's row, i.e. its dequantisation scale); down, the scale of the re-quantised intermediate row.
  auto wsc_raw = [&](const Tile& t, int& raw) {
    if constexpr (ROW8) {
      const v4i rd = make_rsrc(a.w_cscale ? (const void*)a.w_cscale : (const void*)a.tp2id, 0xffffffffu);
      ld_b32(raw, a.w_cscale ? ((a.cscale_experts > 1 ? (uint32_t)t.e * ncols : 0u) + natural_col(t)) << 2 : 0u, rd, 0);
    }
  };
  auto wsc_put = [&](int buf, int raw) {
    if constexpr (ROW8) s_wsc[buf][tid] = a.w_cscale ? __builtin_bit_cast(float, raw) : 1.f;
  };
  auto rs_raw = [&](const Tile& t, int buf, int (&raw)[2]) {
    if constexpr (ROW8) {
      // (bf16: nothing to fetch; the load stays, from an address that is valid, so that every format issues the
      // same loads)
      const v4i rd = make_rsrc((STAGE == 1 || BF16) ? (const void*)a.A : (const void*)a.a_rscale, 0xffffffffu);
#pragma unroll
      for (int j = 0; j < (ROWS2 ? 2 : 1); ++j) {
        const int r = tid + 256 * j;
        uint32_t off;
        if (STAGE == 1) {
          const int id = s_tok[buf][(r < NMT * 16) ? r : 0];
          off = (uint32_t)((id >= 0) ? id : 0) * (uint32_t)a.a_stride + (BF16 ? 0u : (uint32_t)a.H);
        } else {
          off = (uint32_t)(t.slot0 + ((r < t.nrows) ? r : t.nrows - 1)) << 2;
        }
        ld_b32(raw[j], off, rd, 0);
      }
    }
  };
  // (gate/up under PRE_SCALE: `aff` holds what aff_raw fetched for the same rows)
  auto rs_put = [&](int e, int buf, const int (&raw)[2], const int (&aff)[2]) {
    if constexpr (ROW8) {
      const bool pre = STAGE == 1 && (a.scaling_mode == MOE_SCALE_PRE || a.scaling_mode == MOE_SCALE_PRE_DELAYED);
#pragma unroll
      for (int j = 0; j < (ROWS2 ? 2 : 1); ++j) {
        const int r = tid + 256 * j;
        if (r < NMT * 16) {
          float v = BF16 ? 1.f : __builtin_bit_cast(float, raw[j]);
          if (STAGE == 1 && s_tok[buf][r] < 0) v = 0.f;
          if (pre && a.aff && s_tok[buf][r] >= 0) v *= elem_value(aff[j], aff_index(e, buf, r), a.aff_dtype == MOE_DT_BF16);
          s_rs[buf][r] = v;
        }
      }
    }
  };
  // which stages fetch the affinities: down always; gate/up of the fp8-row kind, for PRE_SCALE
  constexpr bool AFF_ROWS = STAGE == 2 || ROW8;
  // what has been requested with the *_raw functions above may be used once this has passed
  auto all_loads_landed = [&](int (&x)[2], int (&y)[2], int& z, int (&u)[2], int& v) {
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    asm volatile("" : "+v"(x[0]), "+v"(x[1]), "+v"(y[0]), "+v"(y[1]), "+v"(z));
    if constexpr (ROW8) asm volatile("" : "+v"(u[0]), "+v"(u[1]), "+v"(v));
  };

  // A staging: thread covers rows (tid>>3) + 32 j; its load goes straight to LDS slot tid&7 of that
  // row and fetches the 16-byte chunk (tid&7) ^ (row&7) that belongs there
  const int arow0 = tid >> 3, ach = tid & 7;
  constexpr int NAJ = NMT / 2;  // 32-row groups that hold rows of the NMT tiles
  // Per-lane 32-bit byte offsets (row * stride + chunk); the K offset is wave-uniform and is added
  // to the scalar base, so a load needs one VGPR of address.  Rows without a token (padding
  // slots, rows past the end of the chunk) point past the end of the buffer and load as zero rows,
  // without a branch (see aim_loads_at).
  // (down stage: the rows are consecutive slots, so one per-lane offset serves all row groups and the group goes
  // into the scalar offset; rows past the chunk's end may then lie past the end of the buffer, where the range
  // check of the descriptor returns zeros)
  constexpr int NAV = (STAGE == 1) ? NAJ : 1;
  uint32_t a_voff[NAV];
  // A scales: thread covers row tid (and, in a chunk of more than 256 rows, row 256 + tid % 64: every
  // wave issues that load so that all waves count the same loads, the first wave's is used)
  uint32_t as_voff = 0, as_voff2 = 0;
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
  // A lane loads 16 bytes = 4 adjacent columns of one K row: column 4*cl + t belongs to column tile
  // t.  In the gate/up stage the wave's 32 gate columns take lanes c = 0..7 of each group and its 32
  // up columns lanes c = 8..15, so every column tile is half gate, half up, and one load instruction
  // fetches 128 contiguous bytes of gate and of up for 4 K rows.  (8-byte loads, one tile pair per
  // load, cost the memory pipeline as much per instruction as 16-byte ones.)
  // 4-bit weights (x4: four K values in a 2-byte element): lane group g needs K 32g .. 32g+31 of the
  // slice = partitions 8g .. 8g+7, one 8-byte load (4 columns) per partition; 8-bit weights (4-byte
  // elements): partitions 4g .. 4g+3 and 16+4g .. 16+4g+3, one 16-byte load each.
  constexpr bool FP4 = WFMT == MX_WFMT_E2M1;
  constexpr int ES = FP4 ? 2 : 4;      // bytes of a weight element
  constexpr int GROWS = FP4 ? 8 : 4;   // partition rows between the lane groups' first rows
  const uint8_t* Wb = (const uint8_t*)a.W;
  // element strides (4-byte weights; scales use the same counts in bytes)
  const int64_t w_pstride = (STAGE == 1) ? 2 * nH * a.I : (int64_t)a.nI * a.H;
  const int64_t w_tstride = (STAGE == 1) ? a.I : a.H;
  // a.w_packed: the weights are a copy in the order these loads read them (see mx_pack_weights_kernel): load i of
  // wave q in slice ks of column tile xt is 1 KB (4-bit weights: 512 bytes) at ((xt * nks + ks) * 4 + q) * 8 + i
  // such units into the expert's copy, a lane's 16 (8) bytes in lane order: each workgroup reads its weights as one
  // contiguous 32 (16) KB run per slice.
  // (the two address forms are blended with the 0 / 1 flag as a factor: a conditional expression here may become
  // a branch, and values that cross a branch in this function are no longer known to the compiler as uniform)
  const int pk = a.w_packed ? 1 : 0, npk = 1 - pk;
  constexpr int PK_LANE = FP4 ? 8 : 16;        // bytes a lane loads
  constexpr int PK_LOAD = 64 * PK_LANE;         // ... a load instruction
  constexpr int PK_WAVE = 8 * PK_LOAD;          // ... a wave per K slice
  constexpr int PK_SLICE = 4 * PK_WAVE;         // ... the workgroup per K slice
  const uint32_t w_voff = (uint32_t)pk * (uint32_t)(lane * PK_LANE) +
                          (uint32_t)npk * ((STAGE == 1) ? (uint32_t)((GROWS * g * w_pstride + hcol * nH * a.I + 4 * cl) * ES)
                                                        : (uint32_t)((GROWS * g * w_pstride + 4 * c) * ES));
  const uint32_t s_voff = (STAGE == 1) ? (uint32_t)(g * w_pstride + hcol * nH * a.I + 4 * cl)
                                       : (uint32_t)(g * w_pstride + 4 * c);
  // bytes of one expert's weights: the reference layout's, or col_tiles x nks runs of 32 KB
  const int64_t w_expert_bytes = pk * ((int64_t)a.col_tiles * nks * PK_SLICE) +
                                 npk * ((STAGE == 1) ? 128 * w_pstride * ES : (int64_t)a.pI * w_pstride * ES);
  v4i rw_, rs_;  // the expert's weights and scales

  // A K slice's loads, numbered in issue order:
  //   0 .. NAJ-1            activation rows (16 bytes per lane each, straight into the LDS ring)
  //   NAJ .. NAJ+NSC-1      activation scales of D slices (4 D bytes per lane, into registers), only in the
  //                         first slice of every D
  //   then NBL              weights (16 bytes per lane each, into a raw register set)
  //   then 1                weight scales
  // (SCALED: the MX formats.  The fp8-row and bf16 kinds have block scales of 2^0 throughout: their K loop loads
  // no scales at all and hands the MFMAs the constant)
  constexpr bool SCALED = !ROW8;
  constexpr int UNIT_SCALES = 0x7f7f7f7f;
  constexpr int NBL = 8;
  constexpr int NSC = SCALED ? (BIG ? 2 : 1) : 0;
  constexpr int NLB = NBL + (SCALED ? 1 : 0);  // weight loads of a slice
  constexpr int N1 = NAJ + NLB;             // loads of a slice that carries no activation scales
  constexpr int N0 = N1 + NSC;              // loads of one that does
  typedef typename std::conditional<D == 3, v3i, v2i>::type ScaleRegs;
  typedef typename std::conditional<FP4, v2i, v4i>::type RawLoad;
  typedef typename std::conditional<FP4, v4i, v8i>::type BOperand;
  struct BRaw {
    RawLoad d[NBL];
    int sc;
  };
  v4i ra_ = make_rsrc(a.A, (uint32_t)(a.a_rows * a.a_stride)),
      ras_ = make_rsrc(a.A_scale, (uint32_t)(a.a_scale_bytes ? a.a_scale_bytes : a.a_rows * a.a_scale_stride));
  const int ra_rec = ra_[2], ras_rec = ras_[2];
  int rw_rec = 0, rs_rec = 0;
  const int a_group_bytes = uni((int)(32 * a.a_stride));  // down stage: bytes between row groups of 32 slots
  // Scalar byte offset of a weight load = (offset of its row and column within the slice, fixed per
  // load and kept in scalar registers) + (offset of the slice, computed once per slice): one scalar
  // add per load.  Address arithmetic done per load costs more issue cycles than the MFMAs between
  // two loads take.
  int w_soff[NBL];
  int s_soff = 0;
  // Point the loads at a tile: rows (token ids of the tile sit in s_tok[buf]), expert, columns.
  auto aim_loads_at = [&](const Tile& t, int buf) {
#pragma unroll
    for (int j = 0; j < NAV; ++j) {
      const int row = arow0 + 32 * j;
      uint32_t r;
      if (STAGE == 1) {
        // a row without a token (padding slot, row past the end of the chunk) points past the end of the buffer:
        // the range check of the descriptor turns such a load into zeros without any traffic, so the row is a zero
        // row (what the activation checkpoints must show for it) and its MFMAs multiply zeros
        const int tok = s_tok[buf][row];
        r = (tok >= 0) ? (uint32_t)tok : (uint32_t)a.a_rows;
      } else {
        r = (uint32_t)(t.slot0 + row);
      }
      a_voff[j] = r * (uint32_t)a.a_stride + (uint32_t)((ach ^ (arow0 & 7)) * 16);
    }
    auto scale_row_off = [&](int row) {
      if (STAGE == 1) {
        const int tok = s_tok[buf][row];
        return ((tok >= 0) ? (uint32_t)tok : 0u) * (uint32_t)a.a_scale_stride;
      }
      return (uint32_t)(t.slot0 + ((row < t.nrows) ? row : (t.nrows - 1))) * (uint32_t)a.a_scale_stride;
    };
    as_voff = scale_row_off(tid);
    as_voff2 = BIG ? scale_row_off(256 + (tid & 63)) : 0u;
    int64_t colu;
    if (STAGE == 1) {
      colu = (int64_t)tile_tI(t) * 512 + (int64_t)q * tile_Pt(t) + tile_p0(t);
      rw_ = make_rsrc(Wb + (int64_t)t.e * w_expert_bytes, (uint32_t)w_expert_bytes);
      rs_ = make_rsrc(a.W_scale + (int64_t)(a.w_scale_shared ? 0 : t.e) * 16 * w_pstride, (uint32_t)(16 * w_pstride));
    } else {
      colu = tile_h0(t) + 64 * q;
      const int64_t sp = (a.pI + 7) / 8;
      rw_ = make_rsrc(Wb + (int64_t)t.e * w_expert_bytes, (uint32_t)w_expert_bytes);
      rs_ = make_rsrc(a.W_scale + (int64_t)(a.w_scale_shared ? 0 : t.e) * sp * w_pstride, (uint32_t)(sp * w_pstride));
    }
    rw_rec = rw_[2];
    rs_rec = rs_[2];
#pragma unroll
    for (int i = 0; i < NBL; ++i) {
      const int pr = FP4 ? i : ((i < 4) ? i : (16 + i - 4));
      w_soff[i] = uni(pk * (((t.xt * nks) * 4 + q) * PK_WAVE + i * PK_LOAD) + npk * (int)(((int64_t)pr * w_pstride + colu) * ES));
    }
    s_soff = uni(colu);
  };
  // Everything a slice's loads share: descriptors (of zero records past the end: such a load is out
  // of range, fetches nothing and returns zeros, so the K loop needs no conditions around its loads)
  // and the slice's scalar offsets.
  // The four descriptors are kept once; what changes from slice to slice is their record count (word 2), which is
  // set in place for the slice whose loads are about to be issued.
  int tile_live = -1;  // 0: the loads being issued belong to no tile (behind the last tile of the list)
  struct SliceAddr {
    int a_off, as_off, w_off, s_off;
    uint32_t lds_a;  // LDS address of the ring stage that receives this slice's activations
  };
  const uint32_t lds_ring = (uint32_t)(uintptr_t)sA;
  auto slice_addr = [&](int ks, int st) {
    SliceAddr r;
    r.lds_a = uni((int)(lds_ring + (uint32_t)st * SA));
    const int live = (ks < nks) ? tile_live : 0;
    ra_[2] = uni(ra_rec & live);
    ras_[2] = uni(ras_rec & live);
    rw_[2] = uni(rw_rec & live);
    rs_[2] = uni(rs_rec & live);
    const int kt = ks >> 2, pb = ks & 3;
    r.a_off = ks * 128;
    r.as_off = ks * 4;
    r.w_off = uni(pk * (ks * PK_SLICE) + npk * (int)(((int64_t)(pb * 32) * w_pstride + (int64_t)kt * w_tstride) * ES));
    r.s_off = uni((int64_t)(pb * 4) * w_pstride + (int64_t)kt * w_tstride);
    return r;
  };
  auto issue_load = [&](auto idx_, const SliceAddr& sa, BRaw& b, ScaleRegs& sc0, ScaleRegs& sc1, auto with_scales_) {
    constexpr int idx = decltype(idx_)::value;
    if constexpr (idx < NAJ) {
      // the wave's 64 lanes fill 8 rows x 128 bytes = 1 KB of the ring stage, in lane order
      if constexpr (STAGE == 1)
        ld_lds_b128(sa.lds_a + (uint32_t)((w * 8 + 32 * idx) * MXROW), a_voff[idx], ra_, sa.a_off);
      else
        ld_lds_b128(sa.lds_a + (uint32_t)((w * 8 + 32 * idx) * MXROW), a_voff[0], ra_, sa.a_off + idx * a_group_bytes);
    } else if constexpr (idx < NAJ + NSC) {
      // the four scale bytes (K blocks) of a row, for this slice and the D-1 after it: a lane's
      // dwords sit in different cache lines, so this load costs the memory pipeline as many
      // requests as all the activation rows of a slice together -- hence one in D slices
      if constexpr (decltype(with_scales_)::value) {
        if constexpr (idx == NAJ) ld_dwords(sc0, as_voff, ras_, sa.as_off);
        else ld_dwords(sc1, as_voff2, ras_, sa.as_off);
      }
    } else if constexpr (idx < NAJ + NSC + NBL) {
      constexpr int i = idx - NAJ - NSC;
      if constexpr (FP4) ld_b64<LASTUSE>(b.d[i], w_voff, rw_, w_soff[i] + sa.w_off);
      else ld_b128<LASTUSE>(b.d[i], w_voff, rw_, w_soff[i] + sa.w_off);
    } else {
      static_assert(SCALED || idx < NAJ + NSC + NBL, "no scale load without scales");
      if constexpr (SCALED) ld_b32(b.sc, s_voff, rs_, s_soff + sa.s_off);
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

  v4f accv[4][4];  // row tiles 16..19

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
    v4i asc = (v4i){UNIT_SCALES, UNIT_SCALES, UNIT_SCALES, UNIT_SCALES};
    int asc_hi = UNIT_SCALES;
    if constexpr (SCALED) {
      asc = *(const v4i*)(sS + st * SS + (g * 16 + c) * SSP);
      if constexpr (BIG) asc_hi = *(const int*)(sS + st * SS + (g * 16 + c) * SSP + 16);
    }
    // first fragments of this slice: in flight while the weights are transposed
    v8i af[2][2];
    af[0][0] = frag_from_lds(plo, phi);
    af[0][1] = frag_from_lds(plo + 16 * MXROW, phi + 16 * MXROW);
    asm volatile("" ::: "memory");
    asm volatile("s_waitcnt vmcnt(%0)" : : "n"(NLB + (D - 2) * N1) : "memory");
    if constexpr (SCALED && U == D - 1) {  // activation scales of slices ks+1 .. ks+D
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
    b.sc = SCALED ? braw.sc : UNIT_SCALES;
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
          mfma_asm<16 * mt + 4 * nt, mt % 4, nt, MFMT>(af[cur][j / 4], b.f[nt], asc[mt / 4], b.sc);
        else
          mfma_asm_v<mt % 4, nt, MFMT>(accv[mt - 16][nt], af[cur][j / 4], b.f[nt], asc_hi, b.sc);
        if constexpr (m == 0) {
          // the scalar arithmetic for the addresses of slice ks+D starts here, behind the first
          // MFMA, instead of ahead of it
          int ksd = ks + D;
          asm volatile("" : "+s"(ksd));
          sad = slice_addr(ksd, wrapst(st + D));
        }
        if constexpr (SCALED && U == D - 1 && m >= 3 && m < 3 + D) {
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

  // The first D slices of a tile are requested at once (for the first tile before anything else, for every later
  // one ahead of the epilogue of the tile before it).
  // (numbered 0 .. D * N0 - 1 in issue order, slice after slice, so that a part of them can be asked for at a time)
  constexpr int NFIRST = D * N0;
  SliceAddr sa_first;  // of the slice whose loads are being issued
  auto request_first = [&](auto n0_, auto n1_) {
    static_for<decltype(n0_)::value, (decltype(n1_)::value < NFIRST ? decltype(n1_)::value : NFIRST)>([&](auto n_) {
      constexpr int n = decltype(n_)::value;
      constexpr int u = n / N0, i = n % N0;
      if constexpr (i == 0) sa_first = slice_addr(u, u);
      issue_load(std::integral_constant<int, i>{}, sa_first, br[u], asr, asr2, std::integral_constant<bool, u == 0>{});
    });
  };
  auto request_first_slices = [&]() { request_first(std::integral_constant<int, 0>{}, std::integral_constant<int, NFIRST>{}); };

  // ---- first tile: nothing is in flight yet, so plain loads and waits do ----------------------------------
  Tile cur = tile_at(L);
  int ids_nn[2] = {0, 0}, aff_n[2] = {0, 0}, bias_n = 0;  // requested ahead of an epilogue, put in place after it
  int rs_n[2] = {0, 0}, wsc_n = 0;                          // (fp8-row kind only)
  ids_raw(cur, ids_nn);
  bias_raw(cur, bias_n);
  wsc_raw(cur, wsc_n);
  all_loads_landed(ids_nn, aff_n, bias_n, rs_n, wsc_n);
  ids_put(0, cur.nrows, ids_nn);
  bias_put(cur, 0, bias_n);
  wsc_put(0, wsc_n);
  __syncthreads();
  if (AFF_ROWS) {
    aff_raw(cur, 0, aff_n);
    rs_raw(cur, 0, rs_n);
    all_loads_landed(ids_nn, aff_n, bias_n, rs_n, wsc_n);
    if (STAGE == 2) aff_put(cur.e, 0, aff_n);
    rs_put(cur.e, 0, rs_n, aff_n);
  }
  aim_loads_at(cur, 0);
  request_first_slices();
  int Ln = L + Lstep;  // the item after the current one
  bool have_next = Ln < endL;
  {
    // (the wait in here also waits for the first slices: once per workgroup and class)
    const Tile nx = tile_at(have_next ? Ln : L);
    ids_raw(nx, ids_nn);
    all_loads_landed(ids_nn, aff_n, bias_n, rs_n, wsc_n);
    if (have_next) ids_put(1, nx.nrows, ids_nn);  // published by the barrier below
  }
  int buf = 0;  // which of the two row tables (s_tok, s_aff, s_bias) belongs to the current tile

  for (;;) {
  acc_fence();
  static_for<0, (BIG ? 16 : NMT) * 16>([&](auto i_) { acc_zero<decltype(i_)::value>(); });
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) accv[i][j] = (v4f){0.f, 0.f, 0.f, 0.f};
  // (the activation rows of slice 0, and the activation scales of the first D slices, are in)
  asm volatile("s_waitcnt vmcnt(%0)" : : "n"(NLB + (D - 1) * N1) : "memory");
  if constexpr (SCALED) {
    asm volatile("" : "+v"(asr));
    if constexpr (BIG) asm volatile("" : "+v"(asr2));
#pragma unroll
    for (int j = 0; j < D; ++j) {
      scales_to_operand_order(j, (uint32_t)asr[j], tid);
      if constexpr (BIG) scales_to_operand_order(j, (uint32_t)asr2[j], row_hi);
    }
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

  // ---- the next tile's first loads, and what the tile after it needs, go out ahead of the epilogue ---------
  // The loads of the next tile's first D slices are in flight from here until the wait that follows the epilogue
  // (into the ring stages 0 .. D-1 and into the raw register sets: the epilogue keeps to the last ring stage and
  // leaves those registers alone), and so are the loads of the next tile's affinities and bias and of the token
  // ids of the tile after it.
  // No branch surrounds any of these loads (see above): after the last tile of the list they are issued all the
  // same, the slices through descriptors of zero records (no traffic), the rest from the addresses of the last
  // tile.
  const bool have_nn = Ln + Lstep < endL;
  const Tile nxt = tile_at(have_next ? Ln : L);
  const Tile nn = tile_at(have_nn ? Ln + Lstep : L);
  const int nbuf = have_next ? buf ^ 1 : buf;  // (behind the last tile: its own row table, which holds valid ids)
  tile_live = have_next ? -1 : 0;
  aim_loads_at(nxt, nbuf);
  // (down stage: they go out a few at a time between the row tiles of the epilogue, see there; not for the smallest
  // tiles, whose launches do little but stream weights: there every load asked for later is time lost, 2 % of the
  // down launch at decode sizes)
  constexpr bool SPREAD_FIRST = STAGE == 2 && NMT >= 8;
  if constexpr (!SPREAD_FIRST) request_first_slices();
  if (AFF_ROWS) aff_raw(nxt, nbuf, aff_n);
  rs_raw(nxt, nbuf, rs_n);
  bias_raw(nxt, bias_n);
  wsc_raw(nxt, wsc_n);
  ids_raw(nn, ids_nn);

  // ---- epilogue ---------------------------------------------------------------------------------------------
  // What the epilogue derives from the thread index it derives again here, from a copy the compiler cannot see
  // through: otherwise those values are kept in registers across the K loop, where every register counts.
  int tid_e = threadIdx.x;
  asm volatile("" : "+v"(tid_e));
  const int c_e = tid_e & 15, g_e = (tid_e & 63) >> 4;
  const int hcol_e = (STAGE == 1) ? (c_e >> 3) : 0, cl_e = (STAGE == 1) ? (c_e & 7) : c_e;
  if (STAGE == 1) {
    // act(gate + bias) * (up + bias) in registers, then through LDS, 64 rows at a time, as
    // [row][q][32 partitions] fp32; then one thread per MX block (8 partitions x 4 q) quantises and
    // writes 32 K-contiguous bytes plus the scale byte.
    // (the exchange buffer is the last ring stage, and for the 256-row variants the first 2 KB of the scale stages
    // behind it: the stages before it are receiving the next tile's first slices)
    float* E = (float*)(smem + (RING - 1) * SA);
    static_assert((RING - 1) * SA + MX_LDS_EPI <= Cfg::LDS, "the exchange buffer must fit behind the stages in flight");
    // the lane's four partitions within the workgroup's 32: 4*cl + t
    float bg[4], bu[4];
    {
      const float4 vg = *(const float4*)(s_bias[buf] + q * 32 + 4 * cl_e), vu = *(const float4*)(s_bias[buf] + 128 + q * 32 + 4 * cl_e);
      bg[0] = vg.x; bg[1] = vg.y; bg[2] = vg.z; bg[3] = vg.w;
      bu[0] = vu.x; bu[1] = vu.y; bu[2] = vu.z; bu[3] = vu.w;
    }
    float sg[4] = {1.f, 1.f, 1.f, 1.f}, su[4] = {1.f, 1.f, 1.f, 1.f};  // fp8-row kind: the columns' weight scales
    if constexpr (ROW8) {
      const float4 vg = *(const float4*)(s_wsc[buf] + q * 32 + 4 * cl_e), vu = *(const float4*)(s_wsc[buf] + 128 + q * 32 + 4 * cl_e);
      sg[0] = vg.x; sg[1] = vg.y; sg[2] = vg.z; sg[3] = vg.w;
      su[0] = vu.x; su[1] = vu.y; su[2] = vu.z; su[3] = vu.w;
    }
    const int pl0 = 4 * cl_e;
    constexpr int NPS = (NMT + 3) / 4;  // passes of 64 rows (the last one may hold two row tiles only)
    // Clamps as an unconditional median of three against +-inf, and the activation kind as a compile-time
    // constant of the pass: a lane evaluates 128 elements here, and per-element decisions made this
    // code longer (and slower) than the K loop.
    // (derived here, behind a statement the compiler cannot look through, and kept in scalar registers: computed
    // once ahead of the tile loop they would sit in vector registers across the K loop)
    int cmask = a.clamp_mask;
    asm volatile("" : "+s"(cmask));
    const float inf = __builtin_inff();
    auto limit = [&](int bit, float v, float none) {
      return __builtin_bit_cast(float, uni(__builtin_bit_cast(int, (cmask & bit) ? v : none)));
    };
    // min(max(v, lo), hi) as one median of three: the same value whenever lo <= hi, and with lo > hi (every v
    // then becomes hi) once lo is lowered to hi
    const float g_hi = limit(MOE_CLAMP_GATE_HI, a.clamp[0], inf);
    const float g_lo = limit(MOE_CLAMP_GATE_LO, fminf(a.clamp[1], g_hi), -inf);
    const float u_hi = limit(MOE_CLAMP_UP_HI, a.clamp[2], inf);
    const float u_lo = limit(MOE_CLAMP_UP_LO, fminf(a.clamp[3], u_hi), -inf);
    // (PLAIN: neither bias nor clamps, the fused act(gate) * up of most layers; their adds and medians are left out)
    // fp8-row and bf16 kinds: the results go out in natural column order, which is the order the lanes hold them in
    // (a lane's four partitions are four neighbouring columns), so they are stored straight from the registers, through
    // a descriptor that ends behind the chunk's last row (rows past it are dropped by the range check); only the MX
    // formats, whose blocks of 32 columns span the four waves, go through the exchange buffer.
    const int y_rowb = uni(BF16 ? (int)(a.y_stride * 2) : (int)(a.y32_stride * 4));
    const v4i rdy = make_rsrc(BF16 ? (const void*)((const uint8_t*)a.Yq + (int64_t)cur.slot0 * y_rowb)
                                   : (const void*)((const uint8_t*)a.Y32 + (int64_t)cur.slot0 * y_rowb),
                              ROW8 ? (uint32_t)(cur.nrows * y_rowb) : 0u);
    const uint32_t y_voff = (uint32_t)((4 * g_e + 2 * hcol_e) * y_rowb) +
                            (uint32_t)(tile_tI(cur) * 512 + q * tile_Pt(cur) + tile_p0(cur) + pl0) * (BF16 ? 2u : 4u);
    auto passes = [&](auto act_, auto plain_) {
    constexpr int ACT = decltype(act_)::value;
    constexpr bool PLAIN = decltype(plain_)::value;
    static_for<0, NPS>([&](auto ps_) {
      constexpr int ps = decltype(ps_)::value;
      if (ps * 64 < cur.nrows) {
        if constexpr (!ROW8) lds_barrier();
        static_for<0, 4>([&](auto m_) {
          constexpr int ml = decltype(m_)::value;
          constexpr int mt = ps * 4 + ml;
          if constexpr (mt < NMT) {
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
          float ckg[4][2], cku[4][2];  // bf16 kind: gate / up ahead of the activation, for the checkpoint
          float rsk[2] = {1.f, 1.f};  // fp8-row kind: the scales of the lane's two rows
          if constexpr (ROW8) {
            const float2 rr = *(const float2*)(s_rs[buf] + ps * 64 + ml * 16 + 4 * g_e + 2 * hcol_e);
            rsk[0] = rr.x; rsk[1] = rr.y;
          }
#pragma unroll
          for (int t = 0; t < 4; ++t) {
#pragma unroll
            for (int k = 0; k < 2; ++k) {
              // (the rotation writes one half of the 16 lanes only: banks 2, 3 = the up lanes take the gate lanes'
              // rows 2, 3; banks 0, 1 = the gate lanes take the up lanes' rows 0, 1; the other half keeps its own)
              const int lo = __builtin_bit_cast(int, av[t][k]), hi = __builtin_bit_cast(int, av[t][2 + k]);
              float gv = __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(lo, hi, 0x128 /* row_ror:8 */, 0xf, 0xc, false));
              float uv = __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(hi, lo, 0x128 /* row_ror:8 */, 0xf, 0x3, false));
              if constexpr (ROW8) {
                gv = (gv * sg[t]) * rsk[k];
                uv = (uv * su[t]) * rsk[k];
              }
              const float gg = PLAIN ? gv : __builtin_amdgcn_fmed3f(gv + bg[t], g_lo, g_hi);
              const float uu = PLAIN ? uv : __builtin_amdgcn_fmed3f(uv + bu[t], u_lo, u_hi);
              y[k][t] = act_apply(gg, ACT) * uu;
              if constexpr (BF16) {
                ckg[t][k] = gg;
                cku[t][k] = uu;
              }
            }
          }
          if constexpr (BF16) {
            // activation checkpoint [N, 2, I, B] (bwmm_shard_on_I.py:160-176): gate / up projections after scale, bias
            // and clamp, transposed: the lane's two rows are neighbours along B
            const int row = ps * 64 + ml * 16 + 4 * g_e + 2 * hcol_e;
            if (a.ckpt != nullptr && row < cur.nrows) {
              const uint32_t slot = (uint32_t)(cur.slot0 + row);
              const uint32_t n = slot / (uint32_t)a.ckpt_B, r = slot - n * (uint32_t)a.ckpt_B;
              const int64_t col = (int64_t)tile_tI(cur) * 512 + (int64_t)q * tile_Pt(cur) + tile_p0(cur) + pl0;
              uint16_t* ck = a.ckpt + (((int64_t)n * 2) * a.ckpt_I + col) * a.ckpt_B + r;
              // (an even block size keeps the pair inside one block and the store aligned; otherwise row by row)
              const bool pair = (a.ckpt_B & 1) == 0;
              const uint32_t slot1 = slot + 1, n1 = slot1 / (uint32_t)a.ckpt_B, r1 = slot1 - n1 * (uint32_t)a.ckpt_B;
              uint16_t* ck1 = a.ckpt + (((int64_t)n1 * 2) * a.ckpt_I + col) * a.ckpt_B + r1;
#pragma unroll
              for (int t = 0; t < 4; ++t) {
                const uint32_t gp = pack2_bf16(ckg[t][0], ckg[t][1]), up = pack2_bf16(cku[t][0], cku[t][1]);
                if (pair) {
                  *(uint32_t*)(ck + (int64_t)t * a.ckpt_B) = gp;
                  *(uint32_t*)(ck + ((int64_t)a.ckpt_I + t) * a.ckpt_B) = up;
                } else {
                  ck[(int64_t)t * a.ckpt_B] = (uint16_t)gp;
                  ck[((int64_t)a.ckpt_I + t) * a.ckpt_B] = (uint16_t)up;
                  if (row + 1 < cur.nrows) {
                    ck1[(int64_t)t * a.ckpt_B] = (uint16_t)(gp >> 16);
                    ck1[((int64_t)a.ckpt_I + t) * a.ckpt_B] = (uint16_t)(up >> 16);
                  }
                }
              }
            }
          }
#pragma unroll
          for (int k = 0; k < 2; ++k) {
            if constexpr (BF16) {
              typedef __bf16 v2bf_ __attribute__((ext_vector_type(2)));
              typedef float v2f_ __attribute__((ext_vector_type(2)));
              const v2f_ p0 = {y[k][0], y[k][1]}, p1 = {y[k][2], y[k][3]};
              const v2i o = {__builtin_bit_cast(int, __builtin_convertvector(p0, v2bf_)),
                             __builtin_bit_cast(int, __builtin_convertvector(p1, v2bf_))};
              st_b64(o, y_voff, rdy, (ps * 64 + ml * 16 + k) * y_rowb);
            } else if constexpr (ROW8) {
              const v4i o = {__builtin_bit_cast(int, y[k][0]), __builtin_bit_cast(int, y[k][1]),
                             __builtin_bit_cast(int, y[k][2]), __builtin_bit_cast(int, y[k][3])};
              st_b128(o, y_voff, rdy, (ps * 64 + ml * 16 + k) * y_rowb);
            } else {
              const int rl = ml * 16 + 4 * g_e + 2 * hcol_e + k;
              *(float4*)(E + rl * MX_EP + q * 32 + pl0) = make_float4(y[k][0], y[k][1], y[k][2], y[k][3]);
            }
          }
          }
        });
        if constexpr (!ROW8) {
        lds_barrier();
        // thread (rl = tid/4, j = tid%4): MX block of chunk row ps*64 + rl, partitions 8j .. 8j+7 of the 32 (x 4 q)
        const int rl = tid_e >> 2, j = tid_e & 3;
        const int row = ps * 64 + rl;
        if (row < cur.nrows) {
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
          const int64_t slot = cur.slot0 + row;
          const int pw = tile_p0(cur) + 8 * j;  // first partition of the block within the intermediate tile
          uint4* o = (uint4*)(a.Yq + slot * a.y_stride + tile_tI(cur) * 512 + pw * 4);
          o[0] = make_uint4(d[0], d[1], d[2], d[3]);
          o[1] = make_uint4(d[4], d[5], d[6], d[7]);
          a.Ys[slot * a.ys_stride + tile_tI(cur) * 16 + (pw >> 3)] = (uint8_t)sb;
        }
        }
      }
    });
    };
    // (the plain form exists for SiLU alone: every instance of this code lengthens the build)
    const bool plain = cmask == 0 && a.bias == nullptr;
    switch (a.act_fn) {
      case MOE_ACT_SILU:
        if (plain) passes(std::integral_constant<int, MOE_ACT_SILU>{}, std::true_type{});
        else passes(std::integral_constant<int, MOE_ACT_SILU>{}, std::false_type{});
        break;
      case MOE_ACT_GELU: passes(std::integral_constant<int, MOE_ACT_GELU>{}, std::false_type{}); break;
      case MOE_ACT_GELU_TANH: passes(std::integral_constant<int, MOE_ACT_GELU_TANH>{}, std::false_type{}); break;
      default: passes(std::integral_constant<int, MOE_ACT_SWISH>{}, std::false_type{}); break;
    }
    // the scale stages that the exchange buffer reaches into are written at the top of the next tile
    if constexpr (!ROW8) lds_barrier();
  } else {
    const int64_t col0 = tile_h0(cur) + 64 * q + 4 * c_e;
    float bd[4];
    {
      const float4 vb = *(const float4*)(s_bias[buf] + 64 * q + 4 * c_e);
      bd[0] = vb.x; bd[1] = vb.y; bd[2] = vb.z; bd[3] = vb.w;
    }
    float sd[4] = {1.f, 1.f, 1.f, 1.f};  // fp8-row kind: the columns' weight scales
    if constexpr (ROW8) {
      const float4 vs = *(const float4*)(s_wsc[buf] + 64 * q + 4 * c_e);
      sd[0] = vs.x; sd[1] = vs.y; sd[2] = vs.z; sd[3] = vs.w;
    }
    const bool post = a.scaling_mode == MOE_SCALE_POST;
    // Rows go out through a descriptor that ends after the chunk's last row, so rows past the end
    // are dropped by the range check and the stores need no branches.  (Rows of padding slots
    // inside the chunk are written too: nothing reads the contributions of such slots.)
    const v4i rd = make_rsrc(a.D + (int64_t)cur.slot0 * a.H, (uint32_t)((int64_t)cur.nrows * a.H * 2));
    // bf16 kind: the down checkpoint [N, B, H] = [slots, H] (bwmm_shard_on_I.py:160-176) takes the same rows ahead of
    // the affinity (a descriptor of zero records when there is none: the stores then go nowhere)
    const v4i rdc = make_rsrc((BF16 && a.ckpt) ? a.ckpt + (int64_t)cur.slot0 * a.H : a.D,
                              (BF16 && a.ckpt) ? (uint32_t)((int64_t)cur.nrows * a.H * 2) : 0u);
    const uint32_t d_voff = (uint32_t)((4 * g_e * a.H + col0) * 2);
    const int rowb = uni(a.H * 2);
    typedef __bf16 v2bf __attribute__((ext_vector_type(2)));
    typedef float v2f __attribute__((ext_vector_type(2)));
    // the affinities of the lane's rows (4 consecutive rows per row tile) are read two row tiles ahead of their
    // use: a read per store, waited for on the spot, made the LDS latency the epilogue's pace
    v4f aff_q[3];
    aff_q[0] = *(const v4f*)(s_aff[buf] + 0 * 16 + 4 * g_e);
    aff_q[1] = *(const v4f*)(s_aff[buf] + 1 * 16 + 4 * g_e);
    v4f rs_q[3];  // fp8-row kind: the rows' activation scales, read ahead the same way
    if constexpr (ROW8) {
      rs_q[0] = *(const v4f*)(s_rs[buf] + 0 * 16 + 4 * g_e);
      rs_q[1] = *(const v4f*)(s_rs[buf] + 1 * 16 + 4 * g_e);
    }
    static_for<0, NMT>([&](auto mt_) {
      constexpr int mt = decltype(mt_)::value;
      if constexpr (mt + 2 < NMT) aff_q[(mt + 2) % 3] = *(const v4f*)(s_aff[buf] + (mt + 2) * 16 + 4 * g_e);
      if constexpr (ROW8 && mt + 2 < NMT) rs_q[(mt + 2) % 3] = *(const v4f*)(s_rs[buf] + (mt + 2) * 16 + 4 * g_e);
      const v4f aff4 = post ? aff_q[mt % 3] : (v4f){1.f, 1.f, 1.f, 1.f};
      float av[4][4];  // [column tile][row]
      static_for<0, 16>([&](auto i_) {
        constexpr int i = decltype(i_)::value;
        if constexpr (mt < 16) av[i / 4][i % 4] = acc_get<16 * mt + i>();
        else av[i / 4][i % 4] = accv[mt - 16][i / 4][i % 4];
      });
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const float af = aff4[r];
        if constexpr (ROW8) {
          const float rs = rs_q[mt % 3][r];
#pragma unroll
          for (int t = 0; t < 4; ++t) av[t][r] = (av[t][r] * sd[t]) * rs;
        }
        v2i o;
        if constexpr (BF16) {
          v2i oc;
#pragma unroll
          for (int t = 0; t < 4; t += 2) {
            const v2f d = {av[t][r] + bd[t], av[t + 1][r] + bd[t + 1]};
            oc[t >> 1] = __builtin_bit_cast(int, __builtin_convertvector(d, v2bf));
          }
          st_b64(oc, d_voff, rdc, (mt * 16 + r) * rowb);
        }
#pragma unroll
        for (int t = 0; t < 4; t += 2) {
          const v2f d = {(av[t][r] + bd[t]) * af, (av[t + 1][r] + bd[t + 1]) * af};
          o[t >> 1] = __builtin_bit_cast(int, __builtin_convertvector(d, v2bf));
        }
        st_b64(o, d_voff, rd, (mt * 16 + r) * rowb);
      }
      // The next tile's first slices, a share behind every row tile: asked for all at once ahead of the epilogue
      // they fill the CU's load queue, the wave stands at the first instruction that does not fit until the memory
      // system has worked the queue down, and this arithmetic and these stores, which could run meanwhile, wait
      // behind it.
      constexpr int PER = (NFIRST + NMT - 1) / NMT;
      if constexpr (SPREAD_FIRST) request_first(std::integral_constant<int, mt * PER>{}, std::integral_constant<int, (mt + 1) * PER>{});
    });
  }
  tile_live = -1;

  // ---- hand over to the next tile ------------------------------------------------------------------------
  // Everything in flight lands here: the next tile's first slices, this tile's stores (stores and loads share
  // the counter but complete in no fixed order between them, so the K loop's counting waits must not start
  // while stores are out), and the small loads issued ahead of the epilogue, which may be used from here on.
  all_loads_landed(ids_nn, aff_n, bias_n, rs_n, wsc_n);
  if (!have_next) break;
  if (STAGE == 2) aff_put(nxt.e, buf ^ 1, aff_n);
  rs_put(nxt.e, buf ^ 1, rs_n, aff_n);
  bias_put(nxt, buf ^ 1, bias_n);
  wsc_put(buf ^ 1, wsc_n);
  if (have_nn) ids_put(buf, nn.nrows, ids_nn);  // the table of the tile that has just ended
  cur = nxt;
  L = Ln;
  Ln += Lstep;
  have_next = have_nn;
  buf ^= 1;
  }
  return Ln;
}


// One translation unit per (stage, weight format): the build compiles this file once for each with
// MX_INST_STAGE / MX_INST_WFMT defined, and once without them for the dispatcher below.
#if defined(MX_INST_STAGE)
template <int STAGE, int WFMT>
__global__ __launch_bounds__(MXT) __attribute__((amdgpu_waves_per_eu(1, 1))) void mx_gemm_kernel(const MxArgs a) {
  extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
  __shared__ int s_tok[2][MX_ROWS_MAX];
  __shared__ __attribute__((aligned(16))) float s_aff[2][MX_ROWS_MAX];
  __shared__ __attribute__((aligned(16))) float s_bias[2][MXT];
  // the fp8-row kind's row and column scales (a token entry each for the other formats)
  __shared__ __attribute__((aligned(16))) float s_rs[2][(WFMT == MX_WFMT_ROW8 || WFMT == MX_WFMT_BF16) ? MX_ROWS_MAX : 4];
  __shared__ __attribute__((aligned(16))) float s_wsc[2][(WFMT == MX_WFMT_ROW8 || WFMT == MX_WFMT_BF16) ? MXT : 4];
  // One workgroup per CU, for the whole launch.  Workgroups are handed to the 8 XCDs round-robin by linear
  // index, and each XCD has its own L2.  XCD x therefore takes the x-th of eight contiguous parts of the chunk
  // list (chunks are ordered by expert; the parts hold about equal work), as a queue of items (chunk, column
  // tile) with the chunks grouped by class and, inside a class, the column tiles innermost (or alternating between
  // a few chunks of one expert, see tile_at); its workgroups take the items w, w + W, w + 2W, ... (W workgroups on
  // the XCD).  The workgroups that share an activation tile, and the chunks that share an expert's weights, then run
  // at the same time behind the same L2, so each operand crosses the fabric about once; and a workgroup's
  // consecutive items are of one class, i.e. one instance of the code below, which carries its loads from tile
  // to tile.
  const int xcd = blockIdx.x & 7, w = blockIdx.x >> 3, W = gridDim.x >> 3;
  // (for a caller that wants to know the clock the part held under this launch, see MxArgs::clk)
  const long long clk0 = a.clk ? clock64() : 0, tick0 = a.clk ? wall_clock64() : 0;
  const int32_t* qo = a.q_off + xcd * (CHUNK_CLASSES + 1);
  const int qbase = __builtin_amdgcn_readfirstlane(qo[0]);
  const int interleave = __builtin_amdgcn_readfirstlane(a.q_off[8 * (CHUNK_CLASSES + 1)]);
  int L = w;
  // classes in queue order (CHUNK_CLASS_TILES / CHUNK_CLASS_LAST in combine.hpp)
#define MX_RUN_CLASS(CLS_)                                                                                     \
  {                                                                                                            \
    const int startL = (__builtin_amdgcn_readfirstlane(qo[CLS_]) - qbase) * a.col_tiles;                       \
    const int endL = (__builtin_amdgcn_readfirstlane(qo[CLS_ + 1]) - qbase) * a.col_tiles;                     \
    if (L < endL)                                                                                              \
      L = mx_gemm_tiles<STAGE, CHUNK_CLASS_TILES[CLS_], CHUNK_CLASS_LAST[CLS_], WFMT>(                         \
          a, smem, s_tok, s_aff, s_bias, (float(*)[MX_ROWS_MAX])s_rs, (float(*)[MXT])s_wsc, L, startL, endL,  \
          W, qbase, interleave);                                                                               \
    __syncthreads();                                                                                           \
  }
  // The same for a run of neighbouring classes on one instance of the tile loop (whose row tiles cover the largest).
#define MX_RUN_RANGE(C0_, C1_, TILES_, LAST_)                                                                  \
  {                                                                                                            \
    static_assert(CHUNK_CLASS_TILES[C0_] <= TILES_ && CHUNK_CLASS_LAST[C0_] == LAST_ &&                        \
                  CHUNK_CLASS_LAST[C1_] == LAST_, "the instance covers the classes of the run");              \
    const int startL = (__builtin_amdgcn_readfirstlane(qo[C0_]) - qbase) * a.col_tiles;                        \
    const int endL = (__builtin_amdgcn_readfirstlane(qo[C1_ + 1]) - qbase) * a.col_tiles;                      \
    if (L < endL)                                                                                              \
      L = mx_gemm_tiles<STAGE, TILES_, LAST_, WFMT>(a, smem, s_tok, s_aff, s_bias, (float(*)[MX_ROWS_MAX])s_rs, \
                                                    (float(*)[MXT])s_wsc, L, startL, endL, W, qbase, interleave); \
    __syncthreads();                                                                                           \
  }
  static_assert(CHUNK_CLASSES == 12, "one MX_RUN_CLASS per class");
  if constexpr (WFMT == MX_WFMT_E4M3) {
    MX_RUN_CLASS(0)
    MX_RUN_CLASS(1)
    MX_RUN_CLASS(2)
    MX_RUN_CLASS(3)
    MX_RUN_CLASS(4)
    MX_RUN_CLASS(5)
    MX_RUN_CLASS(6)
    MX_RUN_CLASS(7)
    MX_RUN_CLASS(8)
    MX_RUN_CLASS(9)
    MX_RUN_CLASS(10)
    MX_RUN_CLASS(11)
  } else {
    // Every other format runs the last chunks of 10 .. 18 row tiles on the instances of 16 and 20: the finer
    // classes pay where experts hold a router's ragged 256 +- 15 rows (the e4m3 workloads that are timed), and
    // each instance costs this file a twelfth of its compile time.
    MX_RUN_RANGE(0, 0, 20, false)
    MX_RUN_RANGE(1, 2, 20, true)
    MX_RUN_RANGE(3, 3, 16, false)
    MX_RUN_RANGE(4, 7, 16, true)
    MX_RUN_RANGE(8, 8, 8, false)
    MX_RUN_RANGE(9, 9, 8, true)
    MX_RUN_RANGE(10, 10, 4, false)
    MX_RUN_RANGE(11, 11, 4, true)
  }
#undef MX_RUN_RANGE
#undef MX_RUN_CLASS
  if (a.clk && blockIdx.x == 0 && threadIdx.x == 0) {
    a.clk[0] = clock64() - clk0;
    a.clk[1] = wall_clock64() - tick0;
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

// The weights of one stage in the kernel's read order (see launch_mx_pack_weights in bwmm.hpp).  One thread per
// lane-sized piece (16 bytes, 8 for 4-bit weights); the source address is what mx_gemm_tiles computes for that load
// (w_voff + w_soff[i] + w_off).
template <int LB>
__global__ __launch_bounds__(256) void mx_pack_weights_kernel(int stage, const uint8_t* __restrict__ W,
                                                              uint8_t* __restrict__ dst, int64_t H, int64_t I,
                                                              int64_t col_tiles, int64_t nks, int64_t pieces) {
  constexpr bool FP4 = LB == 8;
  constexpr int ES = FP4 ? 2 : 4, GROWS = FP4 ? 8 : 4;
  const int64_t d = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (d >= pieces) return;
  const int lane = (int)(d & 63), i = (int)((d >> 6) & 7), q = (int)((d >> 9) & 3);
  const int64_t ks = (d >> 11) % nks, xt = ((d >> 11) / nks) % col_tiles, e = (d >> 11) / (nks * col_tiles);
  const int g = lane >> 4, c = lane & 15;
  const int64_t pr = FP4 ? i : ((i < 4) ? i : (16 + i - 4)), kt = ks >> 2, pb = ks & 3;
  int64_t elem, expert_elems;
  if (stage == 1) {
    const int64_t nH = H / 512, pstride = 2 * nH * I;
    const int64_t tI = xt >> 2, p0 = (xt & 3) * 32;
    const int64_t rows_t = (I - tI * 512 < 512) ? (I - tI * 512) : 512;
    const int64_t colu = tI * 512 + q * (rows_t / 4) + p0;
    elem = (GROWS * g + pr + pb * 32) * pstride + (c >> 3) * nH * I + 4 * (c & 7) + colu + kt * I;
    expert_elems = 128 * pstride;
  } else {
    const int64_t nI = (I + 511) / 512, pI = I > 512 ? 128 : I / 4, pstride = nI * H;
    elem = (GROWS * g + pr + pb * 32) * pstride + 4 * c + xt * 256 + 64 * q + kt * H;
    expert_elems = pI * pstride;
  }
  const uint8_t* src = W + (e * expert_elems + elem) * ES;
  if constexpr (FP4) *(uint2*)(dst + d * LB) = *(const uint2*)src;
  else *(uint4*)(dst + d * LB) = *(const uint4*)src;
}

static void mx_pack_geometry(int stage, int64_t H, int64_t I, int64_t* col_tiles, int64_t* nks) {
  const int64_t over_i = (I / 512) * 4 + (I % 512) / 128;
  *col_tiles = stage == 1 ? over_i : H / 256;
  *nks = stage == 1 ? H / 128 : over_i;
}
size_t mx_packed_weights_bytes(int stage, int fp4, int64_t E, int64_t H, int64_t I) {
  int64_t ct, nks;
  mx_pack_geometry(stage, H, I, &ct, &nks);
  return (size_t)E * ct * nks * (fp4 ? 16384 : 32768);
}
int launch_mx_pack_weights(int stage, int fp4, const void* W, void* dst, int64_t E, int64_t H, int64_t I,
                           hipStream_t s) {
  if (!mx_fast_path_ok(H, I) || (((uintptr_t)W) & 15) != 0 || (((uintptr_t)dst) & 15) != 0) return MOE_E_BAD_ARG;
  int64_t ct, nks;
  mx_pack_geometry(stage, H, I, &ct, &nks);
  const int64_t pieces = E * ct * nks * 2048;
  if ((pieces + 255) / 256 >= (int64_t)1 << 31) return MOE_E_BAD_SHAPE;
  const dim3 grid((unsigned)((pieces + 255) / 256));
  if (fp4)
    hipLaunchKernelGGL(mx_pack_weights_kernel<8>, grid, dim3(256), 0, s, stage, (const uint8_t*)W, (uint8_t*)dst, H, I,
                       ct, nks, pieces);
  else
    hipLaunchKernelGGL(mx_pack_weights_kernel<16>, grid, dim3(256), 0, s, stage, (const uint8_t*)W, (uint8_t*)dst, H, I,
                       ct, nks, pieces);
  MOE_CHECK_LAUNCH();
  return MOE_OK;
}

int launch_mx_gemm_s1_f0(const MxArgs& m, unsigned grid, hipStream_t s);
int launch_mx_gemm_s2_f0(const MxArgs& m, unsigned grid, hipStream_t s);
int launch_mx_gemm_s1_f1(const MxArgs& m, unsigned grid, hipStream_t s);
int launch_mx_gemm_s2_f1(const MxArgs& m, unsigned grid, hipStream_t s);
int launch_mx_gemm_s1_f2(const MxArgs& m, unsigned grid, hipStream_t s);
int launch_mx_gemm_s2_f2(const MxArgs& m, unsigned grid, hipStream_t s);
int launch_mx_gemm_s1_f3(const MxArgs& m, unsigned grid, hipStream_t s);
int launch_mx_gemm_s2_f3(const MxArgs& m, unsigned grid, hipStream_t s);
int launch_mx_gemm_s1_f4(const MxArgs& m, unsigned grid, hipStream_t s);
int launch_mx_gemm_s2_f4(const MxArgs& m, unsigned grid, hipStream_t s);

int launch_mx_gemm(int stage, const MxArgs& m0, unsigned gx, unsigned gy, hipStream_t s) {
  if (gx == 0 || gy == 0) return MOE_OK;
  MxArgs m = m0;
  m.col_tiles = (int32_t)gx;
  // one workgroup per CU (a workgroup fills a CU's registers and most of its LDS, and walks its share of the
  // tiles itself); fewer when there cannot be that many tiles (gy = upper bound on the number of chunks)
  int dev = 0, cus = 0;
  if (hipGetDevice(&dev) != hipSuccess ||
      hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus < 8)
    return MOE_E_LAUNCH;
  const uint64_t tiles = (uint64_t)gx * gy;
  unsigned per_xcd = (unsigned)cus / 8u;
  if ((tiles + 7u) / 8u < per_xcd) per_xcd = (unsigned)((tiles + 7u) / 8u);
  const unsigned grid = 8u * per_xcd;
  switch (m.wfmt) {
    case MX_WFMT_E4M3: return stage == 1 ? launch_mx_gemm_s1_f0(m, grid, s) : launch_mx_gemm_s2_f0(m, grid, s);
    case MX_WFMT_E5M2: return stage == 1 ? launch_mx_gemm_s1_f1(m, grid, s) : launch_mx_gemm_s2_f1(m, grid, s);
    case MX_WFMT_E2M1: return stage == 1 ? launch_mx_gemm_s1_f2(m, grid, s) : launch_mx_gemm_s2_f2(m, grid, s);
    case MX_WFMT_ROW8: return stage == 1 ? launch_mx_gemm_s1_f3(m, grid, s) : launch_mx_gemm_s2_f3(m, grid, s);
    case MX_WFMT_BF16: return stage == 1 ? launch_mx_gemm_s1_f4(m, grid, s) : launch_mx_gemm_s2_f4(m, grid, s);
    default: return MOE_E_BAD_ARG;
  }
}

#endif

}  // namespace moe
