// MXFP8 blockwise expert GEMMs for gfx950, large-tile version.
//
// A 256-thread workgroup (4 waves, one per SIMD) owns an "expert chunk" of up to 256 consecutive
// slots of one expert (two 128-token blocks) and 256 output columns:
//   gate/up: 32 intermediate partitions p x 4 q, for gate and for up; wave w owns q = w
//   down:    256 hidden columns; wave w owns 64 of them
// so every weight byte that enters the CU is used by 256 rows, and both operands enter the CU
// exactly once per workgroup: the bytes a CU pulls through its L1 per flop are what bounds this
// kernel (smaller or split tiles were measured: 128-row workgroups double the traffic into the
// CU and, because sibling workgroups drift apart by more K slices than the L2 holds, the traffic
// over the fabric as well).  Each wave keeps a 256 x 64 accumulator tile (16 x 4 MFMA 16x16
// tiles, 256 accumulator registers).
//
// With one wave per SIMD nothing overlaps unless the instruction stream says so:
//   * the loads of the coming K slices are issued a few at a time between the MFMA groups of slice ks
//     (a burst of loads blocks the wave at the issue stage for thousands of cycles while the
//     matrix pipe drains);
//   * expert weights (B operand) go global -> registers, never through LDS.  In the reference
//     layout a weight column's K runs over partitions p (4 K-bytes per 4-byte element), and lane
//     group g of v_mfma_scale_f32_16x16x128_f8f6f4 needs K bytes [16g,16g+16) and [64+16g,
//     64+16g+16) of the 128-byte K slice, i.e. partitions 4g..4g+3 and 16+4g..16+4g+3 of the 32
//     partitions of the slice: eight loads per lane, each fetching 2 (gate/up) or 4 (down)
//     adjacent columns = 2 or 4 MFMA column tiles at once.  One load instruction reads four
//     full 128/256-byte row segments.  The loads land in one of two "raw" register sets, two
//     slices ahead; a set is transposed into MFMA operand order at the top of the slice that uses
//     it;
//   * activations (A operand, rows gathered through token_position_to_id) are staged through a
//     three-deep LDS ring of 256 rows x 128 K-bytes, read by all four waves; the fragments of the
//     next two row tiles are read while the current two multiply;
//   * E8M0 scales ride along: A scales sit in LDS transposed to [g][row%16][row/16] so that one
//     16-byte read gives a lane the scales of all 16 row tiles (selected with op_sel); B scales
//     are 2-4 bytes per lane per K slice straight from global.
// The gate/up epilogue computes act(gate)*up in registers (a lane holds gate and up of the same
// element) and exchanges the products through LDS so that the MX re-quantisation sees the
// reference's blocks (8 partitions x 4 q) and writes K-contiguous rows for the down GEMM.
//
// Reference semantics: test/integration/nkilib/core/mlp/test_mlp_common.py:550-682 (layouts,
// re-quantisation), test/integration/nkilib/core/moe/moe_cte/test_utils.py:474-735 (block loop).
#include <type_traits>

#include "bwmm.hpp"

#ifndef MX_DBG_WAIT0
#define MX_DBG_WAIT0 0
#endif
namespace moe {

constexpr int MXT = 256;                       // threads
constexpr int MXM = CHUNK_ROWS;                // 256 rows per workgroup
constexpr int MXROW = 128;                     // LDS pitch of one staged row; 16-byte chunk ch of row r sits in
                                               // slot ch ^ (r & 7), which makes the fragment reads (16 rows x 4
                                               // chunks per instruction) and the staging writes conflict free
constexpr int MX_NST = 3;                      // depth of the activation ring
constexpr int MX_SA = MXM * MXROW;             // one A buffer (32 KB)
constexpr int MX_SS = 4 * 16 * 16;             // one A-scale buffer, [g][c][mt] bytes
constexpr int MX_EP = 128 + 8;                 // epilogue exchange: floats per row ([q][32 partitions] + pad)
constexpr int MX_LDS_LOOP = MX_NST * (MX_SA + MX_SS);
constexpr int MX_LDS_EPI = 64 * MX_EP * 4;
constexpr int MX_LDS = MX_LDS_EPI > MX_LDS_LOOP ? MX_LDS_EPI : MX_LDS_LOOP;
static_assert(MXM == 256, "the kernel is written for 256-row chunks");

template <int I, int N, class F>
__device__ __forceinline__ void static_for(F&& f) {
  if constexpr (I < N) {
    f(std::integral_constant<int, I>{});
    static_for<I + 1, N>(f);
  }
}

struct BFrag {
  v8i f[4];  // four column tiles
  int sc;    // their E8M0 scale bytes (byte t = tile t)
};

__device__ __forceinline__ v8i frag_from_lds(const uint8_t* plo, const uint8_t* phi) {
  const v4i lo = *(const v4i*)plo;
  const v4i hi = *(const v4i*)phi;
  v8i r;
  r[0] = lo[0]; r[1] = lo[1]; r[2] = lo[2]; r[3] = lo[3];
  r[4] = hi[0]; r[5] = hi[1]; r[6] = hi[2]; r[7] = hi[3];
  return r;
}

// One MFMA of row-tile fragment `af` (scale byte OA of `sa`) with column tile NT of `b`, written as
// an instruction: statements of this kind keep their order, so what the source puts between two
// MFMAs (a load, an LDS read) is issued between them and runs in the shadow of the first -- with one
// wave per SIMD nothing else hides it.  op_sel / op_sel_hi carry bit 0 / bit 1 of the two scale
// byte selectors.
#define MX_MFMA_CASE(OA_, OB_, SEL_, SELHI_)                                                              \
  if constexpr (OA == OA_ && OB == OB_)                                                                   \
    asm volatile("v_mfma_scale_f32_16x16x128_f8f6f4 %0, %1, %2, %0, %3, %4 op_sel:" SEL_ " op_sel_hi:" SELHI_ \
                 : "+a"(c) : "v"(af), "v"(bf), "v"(sa), "v"(sb))
template <int OA, int OB>
__device__ __forceinline__ void mfma_asm(v4f& c, const v8i& af, const v8i& bf, int sa, int sb) {
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
template <int OA, int NT>
__device__ __forceinline__ void mfma_tile(const v8i& af, const BFrag& b, v4f& c, int sa) {
  mfma_asm<OA, NT>(c, af, b.f[NT], sa, b.sc);
}

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
__device__ __forceinline__ void ld_b128(v4i& d, uint32_t voff, const v4i& rsrc, int soff) {
  asm volatile("buffer_load_dwordx4 %0, %1, %2, %3 offen" : "+v"(d) : "v"(voff), "s"(rsrc), "s"(soff) : "memory");
}
// One load into d1 if sel != 0, else into d0.  The choice is made inside the statement, so the
// compiler sees straight-line code that updates both variables in place (a branch of its own would
// end in copies of registers whose loads are still in flight).
__device__ __forceinline__ void ld2_b128(v4i& d0, v4i& d1, int sel, uint32_t voff, const v4i& rsrc, int soff) {
  asm volatile(
      "s_cmp_lg_u32 %5, 0\n\ts_cbranch_scc1 .Lmx%=_1\n\tbuffer_load_dwordx4 %0, %2, %3, %4 offen\n\ts_branch .Lmx%=_2\n"
      ".Lmx%=_1:\n\tbuffer_load_dwordx4 %1, %2, %3, %4 offen\n.Lmx%=_2:"
      : "+v"(d0), "+v"(d1) : "v"(voff), "s"(rsrc), "s"(soff), "s"(sel) : "memory", "scc");
}
__device__ __forceinline__ void ld2_b32(int& d0, int& d1, int sel, uint32_t voff, const v4i& rsrc, int soff) {
  asm volatile(
      "s_cmp_lg_u32 %5, 0\n\ts_cbranch_scc1 .Lmx%=_1\n\tbuffer_load_dword %0, %2, %3, %4 offen\n\ts_branch .Lmx%=_2\n"
      ".Lmx%=_1:\n\tbuffer_load_dword %1, %2, %3, %4 offen\n.Lmx%=_2:"
      : "+v"(d0), "+v"(d1) : "v"(voff), "s"(rsrc), "s"(soff), "s"(sel) : "memory", "scc");
}
__device__ __forceinline__ void st_b64(const v2i& d, uint32_t voff, const v4i& rsrc, int soff) {
  asm volatile("buffer_store_dwordx2 %0, %1, %2, %3 offen" : : "v"(d), "v"(voff), "s"(rsrc), "s"(soff) : "memory");
}
// 16 bytes per lane straight into LDS at lds + 16 * lane (no destination registers).
__device__ __forceinline__ void ld_lds_b128(uint32_t lds, uint32_t voff, const v4i& rsrc, int soff) {
  asm volatile("s_mov_b32 m0, %0\n\tbuffer_load_dwordx4 %1, %2, %3 offen lds"
               : : "s"(lds), "v"(voff), "s"(rsrc), "s"(soff) : "memory", "m0");
}
__device__ __forceinline__ void ld_b32(int& d, uint32_t voff, const v4i& rsrc, int soff) {
  asm volatile("buffer_load_dword %0, %1, %2, %3 offen" : "+v"(d) : "v"(voff), "s"(rsrc), "s"(soff) : "memory");
}

// NMT = number of 16-row tiles this instantiation multiplies (the chunk has at most NMT*16 rows).
// Keeping it a compile-time constant keeps the K loop free of branches around the MFMAs.
template <int STAGE, int NMT>
__device__ __forceinline__ void mx_gemm_body(const MxArgs& a, uint8_t* smem, int* s_tok, float* s_aff, int nrows, int e,
                                             int64_t slot0, int xt) {
  uint8_t* sA = smem;
  uint8_t* sS = smem + MX_NST * MX_SA;

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
  {
    int id = -1;
    if (tid < nrows) {
      id = a.tp2id[slot0 + tid];
      if (id < 0 || id >= a.n_real) id = -1;
    }
    s_tok[tid] = id;
    if (STAGE == 2) {
      float af = 0.f;
      if (id >= 0 && a.aff)
        af = (a.aff_dtype == MOE_DT_BF16) ? bf16_bits_to_f32(((const uint16_t*)a.aff)[(int64_t)id * a.E + e])
                                          : ((const float*)a.aff)[(int64_t)id * a.E + e];
      s_aff[tid] = af;
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
  // A scales: thread covers row tid
  uint32_t as_voff;
  if (STAGE == 1) {
    const int tok = s_tok[tid];
    as_voff = ((tok >= 0) ? (uint32_t)tok : 0u) * (uint32_t)a.a_scale_stride;
  } else {
    as_voff = (uint32_t)(slot0 + ((tid < nrows) ? tid : (nrows - 1))) * (uint32_t)a.a_scale_stride;
  }

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
  if (STAGE == 1) {
    w_pstride = 2 * nH * a.I;
    w_tstride = a.I;
    colu = (int64_t)tI * 512 + (int64_t)q * Pt + p0;
    rw_ = make_rsrc(a.W + (int64_t)e * 128 * w_pstride, (uint32_t)(128 * w_pstride * 4));
    rs_ = make_rsrc(a.W_scale + (int64_t)e * 16 * w_pstride, (uint32_t)(16 * w_pstride));
    w_voff = (uint32_t)((4 * g * w_pstride + hcol * nH * a.I + 4 * cl) * 4);
    s_voff = (uint32_t)(g * w_pstride + hcol * nH * a.I + 4 * cl);
  } else {
    w_pstride = (int64_t)a.nI * a.H;
    w_tstride = a.H;
    colu = h0 + 64 * q;
    const int64_t sp = (a.pI + 7) / 8;
    rw_ = make_rsrc(a.W + (int64_t)e * a.pI * w_pstride, (uint32_t)(a.pI * w_pstride * 4));
    rs_ = make_rsrc(a.W_scale + (int64_t)e * sp * w_pstride, (uint32_t)(sp * w_pstride));
    w_voff = (uint32_t)((4 * g * w_pstride + 4 * c) * 4);
    s_voff = (uint32_t)(g * w_pstride + 4 * c);
  }

  // A K slice's loads, numbered so that they can be issued a few at a time:
  //   0 .. NAJ-1            activation rows (16 bytes per lane each)
  //   NAJ                   activation scales
  //   NAJ+1 .. NAJ+NBL      weights
  //   NAJ+NBL+1 ..          weight scales
  constexpr int NBL = 8;
  constexpr int NBS = 1;
  constexpr int NLOADS = NAJ + 1 + NBL + NBS;
  struct BRaw {
    v4i d[NBL];
    int sc;
  };
  struct AStage {
    int sc;
  };
  const v4i ra_ = make_rsrc(a.A, 0xffffffffu), ras_ = make_rsrc(a.A_scale, 0xffffffffu);
  // Scalar byte offset of a weight load = (offset of its row and column within the slice, fixed per
  // load and kept in scalar registers) + (offset of the slice, computed once per slice): one scalar
  // add per load.  Address arithmetic done per load costs more issue cycles than the MFMAs between
  // two loads take.
  int w_soff[NBL], s_soff[NBS];
#pragma unroll
  for (int i = 0; i < NBL; ++i) {
    const int pr = (i < 4) ? i : (16 + i - 4);
    w_soff[i] = uni(((int64_t)pr * w_pstride + colu) * 4);
  }
#pragma unroll
  for (int i = 0; i < NBS; ++i) s_soff[i] = uni(colu);
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
    r.lds_a = uni((int)(lds_ring + (uint32_t)st * MX_SA));
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
    r.w_off = uni(((int64_t)(pb * 32) * w_pstride + (int64_t)kt * w_tstride) * 4);
    r.s_off = uni((int64_t)(pb * 4) * w_pstride + (int64_t)kt * w_tstride);
    return r;
  };
  auto issue_load = [&](auto idx_, const SliceAddr& sa, AStage& as, BRaw& b, BRaw& b1, int sel) {
    constexpr int idx = decltype(idx_)::value;
    if constexpr (idx < NAJ) {
      // the wave's 64 lanes fill 8 rows x 128 bytes = 1 KB of the ring stage, in lane order
      ld_lds_b128(sa.lds_a + (uint32_t)((w * 8 + 32 * idx) * MXROW), a_voff[idx], sa.ra, sa.a_off);
    } else if constexpr (idx == NAJ) {
      ld_b32(as.sc, as_voff, sa.ras, sa.as_off);
    } else if constexpr (idx < NAJ + 1 + NBL) {
      constexpr int i = idx - NAJ - 1;
      ld2_b128(b.d[i], b1.d[i], sel, w_voff, sa.rw, w_soff[i] + sa.w_off);
    } else {
      ld2_b32(b.sc, b1.sc, sel, s_voff, sa.rs, s_soff[0] + sa.s_off);
    }
  };
  constexpr int NLA = NAJ + 1;        // activation loads come first in the numbering and in issue order
  constexpr int NLB = NLOADS - NLA;   // weight loads of a slice
  auto issue_a = [&](int ks, int st, AStage& as, BRaw& b0, BRaw& b1) {
    const SliceAddr sa = slice_addr(ks, st);
    static_for<0, NLA>([&](auto i_) { issue_load(i_, sa, as, b0, b1, 0); });
  };
  auto issue_b = [&](int ks, AStage& as, BRaw& b0, BRaw& b1, int sel) {
    const SliceAddr sa = slice_addr(ks, 0);
    static_for<NLA, NLOADS>([&](auto i_) { issue_load(i_, sa, as, b0, b1, sel); });
  };
  // Waits until at most N of this wave's loads are outstanding (they complete in issue order), and
  // ties the registers that the oldest of them fill to that point.
  // (The wait itself names no register: an in/out operand may be copied into place before the
  // statement, i.e. read while its load is still in flight.)
  auto wait_a = [&](auto n_, AStage& as) {
    constexpr int N = decltype(n_)::value;
    asm volatile("s_waitcnt vmcnt(%0)" : : "n"(MX_DBG_WAIT0 ? 0 : N) : "memory");
    asm volatile("" : "+v"(as.sc));
  };
  // `m1` (all ones or zero, uniform) picks set b1 or b0: one select per register does the choice
  // and the transposition together, with no branch (a branch ends in a block of copies per path).
  auto pick = [&](int& d, int x0, int x1, uint64_t m1) {
    asm volatile("v_cndmask_b32 %0, %1, %2, %3" : "=v"(d) : "v"(x0), "v"(x1), "s"(m1));
  };
  auto unpack_b = [&](const BRaw& b0, const BRaw& b1, uint64_t m1, BFrag& f) {
    int t[4][8];
#pragma unroll
    for (int i = 0; i < NBL; ++i)
#pragma unroll
      for (int x = 0; x < 4; ++x) pick(t[x][i], b0.d[i][x], b1.d[i][x], m1);
#pragma unroll
    for (int nt = 0; nt < 4; ++nt)
#pragma unroll
      for (int r = 0; r < 8; ++r) f.f[nt][r] = t[nt][r];
    pick(f.sc, b0.sc, b1.sc, m1);
    asm volatile("s_nop 1");  // the selects feed the first MFMA
  };
  auto store_a = [&](int st, const AStage& r) {
    const uint32_t asreg = (uint32_t)r.sc;
    // scales transposed: row = mt*16 + cc -> [gg][cc][mt]
    uint8_t* sd = sS + st * MX_SS;
    const int mt = tid >> 4, cc = tid & 15;
#pragma unroll
    for (int gg = 0; gg < 4; ++gg) sd[(gg * 16 + cc) * 16 + mt] = (uint8_t)((asreg >> (8 * gg)) & 0xffu);
  };

  v4f acc[NMT][4];
  static_for<0, NMT>([&](auto mt) {
#pragma unroll
    for (int nt = 0; nt < 4; ++nt) acc[mt][nt] = (v4f){0.f, 0.f, 0.f, 0.f};
  });

  // One K slice: row tiles are multiplied in groups of two; the fragments of the next group are
  // read from LDS while the current group's eight MFMAs run.  The groups of the first half are each
  // followed by a share of the loads of slice ks+2.
  const int rd_lo = c * MXROW + ((g ^ (c & 7)) * 16), rd_hi = c * MXROW + (((g + 4) ^ (c & 7)) * 16);
  constexpr int NG = NMT / 2;
  constexpr int NB_AFTER_A = NLB;  // weight loads issued after the last activation load of a slice
  auto compute = [&](int st, BFrag& b, int ks, int ph, AStage& as, BRaw& b0, BRaw& b1) {
    const uint8_t* plo = sA + st * MX_SA + rd_lo;
    const uint8_t* phi = sA + st * MX_SA + rd_hi;
    const v4i asc = *(const v4i*)(sS + st * MX_SS + (g * 16 + c) * 16);
    // first fragments of this slice: in flight while the weights are transposed
    v8i af[2][2];
    af[0][0] = frag_from_lds(plo, phi);
    af[0][1] = frag_from_lds(plo + 16 * MXROW, phi + 16 * MXROW);
    asm volatile("" ::: "memory");
    asm volatile("s_waitcnt vmcnt(%0)" : : "n"(MX_DBG_WAIT0 ? 0 : NLOADS) : "memory");
    unpack_b(b0, b1, ph ? ~0ull : 0ull, b);
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
      // Eight MFMAs; after each one, its share of the loads of slice ks+2 (activations first: they
      // must have arrived by the end of this slice; the weights have until the top of slice ks+2 and
      // go to the raw set that was transposed at the top of this slice).  One or two loads fit in
      // the 32 cycles an MFMA occupies the matrix pipe; a burst of them does not.
      static_for<0, 8>([&](auto j_) {
        constexpr int j = decltype(j_)::value;
        constexpr int mt = 2 * gi + j / 4, nt = j % 4;
        constexpr int m = gi * 8 + j;  // MFMA number within the slice
        mfma_tile<mt % 4, nt>(af[cur][j / 4], b, acc[mt][nt], asc[mt / 4]);
        if constexpr (m == 0) {
          // the scalar arithmetic for the addresses of slice ks+2 starts here, behind the first
          // MFMA, instead of ahead of it
          int ks2 = ks + 2;
          asm volatile("" : "+s"(ks2));
          sad = slice_addr(ks2, (st == 0) ? 2 : st - 1);
        }
        static_for<m * NLOADS / (8 * NG), (m + 1) * NLOADS / (8 * NG)>(
            [&](auto i_) { issue_load(i_, sad, as, b0, b1, ph); });
      });
    });
  };

  // ---- main loop ------------------------------------------------------------------------------------
  // Slice ks multiplies out of ring stage ks % 3 with the weights in `bc`, transposed at its top
  // from raw set ks % 2.  During its first half the loads of slice ks+2 are issued: the weights
  // refill that raw set, the activations fill the staging registers, which go to ring stage
  // (ks+2) % 3 at the end of the slice (that stage was last read in slice ks-1, which every wave
  // left before the barrier that ended it).  One barrier per slice publishes the stores.  The MFMA
  // code exists once; only the few instructions that touch a raw set are selected by the parity of
  // ks (two copies of the MFMA sequence do not survive register allocation).
  BRaw br0, br1;
  AStage as;
  BFrag bc;
  static_for<0, NBL>([&](auto j_) {
    constexpr int j = decltype(j_)::value;
    br0.d[j] = 0;
    br1.d[j] = 0;
  });
  br0.sc = br1.sc = 0;
  as.sc = 0;
  issue_b(0, as, br0, br1, 0);
  issue_b(1, as, br0, br1, 1);
  // both leading slices in one round trip
  AStage as1;
  as1.sc = 0;
  issue_a(0, 0, as, br0, br1);
  issue_a(1, 1, as1, br0, br1);
  wait_a(std::integral_constant<int, 0>{}, as);
  wait_a(std::integral_constant<int, 0>{}, as1);
  store_a(0, as);
  store_a(1, as1);
  __syncthreads();
  int st = 0;
#pragma clang loop unroll(disable)
  for (int ks = 0; ks < nks; ++ks) {
    const int ph = ks & 1;
    // weights of this slice: requested two slices ago; everything issued since is one slice's loads
    compute(st, bc, ks, ph, as, br0, br1);
    const int st2 = (st == 0) ? 2 : st - 1;  // (st + 2) % 3
    // activations of slice ks+2: requested in this slice, NB_AFTER_A weight loads ago
    wait_a(std::integral_constant<int, NB_AFTER_A>{}, as);
    store_a(st2, as);  // past the end: zeros into a stage that nobody reads any more
    __syncthreads();
    st = (st == 2) ? 0 : st + 1;
  }
  // the last MFMAs are still in the pipe: as instructions of unknown kind to the compiler, it adds
  // no wait between them and the first read of an accumulator
  asm volatile("s_waitcnt vmcnt(0)\n\ts_nop 15\n\ts_nop 15" ::: "memory");

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
          // (the accumulators are taken out of their registers here, tile by tile, not all at once
          // ahead of the passes)
          asm volatile("" : "+a"(acc[mt][0]), "+a"(acc[mt][1]), "+a"(acc[mt][2]), "+a"(acc[mt][3]));
          float y[2][4];
#pragma unroll
          for (int t = 0; t < 4; ++t) {
#pragma unroll
            for (int k = 0; k < 2; ++k) {
              const float mine = hcol ? acc[mt][t][2 + k] : acc[mt][t][k];
              const float send = hcol ? acc[mt][t][k] : acc[mt][t][2 + k];
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
    static_for<0, NMT>([&](auto mt_) {
      constexpr int mt = decltype(mt_)::value;
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int row = mt * 16 + 4 * g + r;
        const float af = post ? s_aff[row] : 1.f;
        v2i o;
#pragma unroll
        for (int t = 0; t < 4; t += 2) {
          const v2f d = {(acc[mt][t][r] + bd[t]) * af, (acc[mt][t + 1][r] + bd[t + 1]) * af};
          o[t >> 1] = __builtin_bit_cast(int, __builtin_convertvector(d, v2bf));
        }
        st_b64(o, d_voff, rd, (mt * 16 + r) * rowb);
      }
    });
  }
}

template <int STAGE>
__global__ __launch_bounds__(MXT) __attribute__((amdgpu_waves_per_eu(1, 1))) void mx_gemm_kernel(const MxArgs a) {
  extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
  __shared__ int s_tok[MXM];
  __shared__ float s_aff[MXM];
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
  if (nrows <= 64) mx_gemm_body<STAGE, 4>(a, smem, s_tok, s_aff, nrows, e, slot0, xt);
  else if (nrows <= 128) mx_gemm_body<STAGE, 8>(a, smem, s_tok, s_aff, nrows, e, slot0, xt);
  else mx_gemm_body<STAGE, 16>(a, smem, s_tok, s_aff, nrows, e, slot0, xt);
}

int launch_mx_gemm(int stage, const MxArgs& m0, unsigned gx, unsigned gy, hipStream_t s) {
  if (gx == 0 || gy == 0) return MOE_OK;
  MxArgs m = m0;
  m.col_tiles = (int32_t)gx;
  const unsigned grid = 8u * ((gy + 7u) / 8u) * gx;  // gy = upper bound on the number of chunks
  hipError_t err;
  if (stage == 1) {
    err = hipFuncSetAttribute((const void*)mx_gemm_kernel<1>, hipFuncAttributeMaxDynamicSharedMemorySize, MX_LDS);
    if (err != hipSuccess) return MOE_E_LAUNCH;
    hipLaunchKernelGGL(mx_gemm_kernel<1>, dim3(grid), dim3(MXT), MX_LDS, s, m);
  } else {
    err = hipFuncSetAttribute((const void*)mx_gemm_kernel<2>, hipFuncAttributeMaxDynamicSharedMemorySize, MX_LDS);
    if (err != hipSuccess) return MOE_E_LAUNCH;
    hipLaunchKernelGGL(mx_gemm_kernel<2>, dim3(grid), dim3(MXT), MX_LDS, s, m);
  }
  MOE_CHECK_LAUNCH();
  return MOE_OK;
}

}  // namespace moe
