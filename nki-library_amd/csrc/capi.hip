// C ABI entry points of libmoe_gfx950.so that are not tied to one kernel file: error text,
// device check, workspace planning and the blockwise-MoE driver.
#include <string.h>

#include "bwmm.hpp"

using namespace moe;

extern "C" int moe_rmsnorm_quant_mxfp8(const void*, int, const void*, void*, const void*, int, void*, void*, void*, int64_t,
                                       int64_t, float, int64_t, int, int, void*);

extern "C" const char* moe_error_string(int code) {
  switch (code) {
    case MOE_OK: return "ok";
    case MOE_E_BAD_ARG: return "bad argument (null pointer, negative size or unknown enum value)";
    case MOE_E_BAD_SHAPE: return "shape violates a divisibility or range rule of this kernel";
    case MOE_E_WORKSPACE: return "workspace missing or too small";
    case MOE_E_LAUNCH: return "HIP launch failed";
    case MOE_E_UNSUPPORTED: return "option not supported by the gfx950 implementation";
    case MOE_E_NO_DEVICE: return "current HIP device is not gfx950";
    case MOE_E_STATIC_LIMIT:
      return "size exceeds the built-in scratch of this entry point (it allocates nothing): use the variant that takes a workspace";
    default: return "unknown error code";
  }
}

extern "C" int moe_abi_version(void) { return 7; }

extern "C" int moe_check_device(void) {
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess) return MOE_E_NO_DEVICE;
  hipDeviceProp_t prop;
  if (hipGetDeviceProperties(&prop, dev) != hipSuccess) return MOE_E_NO_DEVICE;
  if (strncmp(prop.gcnArchName, "gfx950", 6) != 0) return MOE_E_NO_DEVICE;
  return moe::build_blocks_static_setup();  // per-device set-up of the entry point that allocates nothing
}

namespace {

inline size_t al256(size_t v) { return (v + 255) & ~(size_t)255; }

struct Plan {
  size_t book, xq, xs, y, yq, ys, d, wt1, wt2, total;
  int64_t Hk;      // BF16 / FP8_ROW: H padded to the K step, row length (elements) of the transposed gate/up weights
  int64_t Iw;      // padded intermediate width (elements) of the stage-2 A operand
  int64_t pI, nI;  // MXFP8
};

int validate(const moe_bwmm_args* a) {
  if (!a || !a->hidden_states || !a->gate_up_proj_weight || !a->down_proj_weight || !a->token_position_to_id ||
      !a->block_to_expert || !a->output)
    return MOE_E_BAD_ARG;
  if (a->T1 <= 0 || a->H <= 0 || a->I <= 0 || a->E <= 0 || a->B <= 0 || a->N <= 0) return MOE_E_BAD_ARG;
  if (a->kind < MOE_KIND_BF16 || a->kind > MOE_KIND_MXFP8) return MOE_E_BAD_ARG;
  if (a->act_fn < MOE_ACT_SILU || a->act_fn > MOE_ACT_SWISH) return MOE_E_BAD_ARG;
  if (a->scaling_mode < MOE_SCALE_NONE || a->scaling_mode > MOE_SCALE_PRE_DELAYED) return MOE_E_BAD_ARG;
  if (a->scaling_mode != MOE_SCALE_NONE && !a->expert_affinities_masked) return MOE_E_BAD_ARG;
  if (a->affinity_dtype != MOE_DT_BF16 && a->affinity_dtype != MOE_DT_FP32) return MOE_E_BAD_ARG;
  if ((a->gate_and_up_proj_bias || a->down_proj_bias) && a->bias_dtype != MOE_DT_BF16 && a->bias_dtype != MOE_DT_FP32)
    return MOE_E_BAD_ARG;
  if (a->conditions && a->n_conditions <= 0) return MOE_E_BAD_ARG;
  if (a->out_row_stride < a->H) return MOE_E_BAD_SHAPE;
  if (a->E > COMBINE_MAX_K) return MOE_E_UNSUPPORTED;
  if (a->N * a->B >= ((int64_t)1 << 31) || a->T1 * a->E >= ((int64_t)1 << 31)) return MOE_E_BAD_SHAPE;
  const int64_t Ipad = a->I_pad > 0 ? a->I_pad : a->I;
  if (Ipad < a->I) return MOE_E_BAD_SHAPE;
  if ((a->gate_up_activations_T || a->down_activations) && a->kind != MOE_KIND_BF16) return MOE_E_UNSUPPORTED;
  switch (a->kind) {
    case MOE_KIND_BF16:
      if (a->H % 8 != 0) return MOE_E_BAD_SHAPE;  // 16-byte row slices of bf16 hidden states
      if (a->weight_dtype != MOE_DT_BF16 && a->weight_dtype != MOE_DT_FP8_E4M3) return MOE_E_BAD_ARG;
      if (a->weight_dtype == MOE_DT_FP8_E4M3 && (!a->gate_up_proj_scale || !a->down_proj_scale)) return MOE_E_BAD_ARG;
      if ((a->gate_up_proj_scale != nullptr) != (a->down_proj_scale != nullptr)) return MOE_E_BAD_ARG;
      if (a->gate_up_proj_scale && a->scale_experts != 1 && a->scale_experts != a->E) return MOE_E_BAD_SHAPE;
      break;
    case MOE_KIND_FP8_ROW:
      if (a->H % 16 != 0 || a->I % 4 != 0) return MOE_E_BAD_SHAPE;
      if (!a->gate_up_proj_scale || !a->down_proj_scale) return MOE_E_BAD_ARG;
      if (a->scale_experts != 1 && a->scale_experts != a->E) return MOE_E_BAD_SHAPE;
      break;
    case MOE_KIND_MXFP8: {
      // bwmm_shard_on_block_mx.py:586-633, moe_cte_mx_utils.py:260-264
      if (a->H % 512 != 0 || a->H < 512 || a->H > 16384) return MOE_E_BAD_SHAPE;
      const int64_t tail = a->I % 512;
      if (a->I % 16 != 0 || (tail != 0 && tail % 32 != 0)) return MOE_E_BAD_SHAPE;
      if (!a->gate_up_proj_scale || !a->down_proj_scale) return MOE_E_BAD_ARG;
      // POST_SCALE only (test_moe_bwmm_mx_cte.py:163-167)
      if (a->scaling_mode == MOE_SCALE_PRE || a->scaling_mode == MOE_SCALE_PRE_DELAYED) return MOE_E_UNSUPPORTED;
      // weight element formats: e4m3 (also for the zero value, MOE_DT_BF16), e5m2, e2m1
      if (a->weight_dtype != MOE_DT_FP8_E4M3 && a->weight_dtype != MOE_DT_BF16 && a->weight_dtype != MOE_DT_FP8_E5M2 &&
          a->weight_dtype != MOE_DT_FP4_E2M1)
        return MOE_E_BAD_ARG;
      break;
    }
  }
  // Address ranges.  The kernels form per-lane offsets in 32 bits; a shape whose tensors outgrow what those
  // offsets reach would read wrong rows without any error, so it is refused here (the reference states its
  // own size limits the same way, bwmm_shard_on_block_mx.py:586-633).
  const int64_t slots = a->N * a->B;
  if (a->kind == MOE_KIND_MXFP8 && mx_fast_path_ok(a->H, a->I)) {
    // large-tile kernels: byte offsets (row * row stride, added to a 64-bit base) and buffer descriptors of at most
    // 2^32 - 1 bytes for the activations, the intermediate and their scales; signed 32-bit byte offsets inside one
    // expert's weights
    const int64_t lim32 = (int64_t)1 << 32, lim31 = (int64_t)1 << 31;
    const int64_t Iw = (a->I + 511) / 512 * 512;
    const int64_t es = a->weight_dtype == MOE_DT_FP4_E2M1 ? 2 : 4;  // bytes of an x4 weight element
    const int64_t pI = a->I > 512 ? 128 : a->I / 4, nI = (a->I + 511) / 512;
    if (a->T1 * a->H >= lim32 || slots * Iw >= lim32) return MOE_E_BAD_SHAPE;
    if (128 * 2 * (a->H / 512) * a->I * es >= lim31 || pI * nI * a->H * es >= lim31) return MOE_E_BAD_SHAPE;
    // the row tables (token ids, affinities, bias) are fetched through 32-bit byte offsets as well
    if (slots * 4 >= lim32 || a->T1 * a->E * 4 >= lim32 || a->E * pI * 2 * nI * 4 * 4 >= lim32 ||
        a->E * a->H * 4 >= lim32)
      return MOE_E_BAD_SHAPE;
  } else if (a->kind != MOE_KIND_MXFP8) {
    // general tiled kernel, dense kinds: row offsets are kept in units of 4 bytes in 32 bits (the value ~0 is
    // reserved for "no such row"), i.e. each A operand must stay below 2^34 - 4 bytes = 16 GiB
    const int64_t lim34 = ((int64_t)1 << 34) - 4;
    const int64_t a1 = a->kind == MOE_KIND_BF16 ? a->H * 2 : a->H + 4;
    const int64_t a2 = a->kind == MOE_KIND_BF16 ? (a->I + 63) / 64 * 64 * 2 : (a->I + 127) / 128 * 128;
    if (a->T1 * a1 >= lim34 || slots * a2 >= lim34) return MOE_E_BAD_SHAPE;
  }
  return MOE_OK;
}

// The dense kinds on the large-tile kernels (bwmm_mx.hip).  Two separate questions:
//   *_shape:     is the expert shape (kind, weight type, H, I, E) one of those kernels', with every 32-bit offset they
//                form inside one expert's weights and tables in range?  This alone decides what a KEPT weight copy
//                holds (x4 read order, or K-contiguous rows for the general kernel): a copy prepared in one call must
//                mean the same in every other call with the same weights, whatever its token count.
//   *_call_fits: do this call's activations (token count, number of blocks) fit the kernels' 32-bit row offsets?
// A call runs there when both hold (activation checkpoints of the bf16 kind included: those epilogues write them).
// A call on such a shape that cannot run there uses the general kernel on K-contiguous copies of its own, made per
// call in the workspace: kept copies are in the other order and are ignored (*_kept_usable).
bool row8_shape(const moe_bwmm_args* a) {
  if (a->kind != MOE_KIND_FP8_ROW || !mx_fast_path_ok(a->H, a->I)) return false;
  const int64_t lim32 = (int64_t)1 << 32, lim31 = (int64_t)1 << 31;
  const int64_t pI = a->I > 512 ? 128 : a->I / 4, nI = (a->I + 511) / 512;
  if (2 * a->H * a->I >= lim31 || pI * nI * a->H * 4 >= lim31) return false;
  if (a->E * 2 * a->I * 4 >= lim32 || a->E * a->H * 4 >= lim32) return false;
  return true;
}
bool row8_call_fits(const moe_bwmm_args* a) {
  const int64_t lim32 = (int64_t)1 << 32;
  const int64_t slots = a->N * a->B, Iw = (a->I + 127) / 128 * 128;
  return a->T1 * (a->H + 4) < lim32 && slots * Iw < lim32 && slots * 4 < lim32 && a->T1 * a->E * 4 < lim32;
}
bool row8_fast(const moe_bwmm_args* a) { return row8_shape(a) && row8_call_fits(a); }
bool row8_kept_usable(const moe_bwmm_args* a) { return row8_fast(a) || !row8_shape(a); }
// (bf16 weights, or fp8 weights widened to bf16 in the copy; K extents in bytes: 2H, 2I)
bool bf16_fast_shape(const moe_bwmm_args* a) {
  if (a->kind != MOE_KIND_BF16 || (a->weight_dtype != MOE_DT_BF16 && a->weight_dtype != MOE_DT_FP8_E4M3)) return false;
  if (a->H % 256 != 0 || a->I % 128 != 0) return false;
  const int64_t lim32 = (int64_t)1 << 32, lim31 = (int64_t)1 << 31;
  const int64_t Ib = 2 * a->I, Hb = 2 * a->H;
  const int64_t pI = Ib > 512 ? 128 : Ib / 4, nI = (Ib + 511) / 512;
  if (2 * Hb * a->I >= lim31 || pI * nI * a->H * 4 >= lim31) return false;
  if (a->E * 2 * a->I * 4 >= lim32 || a->E * a->H * 4 >= lim32) return false;
  return true;
}
bool bf16_call_fits(const moe_bwmm_args* a) {
  const int64_t lim32 = (int64_t)1 << 32;
  const int64_t slots = a->N * a->B;
  return a->T1 * 2 * a->H < lim32 && slots * 2 * a->I < lim32 && slots * 4 < lim32 && a->T1 * a->E * 4 < lim32;
}
bool bf16_fast(const moe_bwmm_args* a) { return bf16_fast_shape(a) && bf16_call_fits(a); }
bool bf16_kept_usable(const moe_bwmm_args* a) { return bf16_fast(a) || !bf16_fast_shape(a); }
// What a kept copy of the fp8-row (bf16) weights holds on that path: the weights in x4 order, one expert's worth of
// E8M0 block scales of 127 (2^0) that serves every expert, and one row of activation block scales of 127 (the bf16
// kernels fetch the tables like the others and ignore what they hold).  K extents in bytes: H, I for fp8, twice
// that for bf16.
struct Row8Copy {
  size_t w_scale, a_scale, a_scale_bytes, total;
};
Row8Copy row8_copy(const moe_bwmm_args* a, int which) {
  auto al = [](size_t v) { return (v + 255) & ~(size_t)255; };
  const size_t es = a->kind == MOE_KIND_BF16 ? 2 : 1;
  const size_t Hb = (size_t)a->H * es, Ib = (size_t)a->I * es;
  const size_t nH = Hb / 512, nI = (Ib + 511) / 512, pI = Ib > 512 ? 128 : Ib / 4;
  Row8Copy c;
  const size_t w = which == 0 ? (size_t)a->E * 2 * Hb * a->I : (size_t)a->E * pI * nI * a->H * 4;
  const size_t ws = which == 0 ? 16 * 2 * nH * (size_t)a->I : ((pI + 7) / 8) * nI * (size_t)a->H;
  c.w_scale = al(w);
  c.a_scale = c.w_scale + al(ws);
  c.a_scale_bytes = al(which == 0 ? Hb / 32 : nI * 16);
  c.total = c.a_scale + c.a_scale_bytes;
  return c;
}

Plan make_plan(const moe_bwmm_args* a) {
  Plan p;
  memset(&p, 0, sizeof(p));
  const size_t slots = (size_t)(a->N * a->B);
  size_t off = 0;
  p.book = off; off += al256(bookkeeping_bytes(a->T1, a->N, a->B));
  if (a->kind == MOE_KIND_MXFP8) {
    p.nI = (a->I + 511) / 512;
    p.pI = a->I > 512 ? 128 : a->I / 4;
    p.Iw = p.nI * 512;
    if (!a->hidden_states_scale) {
      p.xq = off; off += al256((size_t)a->T1 * a->H);
      p.xs = off; off += al256((size_t)a->T1 * (a->H / 32));
    }
    p.yq = off; off += al256(slots * (size_t)p.Iw);
    p.ys = off; off += al256(slots * (size_t)(p.Iw / 32));
  } else if (a->kind == MOE_KIND_BF16) {
    p.Iw = (a->I + 63) / 64 * 64;
    p.y = off; off += al256(slots * (size_t)p.Iw * 2);
    // K-contiguous bf16 copies of the weights: [E, 2, I, Hk] and [E, H, Iw]
    p.Hk = (a->H + 63) / 64 * 64;
    const bool bf = bf16_fast(a);
    if (bf) {  // the x4 geometry of the down weights over 2I bytes of K
      p.nI = (2 * a->I + 511) / 512;
      p.pI = 2 * a->I > 512 ? 128 : a->I / 2;
    }
    const bool kept = bf16_kept_usable(a);
    if (!(a->gate_up_proj_weight_kmajor && kept)) {
      p.wt1 = off; off += al256(bf ? row8_copy(a, 0).total : (size_t)a->E * 2 * a->I * p.Hk * 2);
    }
    if (!(a->down_proj_weight_kmajor && kept)) {
      p.wt2 = off; off += al256(bf ? row8_copy(a, 1).total : (size_t)a->E * a->H * p.Iw * 2);
    }
  } else {
    p.Iw = (a->I + 127) / 128 * 128;
    p.y = off; off += al256(slots * (size_t)a->I * 4);
    p.yq = off; off += al256(slots * (size_t)p.Iw);
    p.ys = off; off += al256(slots * 4);
    // K-contiguous copies of the fp8 weights: [E, 2, I, Hk] and [E, H, Iw]
    p.Hk = (a->H + 127) / 128 * 128;
    const bool r8 = row8_fast(a);
    if (r8) {  // the x4 geometry of the down weights, as for the MXFP8 kind
      p.nI = (a->I + 511) / 512;
      p.pI = a->I > 512 ? 128 : a->I / 4;
    }
    const bool kept = row8_kept_usable(a);
    if (!(a->gate_up_proj_weight_kmajor && kept)) {
      p.wt1 = off; off += al256(r8 ? row8_copy(a, 0).total : (size_t)a->E * 2 * a->I * p.Hk);
    }
    if (!(a->down_proj_weight_kmajor && kept)) {
      p.wt2 = off; off += al256(r8 ? row8_copy(a, 1).total : (size_t)a->E * a->H * p.Iw);
    }
  }
  p.d = off; off += al256(slots * (size_t)a->H * 2);
  p.total = off;
  return p;
}

// Copy of the gate/up (which == 0) or down (which == 1) weights of the BF16 / FP8_ROW kinds: in the large-tile
// kernels' x4 read order (x4), else K-contiguous rows for the general kernel.
int kmajor_copy(const moe_bwmm_args* a, const Plan& p, int which, void* dst, hipStream_t s, bool x4) {
  const int64_t Ipad = a->I_pad > 0 ? a->I_pad : a->I;
  if (x4 && a->kind == MOE_KIND_BF16) {
    const Row8Copy c = row8_copy(a, which);
    int rc = launch_relayout_x4_bf16(a->gate_up_proj_weight, a->down_proj_weight, a->weight_dtype == MOE_DT_FP8_E4M3,
                                     (uint8_t*)dst, which, a->E, a->H, a->I, Ipad, s);
    if (rc != MOE_OK) return rc;
    return launch_fill_bytes((uint8_t*)dst + c.w_scale, c.total - c.w_scale, 127, s);
  }
  if (a->kind == MOE_KIND_BF16) {
    const int w8 = a->weight_dtype == MOE_DT_FP8_E4M3;
    if (which == 0)
      return launch_transpose_w16(a->gate_up_proj_weight, w8, (uint16_t*)dst, a->H, a->I, 2 * a->I, p.Hk, a->E, 2,
                                  a->H * 2 * a->I, a->I, s);
    return launch_transpose_w16(a->down_proj_weight, w8, (uint16_t*)dst, a->I, a->H, a->H, p.Iw, a->E, 1, Ipad * a->H, 0, s);
  }
  if (x4) {
    const Row8Copy c = row8_copy(a, which);
    int rc = launch_relayout_x4((const uint8_t*)a->gate_up_proj_weight, (const uint8_t*)a->down_proj_weight,
                                (uint8_t*)dst, which, a->E, a->H, a->I, Ipad, s);
    if (rc != MOE_OK) return rc;
    return launch_fill_bytes((uint8_t*)dst + c.w_scale, c.total - c.w_scale, 127, s);
  }
  if (which == 0)
    return launch_transpose_fp8((const uint8_t*)a->gate_up_proj_weight, (uint8_t*)dst, a->H, a->I, 2 * a->I, p.Hk, a->E, 2,
                                a->H * 2 * a->I, a->I, s);
  return launch_transpose_fp8((const uint8_t*)a->down_proj_weight, (uint8_t*)dst, a->I, a->H, a->H, p.Iw, a->E, 1,
                              Ipad * a->H, 0, s);
}

}  // namespace

// MXFP8 kind: copies of the weights in the kernels' read order exist on the large-tile path: of the gate/up weights
// for every format, of the down weights for 4-bit ones (whose pieces in the reference layout are 512 bytes; the
// 8-bit ones' 1 KB pieces were measured no slower than a copy).
static bool mx_packable(const moe_bwmm_args* a, int which) {
  if (a->kind != MOE_KIND_MXFP8 || !mx_fast_path_ok(a->H, a->I)) return false;
  return which == 0 || a->weight_dtype == MOE_DT_FP4_E2M1;
}

extern "C" size_t moe_kmajor_weights_bytes(const moe_bwmm_args* a, int which) {
  if (validate(a) != MOE_OK || which < 0 || which > 1) return 0;
  if (a->kind == MOE_KIND_MXFP8)
    return mx_packable(a, which) ? mx_packed_weights_bytes(which + 1, a->weight_dtype == MOE_DT_FP4_E2M1, a->E, a->H, a->I)
                                 : 0;
  const Plan p = make_plan(a);
  const size_t es = a->kind == MOE_KIND_BF16 ? 2 : 1;
  if (row8_shape(a) || bf16_fast_shape(a)) return row8_copy(a, which).total;
  return which == 0 ? (size_t)a->E * 2 * a->I * p.Hk * es : (size_t)a->E * a->H * p.Iw * es;
}

extern "C" int moe_prepare_kmajor_weights(const moe_bwmm_args* a, void* gate_up_kmajor, void* down_kmajor, void* stream) {
  int rc = validate(a);
  if (rc != MOE_OK) return rc;
  if (a->kind == MOE_KIND_MXFP8) {  // down_kmajor is used where moe_kmajor_weights_bytes(a, 1) is not 0
    if (!mx_packable(a, 0)) return MOE_E_UNSUPPORTED;
    const int fp4 = a->weight_dtype == MOE_DT_FP4_E2M1;
    if (!gate_up_kmajor || (((uintptr_t)gate_up_kmajor) & 255) != 0) return MOE_E_BAD_ARG;
    rc = launch_mx_pack_weights(1, fp4, a->gate_up_proj_weight, gate_up_kmajor, a->E, a->H, a->I, (hipStream_t)stream);
    if (rc != MOE_OK || !mx_packable(a, 1)) return rc;
    if (!down_kmajor || (((uintptr_t)down_kmajor) & 255) != 0) return MOE_E_BAD_ARG;
    return launch_mx_pack_weights(2, fp4, a->down_proj_weight, down_kmajor, a->E, a->H, a->I, (hipStream_t)stream);
  }
  if (!gate_up_kmajor || !down_kmajor) return MOE_E_BAD_ARG;
  if ((((uintptr_t)gate_up_kmajor) & 255) != 0 || (((uintptr_t)down_kmajor) & 255) != 0) return MOE_E_BAD_ARG;
  const Plan p = make_plan(a);
  const bool x4 = row8_shape(a) || bf16_fast_shape(a);  // from the expert shape alone, see row8_shape
  rc = kmajor_copy(a, p, 0, gate_up_kmajor, (hipStream_t)stream, x4);
  if (rc != MOE_OK) return rc;
  return kmajor_copy(a, p, 1, down_kmajor, (hipStream_t)stream, x4);
}

extern "C" size_t moe_blockwise_workspace_bytes(const moe_bwmm_args* a) {
  if (validate(a) != MOE_OK) return 0;
  return make_plan(a).total;
}

extern "C" int moe_blockwise(const moe_bwmm_args* a, void* stream) {
  return moe_blockwise_stages(a, MOE_STAGE_ALL, stream);
}

extern "C" int moe_blockwise_stages(const moe_bwmm_args* a, unsigned stages, void* stream) {
  int rc = validate(a);
  if (rc != MOE_OK) return rc;
  const Plan p = make_plan(a);
  if (!a->workspace || a->workspace_bytes < p.total) return MOE_E_WORKSPACE;
  if (((uintptr_t)a->workspace & 255) != 0) return MOE_E_BAD_ARG;
  hipStream_t s = (hipStream_t)stream;
  uint8_t* ws = (uint8_t*)a->workspace;
  const int64_t n_real = a->skip_token ? a->T1 : a->T1 - 1;
  // The chunk / slot bookkeeping: derived here from token_position_to_id, or taken as the block build left it
  // (moe_build_blocks_plan).  Activation checkpoints cover whole blocks, which a plan's chunks do not: the plan is
  // then left aside.
  // (measurement hook: HIP events of the caller's, recorded on the stream between the stages)
  auto mark = [&](int i) {
    if (a->stage_events && a->stage_events[i]) (void)hipEventRecord((hipEvent_t)a->stage_events[i], s);
  };
  mark(0);
  const bool planned = a->block_plan != nullptr && !a->gate_up_activations_T && !a->down_activations;
  if (planned && (a->block_plan_bytes < bookkeeping_bytes(a->T1, a->N, a->B) || ((uintptr_t)a->block_plan & 255) != 0))
    return MOE_E_BAD_ARG;
  const Bookkeeping bk = carve_bookkeeping(planned ? (void*)a->block_plan : (void*)(ws + p.book), a->T1, a->N, a->B);
  if ((stages & MOE_STAGE_PREP) && !planned) {
    rc = launch_prep(bk, a, n_real, s);
    if (rc != MOE_OK) return rc;
  }
  mark(1);

  GemmArgs g;
  memset(&g, 0, sizeof(g));
  g.aff = a->scaling_mode == MOE_SCALE_NONE ? nullptr : a->expert_affinities_masked;
  g.aff_dtype = a->affinity_dtype;
  g.bias_dtype = a->bias_dtype;
  g.tp2id = a->token_position_to_id;
  g.b2e = a->block_to_expert;
  g.n_active = bk.n_active;
  g.valid_rows = bk.valid_rows;
  g.T1 = a->T1; g.H = a->H; g.I = a->I; g.E = a->E; g.B = a->B; g.N = a->N;
  g.I_pad = a->I_pad > 0 ? a->I_pad : a->I;
  g.n_real = n_real;
  g.tiles_per_block = (int32_t)((a->B + 127) / 128);
  g.weight_dtype = a->weight_dtype;
  g.act_fn = a->act_fn;
  g.scaling_mode = a->scaling_mode;
  g.clamp_mask = a->clamp_mask;
  g.clamp[0] = a->gate_clamp_upper; g.clamp[1] = a->gate_clamp_lower;
  g.clamp[2] = a->up_clamp_upper; g.clamp[3] = a->up_clamp_lower;
  g.w_scale_experts = a->scale_experts;
  g.pI = (int32_t)p.pI; g.nI = (int32_t)p.nI;
  const unsigned gy = (unsigned)(a->N * g.tiles_per_block);

  GemmArgs g1 = g, g2 = g;
  g1.W = (const uint8_t*)a->gate_up_proj_weight;
  g1.W_scale = (const uint8_t*)a->gate_up_proj_scale;
  g1.bias = a->gate_and_up_proj_bias;
  g2.W = (const uint8_t*)a->down_proj_weight;
  g2.W_scale = (const uint8_t*)a->down_proj_scale;
  g2.bias = a->down_proj_bias;
  g2.out = ws + p.d;
  g1.ckpt = (uint16_t*)a->gate_up_activations_T;
  g2.ckpt = (uint16_t*)a->down_activations;
  unsigned gx1, gx2 = (unsigned)((a->H + 127) / 128);

  if (a->kind == MOE_KIND_MXFP8) {
    const uint8_t* xq = (const uint8_t*)a->hidden_states;
    const uint8_t* xs = (const uint8_t*)a->hidden_states_scale;
    if (!xs) {
      // online activation quantisation (moe_cte_mx_utils.py:730-771): bf16 rows -> MXFP8 in k' order
      if (stages & MOE_STAGE_ACT_QUANT) {
        rc = moe_rmsnorm_quant_mxfp8(a->hidden_states, MOE_DT_BF16, nullptr, nullptr, nullptr, MOE_DT_BF16, ws + p.xq,
                                     ws + p.xs, nullptr, a->T1, a->H, 0.f, a->H, 0, MOE_MX_LAYOUT_TOKEN_MAJOR, stream);
        if (rc != MOE_OK) return rc;
      }
      xq = ws + p.xq;
      xs = ws + p.xs;
    }
    g1.A = xq; g1.a_stride = a->H; g1.A_scale = xs; g1.a_scale_stride = a->H / 32;
    g1.out = ws + p.yq; g1.out_stride = p.Iw; g1.out_scale = ws + p.ys; g1.out_scale_stride = p.Iw / 32;
    g2.A = ws + p.yq; g2.a_stride = p.Iw; g2.A_scale = ws + p.ys; g2.a_scale_stride = p.Iw / 32;
    gx1 = (unsigned)(p.nI * 4);
  } else if (a->kind == MOE_KIND_BF16) {
    g1.A = (const uint8_t*)a->hidden_states; g1.a_stride = a->H * 2; g1.K = a->H;
    g1.out = ws + p.y; g1.out_stride = p.Iw * 2;
    g2.A = ws + p.y; g2.a_stride = p.Iw * 2; g2.K = p.Iw;
    gx1 = (unsigned)((a->I + 127) / 128);
    // K-contiguous bf16 copies of the weights (fp8 weights are widened on the way), as for the fp8-row kind below
    const bool kept = bf16_kept_usable(a);
    const bool have1 = a->gate_up_proj_weight_kmajor && kept, have2 = a->down_proj_weight_kmajor && kept;
    g1.W = have1 ? (const uint8_t*)a->gate_up_proj_weight_kmajor : ws + p.wt1;
    g2.W = have2 ? (const uint8_t*)a->down_proj_weight_kmajor : ws + p.wt2;
    g1.Kp = p.Hk * 2;
    g2.Kp = p.Iw * 2;
    if ((stages & MOE_STAGE_GATE_UP) && !have1) {
      rc = kmajor_copy(a, p, 0, ws + p.wt1, s, bf16_fast(a));
      if (rc != MOE_OK) return rc;
    }
    if ((stages & MOE_STAGE_DOWN) && !have2) {
      rc = kmajor_copy(a, p, 1, ws + p.wt2, s, bf16_fast(a));
      if (rc != MOE_OK) return rc;
    }
  } else {
    g1.A = (const uint8_t*)a->hidden_states; g1.a_stride = a->H + 4; g1.K = a->H;
    g1.out = ws + p.y; g1.out_stride = a->I * 4;
    g2.A = ws + p.yq; g2.a_stride = p.Iw; g2.K = p.Iw; g2.A_scale = ws + p.ys;
    gx1 = (unsigned)((a->I + 127) / 128);
    // the reference stores the weights N-contiguous ([E, H, 2, I], [E, I_pad, H]); both MFMA operands are read
    // along K, so each stage first writes a K-contiguous copy of its weights
    const bool kept = row8_kept_usable(a);
    const bool have1 = a->gate_up_proj_weight_kmajor && kept, have2 = a->down_proj_weight_kmajor && kept;
    g1.W = have1 ? (const uint8_t*)a->gate_up_proj_weight_kmajor : ws + p.wt1;
    g2.W = have2 ? (const uint8_t*)a->down_proj_weight_kmajor : ws + p.wt2;
    g1.Kp = p.Hk;
    g2.Kp = p.Iw;
    if ((stages & MOE_STAGE_GATE_UP) && !have1) {
      rc = kmajor_copy(a, p, 0, ws + p.wt1, s, row8_fast(a));
      if (rc != MOE_OK) return rc;
    }
    if ((stages & MOE_STAGE_DOWN) && !have2) {
      rc = kmajor_copy(a, p, 1, ws + p.wt2, s, row8_fast(a));
      if (rc != MOE_OK) return rc;
    }
  }

  const bool bf_fast = bf16_fast(a);
  const bool r8_fast = row8_fast(a) || bf_fast;  // (what the two share: x4 copies with unit scale tables)
  const bool mx_fast = (a->kind == MOE_KIND_MXFP8 && mx_fast_path_ok(a->H, a->I)) || r8_fast;
  MxArgs m;
  memset(&m, 0, sizeof(m));
  if (mx_fast) {
    m.bias_dtype = a->bias_dtype;
    m.aff = g.aff;
    m.aff_dtype = a->affinity_dtype;
    m.tp2id = a->token_position_to_id;
    m.n_chunks = bk.n_chunks;
    m.chunk_slot = bk.chunk_slot;
    m.chunk_rows = bk.chunk_rows;
    m.chunk_expert = bk.chunk_expert;
    m.q_chunk = bk.q_chunk;
    m.q_off = bk.q_off;
    m.Yq = ws + p.yq;
    m.Ys = ws + p.ys;
    m.y_stride = p.Iw;
    m.ys_stride = p.Iw / 32;
    m.D = (uint16_t*)(ws + p.d);
    m.H = a->H; m.I = a->I; m.E = a->E; m.n_real = n_real;
    m.pI = (int32_t)p.pI; m.nI = (int32_t)p.nI;
    m.act_fn = a->act_fn; m.scaling_mode = a->scaling_mode; m.clamp_mask = a->clamp_mask;
    m.wfmt = (a->weight_dtype == MOE_DT_FP8_E5M2) ? MX_WFMT_E5M2 : (a->weight_dtype == MOE_DT_FP4_E2M1) ? MX_WFMT_E2M1 : MX_WFMT_E4M3;
    for (int i = 0; i < 4; ++i) m.clamp[i] = g.clamp[i];
    if (r8_fast) {
      m.wfmt = MX_WFMT_ROW8;
      m.cscale_experts = a->scale_experts;
      m.w_scale_shared = 1;
      m.Y32 = (float*)(ws + p.y);
      m.y32_stride = a->I;
    }
    if (bf_fast) {
      m.wfmt = MX_WFMT_BF16;
      m.Y32 = nullptr;
      m.Yq = ws + p.y;  // bf16 [N*B, Iw]
      m.y_stride = p.Iw;
    }
  }
  const unsigned gyc = (unsigned)bk.max_chunks;
  mark(2);
  // checkpoints of blocks that never run stay zero
  if (a->gate_up_activations_T && (stages & MOE_STAGE_GATE_UP)) {
    rc = launch_fill_zero_bytes(a->gate_up_activations_T, (size_t)a->N * 2 * a->I * a->B * 2, s);
    if (rc != MOE_OK) return rc;
  }
  if (a->down_activations && (stages & MOE_STAGE_DOWN)) {
    rc = launch_fill_zero_bytes(a->down_activations, (size_t)a->N * a->B * a->H * 2, s);
    if (rc != MOE_OK) return rc;
  }
  if (stages & MOE_STAGE_GATE_UP) {
    if (mx_fast) {
      MxArgs m1 = m;
      m1.A = g1.A; m1.a_stride = g1.a_stride; m1.A_scale = g1.A_scale; m1.a_scale_stride = g1.a_scale_stride;
      m1.a_rows = n_real;
      m1.W = (const uint32_t*)a->gate_up_proj_weight; m1.W_scale = (const uint8_t*)a->gate_up_proj_scale;
      m1.bias = a->gate_and_up_proj_bias;
      if (mx_packable(a, 0) && a->gate_up_proj_weight_kmajor) {
        m1.W = (const uint32_t*)a->gate_up_proj_weight_kmajor;
        m1.w_packed = 1;
      }
      if (r8_fast) {
        const Row8Copy c = row8_copy(a, 0);
        m1.W = (const uint32_t*)g1.W;  // the x4 copy (kept by the caller or made above)
        m1.W_scale = g1.W + c.w_scale;
        m1.A_scale = g1.W + c.a_scale; m1.a_scale_stride = 0; m1.a_scale_bytes = (int64_t)c.a_scale_bytes;
        m1.w_cscale = (const float*)a->gate_up_proj_scale;
      }
      if (bf_fast) {
        m1.H = 2 * a->H;  // K in bytes
        m1.ckpt = (uint16_t*)a->gate_up_activations_T;
        m1.ckpt_B = a->B; m1.ckpt_I = a->I;
      }
      m1.clk = a->gemm_clocks;

      // column tiles of 32 partitions x 4 q, gate and up: 4 per full intermediate tile + those of a short last one
      rc = launch_mx_gemm(1, m1, (unsigned)((a->I / 512) * 4 + (a->I % 512) / 128), gyc, s);
    } else {
      rc = launch_gemm_stage(a->kind, 1, g1, gx1, gy, s);
    }
    if (rc != MOE_OK) return rc;
  }
  mark(3);
  if (a->kind == MOE_KIND_FP8_ROW && (stages & MOE_STAGE_REQUANT)) {
    rc = launch_row_requant((const float*)(ws + p.y), ws + p.yq, (float*)(ws + p.ys), bk, a->N, a->B, a->I, p.Iw, s);
    if (rc != MOE_OK) return rc;
  }
  mark(4);
  if (stages & MOE_STAGE_DOWN) {
    if (mx_fast) {
      MxArgs m2 = m;
      m2.A = ws + p.yq; m2.a_stride = p.Iw; m2.A_scale = ws + p.ys; m2.a_scale_stride = p.Iw / 32;
      m2.a_rows = a->N * a->B;
      m2.W = (const uint32_t*)a->down_proj_weight; m2.W_scale = (const uint8_t*)a->down_proj_scale;
      m2.bias = a->down_proj_bias;
      if (mx_packable(a, 1) && a->down_proj_weight_kmajor) {
        m2.W = (const uint32_t*)a->down_proj_weight_kmajor;
        m2.w_packed = 1;
      }
      if (r8_fast) {
        const Row8Copy c = row8_copy(a, 1);
        m2.W = (const uint32_t*)g2.W;
        m2.W_scale = g2.W + c.w_scale;
        m2.A_scale = g2.W + c.a_scale; m2.a_scale_stride = 0; m2.a_scale_bytes = (int64_t)c.a_scale_bytes;
        m2.w_cscale = (const float*)a->down_proj_scale;
        m2.a_rscale = (const float*)(ws + p.ys);
      }
      if (bf_fast) {
        m2.A = ws + p.y; m2.a_stride = p.Iw * 2;
        m2.I = 2 * a->I;  // K in bytes
        m2.a_rscale = nullptr;
        m2.ckpt = (uint16_t*)a->down_activations;
        m2.ckpt_B = a->B; m2.ckpt_I = a->I;
      }
      m2.clk = a->gemm_clocks ? a->gemm_clocks + 2 : nullptr;

      rc = launch_mx_gemm(2, m2, (unsigned)(a->H / 256), gyc, s);
    } else {
      rc = launch_gemm_stage(a->kind, 2, g2, gx2, gy, s);
    }
    if (rc != MOE_OK) return rc;
  }
  mark(5);
  if (stages & MOE_STAGE_COMBINE) {
    rc = launch_combine(bk, a, ws + p.d, n_real, s);
    if (rc != MOE_OK) return rc;
  }
  mark(6);
  return MOE_OK;
}
