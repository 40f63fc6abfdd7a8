/*
 * C ABI of libmoe_gfx950.so -- MI355X (gfx950) kernels for the MoE context-encoding
 * path of aws-neuron/nki-library.
 *
 * The reference has no FFI: its operator boundary is the pair of Python kernels
 *   moe_cte(...)               src/nkilib_src/nkilib/core/moe/moe_cte/moe_cte.py:252-277
 *   rmsnorm_quant_kernel(...)  src/nkilib_src/nkilib/core/rmsnorm/rmsnorm_quant.py:86-92
 * This header declares what a Python (ctypes) binding of those two functions
 * calls instead of the NKI device code.  All tensor pointers are DEVICE pointers;
 * `stream` is a hipStream_t passed as void* (NULL = default stream).  Every
 * function returns 0 on success or a negative MOE_E_* code; moe_error_string()
 * turns it into text.  Functions validate shapes before launching anything.
 * No function allocates device memory: scratch comes from the caller through
 * (workspace, workspace_bytes), sized by moe_blockwise_workspace_bytes().
 */
#ifndef MOE_GFX950_H
#define MOE_GFX950_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* ---- error codes ------------------------------------------------------------------- */
#define MOE_OK 0
#define MOE_E_BAD_ARG (-1)       /* null pointer, negative size, unknown enum value            */
#define MOE_E_BAD_SHAPE (-2)     /* shape violates a documented divisibility / range rule     */
#define MOE_E_WORKSPACE (-3)     /* workspace missing or smaller than *_workspace_bytes()     */
#define MOE_E_LAUNCH (-4)        /* hipLaunchKernel / hipMemsetAsync reported an error        */
#define MOE_E_UNSUPPORTED (-5)   /* valid in the reference, not built here                    */
#define MOE_E_NO_DEVICE (-6)     /* current device is not gfx950                              */
#define MOE_E_STATIC_LIMIT (-7)  /* size beyond the built-in scratch of an entry point that allocates nothing */

const char* moe_error_string(int code);
/* ABI version of this header; bumped on any signature change. */
int moe_abi_version(void);
/* 0 when the current HIP device is gfx950, MOE_E_NO_DEVICE otherwise.  Also the library's per-device set-up: it
 * looks up the address of that device's built-in scratch (moe_build_blocks_static), so call it once per device,
 * outside any stream capture, before recording calls of the library into a HIP graph. */
int moe_check_device(void);

/* ---- element types ----------------------------------------------------------------- */
#define MOE_DT_BF16 0
#define MOE_DT_FP16 1
#define MOE_DT_FP32 2
#define MOE_DT_FP8_E4M3 3 /* OCP e4m3fn bit patterns; Neuron float8_e4m3 is the |v|<=240 subset */
#define MOE_DT_FP8_E5M2 4 /* OCP e5m2 bit patterns (MXFP8 weights only)                              */
#define MOE_DT_FP4_E2M1 5 /* OCP e2m1 (MXFP4 weights only): four 4-bit values per 2-byte x4 element   */
#define MOE_DT_INT32 6    /* the index operators only                                                */

/* ---- RMSNorm + quantise front end -------------------------------------------------- */

/* Replaces rmsnorm_quant_kernel with QuantizationType.ROW
 * (rmsnorm_quant.py:86-171, _row_quantize_tile :526-620, store :342-403).
 * x [rows, H] (x_dtype bf16/fp16/fp32), gamma [H] (gamma_dtype) or NULL when do_norm == 0.
 * out: uint8 [rows, H+4]; bytes [0,H) are e4m3 codes of n/dq, bytes [H,H+4) the
 * little-endian fp32 dequant scale dq = max(amax/240, 1e-6).
 * n = x * (1/(sqrt(mean(x^2)) + eps)) * gamma  (the test golden's form,
 * test/integration/nkilib/core/rmsnorm/test_rmsnorm_quant.py:73-75).
 * lower_bound > 0 clips amax and n to +-lower_bound first.  H <= 16384. */
int moe_rmsnorm_quant_fp8_row(const void* x, int x_dtype, const void* gamma, int gamma_dtype, void* out,
                              int64_t rows, int64_t H, float eps, float lower_bound, int do_norm,
                              void* stream);

/* Replaces rmsnorm_quant_kernel with QuantizationType.STATIC (_static_quantize_tile,
 * rmsnorm_quant.py:623-662).  input_dequant_scale: device fp32, element 0 is used
 * (the reference broadcasts one scalar to [128,1]).  out: uint8 [rows, H]
 * = e4m3(clip(n * (1/scale), +-240)). */
int moe_rmsnorm_quant_fp8_static(const void* x, int x_dtype, const void* gamma, int gamma_dtype,
                                 const float* input_dequant_scale, void* out, int64_t rows, int64_t H,
                                 float eps, int do_norm, void* stream);

/* Output layouts of moe_rmsnorm_quant_mxfp8 */
#define MOE_MX_LAYOUT_TOKEN_MAJOR 0 /* q [rows, H] bytes in k' order, scale [rows, H/32]                     */
#define MOE_MX_LAYOUT_REF_DENSE 1   /* q x4 [128, H/512, rows], scale [16, H/512, rows]                      */
#define MOE_MX_LAYOUT_REF_STRIDED 2 /* as 1 but scale [128, H/512, rows], row (s/4)*32 + s%4 holds scale s   */

/* Replaces rmsnorm_mx_quantize_tkg (src/nkilib_src/nkilib/core/subkernels/rmsnorm_mx_quantize_tkg.py:29-40;
 * golden test/integration/nkilib/core/subkernels/test_rmsnorm_mx_quantize_tkg.py:100-137) and the online
 * activation quantisation of the MX MoE kernel (moe_cte_mx_utils.py:730-771).
 * n = bf16(x * (1/sqrt(sum(x^2)/hidden_actual + eps)) * gamma) when do_norm, else bf16(x);
 * then MXFP8-e4m3 with one E8M0 scale per 32 consecutive k', k' = tile*512 + p*4 + q for
 * h = q*(H/4) + tile*128 + p.  H % 512 == 0, H <= 16384.
 * out_norm (nullable): bf16 [128, rows, H/128], element [p, t, h1] = n[t, h1*128 + p].
 * residual / out_residual (both or neither; [rows, H] of x's type): the fused residual add of
 * rmsnorm_mx_quantize_tkg.py:29-40,214-232 (golden test_rmsnorm_mx_quantize_tkg.py:104-117):
 * hidden = x + residual rounded to x's type is what is normalised and quantised, and it is written to
 * out_residual.  (The reference's hidden_dim_tp=False has no kernel behind it there either:
 * "Only hidden_dim_tp=True is supported", norm_tkg_utils.py:467.) */
int moe_rmsnorm_quant_mxfp8(const void* x, int x_dtype, const void* residual, void* out_residual, const void* gamma,
                            int gamma_dtype, void* out_q, void* out_scale, void* out_norm, int64_t rows, int64_t H,
                            float eps, int64_t hidden_actual, int do_norm, int layout, void* stream);

/* ---- router top-k front end ----------------------------------------------------------- */

/* Replaces router_topk (src/nkilib_src/nkilib/core/router_topk/router_topk.py:55-75; semantics
 * router_topk_torch_ref, src/nkilib_src/nkilib/core/router_topk/router_topk_torch.py:23-135).
 * x bf16 [T, H] (the x_hbm_layout == 1 form), w bf16 [H, E], w_bias [E] (bias_dtype) or NULL.
 * logits = x @ w + bias in fp32; expert_index int32 [T, k] = the k largest logits per token in
 * descending order, ties to the lower expert index (NULL to skip the store, like
 * skip_store_expert_index); router_logits [T, E] (bf16 / fp32, NULL = skip_store_router_logits).
 * act_fn: 0 sigmoid, 1 softmax (RouterActFnType).  router_pre_norm != 0: activation over all E
 * experts; with norm_topk_prob the selected values divided by their sum, zero elsewhere; without
 * it the full activation (mask_to_topk != 0 zeroes the unselected experts -- the masked table
 * moe_cte consumes; not a reference option).  router_pre_norm == 0: activation over the k selected
 * logits only, scattered into zeros.  expert_affinities [T (+1 if pad_row), E] bf16 / fp32; with
 * pad_row row T (the padding token of moe_cte) is zeroed.  topk_affinities fp32 [T, k] or NULL
 * (return_eager_affi).  k <= 8, E <= 512, H % 64 == 0.  workspace: moe_router_topk_workspace_bytes. */
size_t moe_router_topk_workspace_bytes(int64_t H, int64_t E);
int moe_router_topk(const void* x, const void* w, const void* w_bias, int bias_dtype, int64_t T, int64_t H,
                    int64_t E, int k, int act_fn, int router_pre_norm, int norm_topk_prob, int mask_to_topk,
                    int pad_row, void* router_logits, int logits_dtype, int32_t* expert_index,
                    void* expert_affinities, int aff_dtype, float* topk_affinities, void* workspace,
                    size_t workspace_bytes, void* stream);

/* ---- token -> block index construction ---------------------------------------------- */

/* Device version of generate_token_position_to_id_and_experts
 * (test/integration/nkilib/core/moe/moe_cte/test_moe_cte_common.py:199-264), bit exact.
 * topk_ids int32 [T, k] (distinct expert ids per row; ids outside [0,E) are ignored).
 * Writes token_position_to_id int32[N*B], block_to_expert int32[N], conditions int32[n_conditions]
 * (nullable; ones for the first N - n_padding_blocks entries... exactly: the trailing
 * n_padding_blocks + (n_conditions - N) entries are 0).  pad id = T, or -1 when skip_token.
 * E <= 1024.  workspace: >= moe_build_blocks_workspace_bytes(E) bytes.  Returns MOE_E_BAD_SHAPE through
 * *status_out (device int32, nullable) == 1 when N is too small for the routing. */
size_t moe_build_blocks_workspace_bytes(int64_t E);
int moe_build_blocks(const int32_t* topk_ids, int64_t T, int64_t k, int64_t E, int64_t B, int64_t N,
                     int skip_token, int use_split_padding, int32_t* token_position_to_id,
                     int32_t* block_to_expert, int32_t* conditions, int64_t n_conditions,
                     void* workspace, size_t workspace_bytes, int32_t* status_out, void* stream);

/* moe_build_blocks that also hands the blockwise layer its bookkeeping.  No counterpart in the reference (whose
 * kernels walk the blocks of token_position_to_id as they are, bwmm_shard_on_block_mx.py:972-1347): moe_blockwise
 * otherwise derives, from token_position_to_id and block_to_expert, the valid rows of every block, every token's
 * list of slots and the expert chunks and work queues of its GEMM launches, in four small launches that read every
 * slot twice; the block build knows all of that while it sorts.  Same arguments and the same three tables, bit for
 * bit, as moe_build_blocks, plus `plan`: device memory of at least moe_block_plan_bytes(T, B, N, skip_token) bytes,
 * 256-byte aligned, which this call fills (one more single-workgroup launch) and which moe_bwmm_args.block_plan
 * passes to moe_blockwise.  A plan describes exactly the tables written by the same call: pass it only together
 * with those token_position_to_id / block_to_expert buffers, unchanged, with the same B, N and token count
 * (T1 = T + 1, or T with skip_token), and with `conditions` either NULL or the array this call wrote.
 * T >= 1, T * k <= N * B and E <= 512 (MOE_E_BAD_SHAPE otherwise: use moe_build_blocks); use_split_padding
 * returns MOE_E_UNSUPPORTED (which blocks run then depends on whether `conditions` is passed on). */
size_t moe_block_plan_bytes(int64_t T, int64_t B, int64_t N, int skip_token);
int moe_build_blocks_plan(const int32_t* topk_ids, int64_t T, int64_t k, int64_t E, int64_t B, int64_t N,
                          int skip_token, int use_split_padding, int32_t* token_position_to_id,
                          int32_t* block_to_expert, int32_t* conditions, int64_t n_conditions, void* workspace,
                          size_t workspace_bytes, int32_t* status_out, void* plan, size_t plan_bytes, void* stream);

/* moe_build_blocks for callers that cannot allocate or pass device scratch memory (code under HIP graph capture,
 * tight serving loops, harnesses that forbid hipMalloc).  No counterpart in the reference.  Same arguments and
 * the same results, bit for bit, as moe_build_blocks minus (workspace, workspace_bytes): the first slots and
 * per-slab counts live in a device array built into the library, MOE_BUILD_BLOCKS_STATIC_BYTES per GPU for the
 * life of the process.  Calls no hipMalloc / hipFree or any other allocating routine.  E above
 * MOE_BUILD_BLOCKS_STATIC_MAX_E returns MOE_E_STATIC_LIMIT (use moe_build_blocks with a workspace instead).  The
 * array's address is looked up once per device, with that device current (the device of `stream` must be current
 * in every call): by moe_check_device(), else by the first call of this entry point there.  That lookup is not
 * guaranteed to be legal while a stream is being captured: before recording this call into a HIP graph on a device,
 * call moe_check_device() or make one call outside the capture there.  All calls
 * on one GPU share that GPU's array: calls that overlap on one GPU (different streams, or threads) race; calls in
 * stream order do not.  Nothing in the array has to be cleared between calls. */
#define MOE_BUILD_BLOCKS_STATIC_MAX_E 512
#define MOE_BUILD_BLOCKS_STATIC_BYTES (((1 + 64) * MOE_BUILD_BLOCKS_STATIC_MAX_E + 4) * 4) /* 133 136 bytes */
int moe_build_blocks_static(const int32_t* topk_ids, int64_t T, int64_t k, int64_t E, int64_t B, int64_t N,
                            int skip_token, int use_split_padding, int32_t* token_position_to_id,
                            int32_t* block_to_expert, int32_t* conditions, int64_t n_conditions,
                            int32_t* status_out, void* stream);

/* The reference's device-side pieces of the same construction, as separate operators
 * (mask [T, E] -> per-expert token lists -> block offsets -> flat token_position_to_id).
 *
 * moe_find_nonzero_indices replaces find_nonzero_indices
 * (src/nkilib_src/nkilib/core/subkernels/find_nonzero_indices.py:34-110; semantics
 * find_nonzero_indices_torch_ref, find_nonzero_indices_torch.py:20-63), bit exact.  input [T, C_full]
 * (MOE_DT_INT32 / FP32 / BF16 / FP16); columns col_start_id[0] .. + n_cols (col_start_id: device
 * int32[1], NULL = column 0; columns outside the input count as all zero).  indices int32
 * [n_cols, T]: per column the ascending row numbers of its nonzero elements, then -1;
 * nonzero_counts int32 [n_cols].
 *
 * moe_indexed_flatten replaces indexed_flatten (src/nkilib_src/nkilib/core/subkernels/
 * indexed_flatten.py:28-86; semantics indexed_flatten_torch_ref, indexed_flatten_torch.py:18-66).
 * input int32 [E, T] seen as [E, T / f_len, f_len]; block p of row e goes to output block
 * row_offsets[start + e] + p when that lies in [0, output_len / f_len) (start =
 * row_offsets_start[0], device int32[1], NULL = 0); where rows overlap the later row wins (the
 * reference's loop order); everything else is padding_val.  output int32 [output_len].
 *
 * moe_cumsum replaces cumsum (src/nkilib_src/nkilib/core/cumsum/cumsum.py:30-75; cumsum_torch.py:20-32):
 * inclusive prefix sum along the last axis of [rows, H]; fp32 accumulation for BF16 / FP16 / FP32
 * (result rounded to the element type), exact for MOE_DT_INT32. */
size_t moe_find_nonzero_indices_workspace_bytes(int64_t T, int64_t n_cols);
int moe_find_nonzero_indices(const void* input, int dtype, int64_t T, int64_t C_full, const int32_t* col_start_id,
                             int64_t n_cols, int32_t* indices, int32_t* nonzero_counts, void* workspace,
                             size_t workspace_bytes, void* stream);
int moe_indexed_flatten(const int32_t* input, int64_t E, int64_t T, int64_t f_len, int64_t output_len,
                        const int32_t* row_offsets, int64_t n_offsets, const int32_t* row_offsets_start,
                        int32_t padding_val, int32_t* output, void* stream);
int moe_cumsum(const void* x, void* y, int dtype, int64_t rows, int64_t H, void* stream);

/* ---- blockwise MoE ------------------------------------------------------------------- */

#define MOE_KIND_BF16 0    /* bf16 activations, bf16 weights or fp8 weights + per-channel fp32 scales */
#define MOE_KIND_FP8_ROW 1 /* fp8 activations with per-row scale ([T1, H+4] records), fp8 weights      */
#define MOE_KIND_MXFP8 2   /* MXFP8 weights (reference x4 layouts), activations quantised to MXFP8     */

/* ActFnType values, src/nkilib_src/nkilib/core/utils/common_types.py:32-36 */
#define MOE_ACT_SILU 0
#define MOE_ACT_GELU 1
#define MOE_ACT_GELU_TANH 2
#define MOE_ACT_SWISH 3
/* ExpertAffinityScaleMode values, common_types.py:48-52 */
#define MOE_SCALE_NONE 0
#define MOE_SCALE_POST 1
#define MOE_SCALE_PRE 2
#define MOE_SCALE_PRE_DELAYED 3

#define MOE_CLAMP_GATE_HI 1
#define MOE_CLAMP_GATE_LO 2
#define MOE_CLAMP_UP_HI 4
#define MOE_CLAMP_UP_LO 8

typedef struct moe_bwmm_args {
  /* -- tensors, named as the arguments of moe_cte (moe_cte.py:253-277) ------------------
   * hidden_states:
   *   BF16 kind     bf16 [T1, H]
   *   FP8_ROW kind  uint8 [T1, H+4]: rmsnorm_quant ROW records (codes + fp32 scale)
   *   MXFP8 kind    bf16 [T1, H] (quantised online, hidden_states_scale == NULL), or
   *                 uint8 [T1, H] e4m3 codes in k' order with hidden_states_scale uint8 [T1, H/32]
   * T1 = T+1 (row T is the all-zero padding token) or T when skip_token. */
  const void* hidden_states;
  const void* hidden_states_scale;
  const void* expert_affinities_masked; /* [T1*E], affinity_dtype (bf16 or fp32), row-major [T1, E] */
  /* BF16: [E,H,2,I] weight_dtype (bf16 | fp8);  FP8_ROW: uint8 [E,H,2,I];
   * MXFP8: uint8 [E,128,2,H/512,I,4] (x4: byte q of element i)                              */
  const void* gate_up_proj_weight;
  /* BF16: [E,I_pad,H];  FP8_ROW: uint8 [E,I_pad,H];  MXFP8: uint8 [E,p_I,ceil(I/512),H,4]    */
  const void* down_proj_weight;
  /* BF16/FP8_ROW: fp32 [E or 1, 1, 2I] / [E or 1, 1, H] (NULL = unquantised bf16 weights);
   * MXFP8: uint8 [E,16,2,H/512,I] / [E,ceil(p_I/8),ceil(I/512),H]                            */
  const void* gate_up_proj_scale;
  const void* down_proj_scale;
  /* bias_dtype; BF16/FP8_ROW: [E,2,I], [E,H];  MXFP8: [E,p_I,2,ceil(I/512),4], [E,H]; nullable */
  const void* gate_and_up_proj_bias;
  const void* down_proj_bias;
  const int32_t* token_position_to_id; /* [N*B] */
  const int32_t* block_to_expert;      /* [N]   */
  const int32_t* conditions;           /* nullable, [n_conditions]; blocks from the first 0 on are skipped */
  void* output;                        /* bf16; row t at output + t*out_row_stride elements, T1 rows written */
  void* workspace;
  size_t workspace_bytes;
  /* -- sizes --------------------------------------------------------------------------- */
  int64_t T1, H, I, E, B, N;
  int64_t I_pad;          /* rows of down_proj_weight per expert (BF16 / FP8_ROW); 0 = I          */
  int64_t n_conditions;   /* entries readable in conditions                                       */
  int64_t out_row_stride; /* in elements; H for [T1,H], 2H for slot 0 of [T1,2,H]                 */
  int32_t scale_experts;  /* leading dim of the fp32 scales: E or 1 (BF16 / FP8_ROW)              */
  /* -- options ------------------------------------------------------------------------- */
  int32_t kind;           /* MOE_KIND_*                                                           */
  int32_t weight_dtype;   /* BF16 kind: MOE_DT_BF16 or MOE_DT_FP8_E4M3; MXFP8 kind: MOE_DT_FP8_E4M3 (also
                           * taken for MOE_DT_BF16, the zero value), MOE_DT_FP8_E5M2 or MOE_DT_FP4_E2M1:
                           * nl.float8_e4m3fn_x4 / float8_e5m2_x4 / float4_e2m1fn_x4 in the reference; 4-bit
                           * weights have the same shapes with 2-byte elements                              */
  int32_t affinity_dtype; /* MOE_DT_BF16 or MOE_DT_FP32                                           */
  int32_t bias_dtype;     /* MOE_DT_BF16 or MOE_DT_FP32                                           */
  int32_t act_fn;         /* MOE_ACT_*                                                            */
  int32_t scaling_mode;   /* MOE_SCALE_*                                                          */
  int32_t skip_token;     /* 1: padding id is -1 and tables have T rows                           */
  int32_t clamp_mask;     /* MOE_CLAMP_* bits                                                     */
  float gate_clamp_upper, gate_clamp_lower, up_clamp_upper, up_clamp_lower;
  /* Activation checkpoints of the bf16 kind (checkpoint_activation, bwmm_shard_on_I.py:160-176;
   * golden test_moe_cte_common.py:312-314,404-405,420-421), both bf16 and nullable:
   * gate_up_activations_T [N, 2, I, B] = gate / up projections after scale, bias and clamp, before the
   * activation; down_activations [N, B, H] = down projection after scale and bias, before the affinity.
   * All B rows of every executed block are written (padding rows hold what a zero input row gives),
   * blocks that conditions stops are zero. */
  void* gate_up_activations_T;
  void* down_activations;
  /* Optional K-contiguous copies of the bf16 / fp8 weights of the BF16 and FP8_ROW kinds, made once by
   * moe_prepare_kmajor_weights (they depend on the weights only).  Both NULL: every call makes its own copies
   * in the workspace.  (What a copy holds depends on the kind, the weight type and the shape only -- for bf16
   * weights with H % 256 == 0 and I % 128 == 0, and fp8-row weights with H % 512 == 0 and I % 128 == 0, the order
   * the large-tile kernels read, otherwise K-contiguous rows -- so one pair serves every call with those weights;
   * a bf16 call on such a shape that asks for activation checkpoints runs the general kernel and makes its own
   * K-contiguous copies regardless.)  MXFP8 kind: the x4 layouts are K-major already and are read in place when both are NULL;
   * on shapes with H % 512 == 0 and I % 128 == 0 the same two calls make a copy of the gate/up weights in the
   * order the kernel reads them (each workgroup then reads its weights as contiguous 32 KB runs: the gate/up GEMM
   * is 5 % faster at H = 7168, I = 2048 with 8-bit weights, for a second copy of those weights in memory); used
   * when gate_up_proj_weight_kmajor is set.  A copy of the down weights exists for 4-bit weights only
   * (moe_kmajor_weights_bytes(args, 1) is 0 otherwise and the pointer is ignored). */
  const void* gate_up_proj_weight_kmajor;
  const void* down_proj_weight_kmajor;
  /* Nullable.  The reference's two-shard kernels return [T1, 2, H] or [2, T1, H] with the sum in shard 0 and
   * zeros in shard 1 (output_shape, moe_cte.py:333-346).  When set, row t of that second plane lies at
   * output_shard1 + t*out_row_stride elements and the combine pass writes it as zeros along with row t of
   * `output`, so the caller needs no separate clear. */
  void* output_shard1;
  /* Nullable, no counterpart in the reference: device int64 [4].  Workgroup 0 of the large-tile gate/up GEMM writes
   * [0] = shader clock cycles and [1] = ticks of the constant 100 MHz counter between its first and last
   * instruction, the down GEMM the same into [2], [3]: cycles / ticks x 0.1 is the shader clock in GHz that the
   * part held under that launch (it is set by power management, not by the data sheet).  Read by bench.py. */
  int64_t* gemm_clocks;
  /* Nullable, no counterpart in the reference: the bookkeeping that moe_build_blocks_plan wrote for exactly these
   * token_position_to_id / block_to_expert tables (see there for the conditions under which it may be passed).
   * With it moe_blockwise launches no bookkeeping kernels of its own.  Ignored when activation checkpoints are
   * requested (their chunks cover whole blocks).  The plan is read only; it may be passed to any number of calls. */
  const void* block_plan;
  size_t block_plan_bytes;
  /* Nullable, no counterpart in the reference: seven hipEvent_t of the caller's (null entries are skipped).  The
   * call records them on `stream`: [0] on entry, [1] after the bookkeeping, [2] ahead of the gate/up stage (after
   * the online activation quantisation and any per-call weight copies), [3] after the gate/up GEMM, [4] after the
   * fp8-row re-quantisation, [5] after the down GEMM, [6] after the combine.  Lets a benchmark time the stages of one
   * ordinary call instead of calling moe_blockwise_stages once per stage.  Read by bench.py. */
  void* const* stage_events;
} moe_bwmm_args;

/* Replaces bwmm_shard_on_block / blockwise_mm_baseline_shard_intermediate* /
 * bwmm_shard_on_block_mx (moe_cte.py:348-489): for every block b before the first
 * conditions[b]==0, rows x = hidden[token_position_to_id[b*B..]], expert e = block_to_expert[b]:
 * out[token] += bf16( down(act(gate(x)) * up(x)) * affinity[token*E+e] ), accumulated per
 * token in block order in bf16, exactly as the golden does
 * (test/integration/nkilib/core/moe/moe_cte/test_moe_cte_common.py:267-447).
 * Rows of `output` not reached by any block are set to zero. */
size_t moe_blockwise_workspace_bytes(const moe_bwmm_args* args);
int moe_blockwise(const moe_bwmm_args* args, void* stream);

/* The same pipeline, one stage (or any subset, always in pipeline order) per call, so that a
 * caller can bracket individual kernels with its own events.  moe_blockwise(args, s) ==
 * moe_blockwise_stages(args, MOE_STAGE_ALL, s).  Stages communicate through `workspace`, which
 * must be the same buffer for all calls of one pass.  No counterpart in the reference (its
 * stages are fused into one traced kernel); used by bench.py for per-kernel timing. */
#define MOE_STAGE_PREP 1u      /* block bookkeeping: active blocks, valid rows, token -> slot lists */
#define MOE_STAGE_ACT_QUANT 2u /* MXFP8 kind with bf16 hidden_states: online activation quantisation */
#define MOE_STAGE_GATE_UP 4u   /* gate/up GEMM + act(gate)*up (+ MXFP8 re-quantisation)              */
#define MOE_STAGE_REQUANT 8u   /* FP8_ROW kind: per-row re-quantisation of the intermediate          */
#define MOE_STAGE_DOWN 16u     /* down GEMM + bias + affinity                                        */
#define MOE_STAGE_COMBINE 32u  /* per-token accumulation of the contributions into the output        */
#define MOE_STAGE_ALL 63u
int moe_blockwise_stages(const moe_bwmm_args* args, unsigned stages, void* stream);

/* No counterpart in the reference, whose dense weights are consumed N-contiguous ([E, H, 2, I], [E, I_pad, H]):
 * the MFMA operands of the BF16 and FP8_ROW kinds are read along K, so the GEMMs run on K-contiguous copies
 * ([E, 2, I, Hk] and [E, H, Ik]; bf16 for the BF16 kind, fp8 weights widened; fp8 for FP8_ROW; tails zero).
 * A caller whose weights do not change (inference) makes the copies once and passes them in
 * moe_bwmm_args.*_kmajor.  moe_kmajor_weights_bytes: bytes of the gate/up (which == 0) or down (which == 1)
 * copy for these args, 0 if the kind has none.  moe_prepare_kmajor_weights fills both (256-byte aligned). */
size_t moe_kmajor_weights_bytes(const moe_bwmm_args* args, int which);
int moe_prepare_kmajor_weights(const moe_bwmm_args* args, void* gate_up_kmajor, void* down_kmajor, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* MOE_GFX950_H */
