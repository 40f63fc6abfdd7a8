// Kernel argument block and launch entry points of the blockwise expert GEMMs.
#pragma once

#include "combine.hpp"

namespace moe {

struct GemmArgs {
  // A operand: stage 1 = hidden rows gathered by token id, stage 2 = intermediate rows by slot
  const uint8_t* A;
  int64_t a_stride;        // bytes between rows of A
  const uint8_t* A_scale;  // MXFP8: uint8 [rows, a_scale_stride]; FP8_ROW stage 2: float [slots]
  int64_t a_scale_stride;
  int64_t K;               // BF16 / FP8_ROW: contraction length in elements (zero padded on the A side)
  // B operand: expert weights in the reference layouts
  const uint8_t* W;
  const uint8_t* W_scale;  // MXFP8: uint8 E8M0; otherwise float per output channel (nullable)
  int32_t w_scale_experts;
  const void* bias;
  int32_t bias_dtype;
  const void* aff;
  int32_t aff_dtype;
  const int32_t* tp2id;
  const int32_t* b2e;
  const int32_t* n_active;
  const int32_t* valid_rows;
  // outputs
  void* out;               // stage 1: intermediate rows; stage 2: bf16 contributions [N*B, H]
  uint8_t* out_scale;      // MXFP8 stage 1: E8M0 scales of the intermediate
  int64_t out_stride;      // stage 1: bytes per intermediate row
  int64_t out_scale_stride;
  int64_t T1, H, I, E, B, N, I_pad, n_real;
  int32_t tiles_per_block;
  int32_t weight_dtype;
  int32_t act_fn, scaling_mode, clamp_mask;
  float clamp[4];          // gate hi, gate lo, up hi, up lo
  int32_t pI, nI;          // MXFP8: partitions per intermediate tile in the down weight, number of tiles
  int64_t Kp;              // BF16 / FP8_ROW: bytes per row of the transposed (K-contiguous) weights W points to
  uint16_t* ckpt;          // BF16 kind, nullable: stage 1 gate/up checkpoint [N, 2, I, B], stage 2 down checkpoint [N, B, H]
};

// Arguments of the large-tile MXFP8 kernels (bwmm_mx.hip).
struct MxArgs {
  const uint8_t* A;        // stage 1: MXFP8 activations [T1, H] in k' order; stage 2: intermediate [N*B, y_stride]
  int64_t a_stride;
  const uint8_t* A_scale;  // E8M0 [rows, a_scale_stride]
  int64_t a_scale_stride;
  int64_t a_rows;          // rows of A and A_scale
  const uint32_t* W;       // x4 weights in the reference layout (4-byte elements; 2-byte ones for 4-bit weights)
  const uint8_t* W_scale;
  const void* bias;
  int32_t bias_dtype;
  const void* aff;
  int32_t aff_dtype;
  const int32_t* tp2id;
  const int32_t* n_chunks;
  const int32_t* chunk_slot;
  const int32_t* chunk_rows;
  const int32_t* chunk_expert;
  const int32_t* q_chunk;  // work queues: two words per chunk, per XCD grouped by class, see Bookkeeping
  const int32_t* q_off;    // [8][CHUNK_CLASSES + 1], then the chunk interleave
  uint8_t* Yq;             // stage 1 output
  uint8_t* Ys;
  int64_t y_stride, ys_stride;
  uint16_t* D;             // stage 2 output, bf16 [N*B, H]
  int64_t H, I, E, n_real;
  int32_t pI, nI;
  int32_t act_fn, scaling_mode, clamp_mask;
  float clamp[4];
  int32_t col_tiles;       // column tiles per chunk (set by the launcher)
  int32_t wfmt;            // element format of the weights, MX_WFMT_*
  int32_t w_packed;        // 1: W is a copy of the weights in the kernel's read order (launch_mx_pack_weights)
  // MX_WFMT_ROW8 (the fp8-row kind on these kernels): e4m3 operands whose E8M0 tables are constants of 127, a
  // per-row fp32 scale of the activations and a per-output-channel fp32 scale of the weights in the epilogue
  const float* w_cscale;   // [cscale_experts][2*I] (gate/up: gate then up) or [cscale_experts][H] (down)
  int32_t cscale_experts;  // E or 1
  int32_t w_scale_shared;  // 1: W_scale holds one expert's worth of block scales that serves every expert
  const float* a_rscale;   // stage 2: row scale of the re-quantised intermediate, [N*B]; stage 1: null, a row's scale
                           // is the fp32 behind its H codes (the RMSNorm-Quant ROW record)
  int64_t a_scale_bytes;   // size of the A_scale table when it is not a_rows * a_scale_stride (stride 0: one row
                           // of constants for every row)
  float* Y32;              // stage 1 output of this format: fp32 [N*B, y32_stride], columns in natural order
  int64_t y32_stride;
  uint16_t* ckpt;          // MX_WFMT_BF16, nullable: stage 1 gate/up checkpoint [N, 2, I, B], stage 2 down checkpoint [N, B, H]
  int64_t ckpt_B, ckpt_I;  // block size and intermediate size of the checkpoint layout (elements)
  int64_t* clk;            // nullable: workgroup 0 stores its shader cycles and 100 MHz ticks from start to end here
  // MX_WFMT_BF16 (the bf16 kind on these kernels): both operands bf16, read as bytes exactly like the 8-bit formats
  // (a 128-byte K slice is 64 elements, multiplied by two v_mfma_f32_16x16x32_bf16 where the 8-bit formats issue
  // one 128-deep MFMA), so H (gate/up) and I (down) are the K extents in BYTES; no scales of any kind (w_cscale
  // may still carry per-channel scales of weights widened from fp8); gate/up writes bf16 [N*B, y_stride elements]
  // in natural column order through Yq.
};

constexpr int MX_WFMT_E4M3 = 0, MX_WFMT_E5M2 = 1, MX_WFMT_E2M1 = 2, MX_WFMT_ROW8 = 3, MX_WFMT_BF16 = 4;

// True when the large-tile kernels cover the shape: every intermediate tile holds a multiple
// of 32 partitions (I % 128 == 0); other shapes run the general kernel.
inline bool mx_fast_path_ok(int64_t H, int64_t I) { return H % 512 == 0 && I % 128 == 0; }
int launch_mx_gemm(int stage, const MxArgs& m, unsigned gx, unsigned gy, hipStream_t s);
// Copy of the x4 weights of one stage (1 gate/up, 2 down) in the order the large-tile kernel reads them: for expert
// e, column tile xt, K slice ks, wave q, load i, lane l the 16 bytes (4-bit weights: 8) that the lane's i-th load of
// that slice fetches, at ((((e * col_tiles + xt) * nks + ks) * 4 + q) * 8 + i) * 64 + l such pieces.
int launch_mx_pack_weights(int stage, int fp4, const void* W, void* dst, int64_t E, int64_t H, int64_t I, hipStream_t s);
size_t mx_packed_weights_bytes(int stage, int fp4, int64_t E, int64_t H, int64_t I);

int launch_gemm_stage(int kind, int stage, const GemmArgs& g, unsigned gx, unsigned gy, hipStream_t s);
// batches [nb0][nb1] of byte matrices [R, C] -> [C, Kp] (K-contiguous, zero tail), see bwmm.hip
// the bf16 kind: [R, C] bf16 (or fp8 widened to bf16 when w8) -> bf16 [C, Kp], Kp in elements, a multiple of 64
int launch_transpose_w16(const void* src, int w8, uint16_t* dst, int64_t R, int64_t C, int64_t src_row_stride, int64_t Kp,
                         int64_t nb0, int nb1, int64_t src_bs0, int64_t src_bs1, hipStream_t s);
int launch_transpose_fp8(const uint8_t* src, uint8_t* dst, int64_t R, int64_t C, int64_t src_row_stride, int64_t Kp,
                         int64_t nb0, int nb1, int64_t src_bs0, int64_t src_bs1, hipStream_t s);
// The fp8-row kind's weights in the x4 order the large-tile kernels read, K in natural order: gate/up
// [E, H, 2, I] -> [E, 128 (p), 2, H/512 (t), I, 4 (q)] with h = t*512 + p*4 + q; down [E, I_pad, H] ->
// [E, pI, nI, H, 4] with i = t*512 + p*4 + q (zeros past I).
int launch_relayout_x4(const uint8_t* gate_up, const uint8_t* down, uint8_t* dst, int which, int64_t E, int64_t H,
                       int64_t I, int64_t I_pad, hipStream_t s);
// The same for the bf16 kind's weights ([E, H, 2, I] / [E, I_pad, H] bf16, or fp8-e4m3 when w8, widened to bf16): an
// x4 element holds two consecutive K values of its column, the layout that of 8-bit weights with K extents of
// 2H / 2I bytes.
int launch_relayout_x4_bf16(const void* gate_up, const void* down, int w8, uint8_t* dst, int which, int64_t E, int64_t H,
                            int64_t I, int64_t I_pad, hipStream_t s);
int launch_fill_bytes(void* p, size_t bytes, uint8_t value, hipStream_t s);
int launch_row_requant(const float* Y, uint8_t* Yq, float* ys, const Bookkeeping& k, int64_t N, int64_t B, int64_t I,
                       int64_t Iw, hipStream_t s);

}  // namespace moe
