// Fused RMSNorm + quantise front end for gfx950: fp8-e4m3 per-row / static scale, and MXFP8.
//
// One 256-thread workgroup owns one row; the row is read once (16-byte coalesced loads),
// kept in registers across the two reductions (sum of squares, absolute maximum) and written
// once.  HBM traffic per row is the algorithmic minimum: 2H bytes in, H (+4 or +H/32) out.
//
// The fp32 arithmetic follows the reference goldens operation by operation (no FMA
// contraction) so that quantised codes are reproducible.  The one quantity whose value depends
// on evaluation order, the row's sum of squares, is accumulated in fp64 and rounded once, i.e.
// it is the correctly rounded fp32 sum that any fp32 summation order approximates:
//   ROW / STATIC: test/integration/nkilib/core/rmsnorm/test_rmsnorm_quant.py:46-97
//   MX:           test/integration/nkilib/core/subkernels/test_rmsnorm_mx_quantize_tkg.py:100-137,
//                 rms_norm test/integration/nkilib/utils/test_kernel_common.py:26-41,
//                 quantise rule test/utils/mx_utils.py:55-95
#include "common.hpp"

#pragma clang fp contract(off)

namespace moe {

constexpr int RQ_THREADS = 256;
constexpr int RQ_MAX_H = 16384;                       // rmsnorm_quant_constants.py:60-62 (MAX_H)
constexpr int RQ_MAX_CHUNKS = RQ_MAX_H / (RQ_THREADS * 8);  // 8-element chunks per thread

// Loads 8 consecutive elements starting at element index i (i % 8 == 0, i + 8 <= n guaranteed
// by the caller when `full`), converting to fp32.
__device__ __forceinline__ void load8(const void* base, int dtype, int64_t i, int64_t n, bool vec_ok, float* v) {
  if (dtype == MOE_DT_FP32) {
    const float* p = (const float*)base + i;
    if (vec_ok && i + 8 <= n) {
      float4 a = *(const float4*)p, b = *(const float4*)(p + 4);
      v[0] = a.x; v[1] = a.y; v[2] = a.z; v[3] = a.w; v[4] = b.x; v[5] = b.y; v[6] = b.z; v[7] = b.w;
    } else {
#pragma unroll
      for (int k = 0; k < 8; ++k) v[k] = (i + k < n) ? p[k] : 0.f;
    }
  } else {
    const uint16_t* p = (const uint16_t*)base + i;
    uint16_t h[8];
    if (vec_ok && i + 8 <= n) {
      uint4 a = *(const uint4*)p;
      h[0] = a.x & 0xffff; h[1] = a.x >> 16; h[2] = a.y & 0xffff; h[3] = a.y >> 16;
      h[4] = a.z & 0xffff; h[5] = a.z >> 16; h[6] = a.w & 0xffff; h[7] = a.w >> 16;
    } else {
#pragma unroll
      for (int k = 0; k < 8; ++k) h[k] = (i + k < n) ? p[k] : (uint16_t)0;
    }
#pragma unroll
    for (int k = 0; k < 8; ++k) v[k] = (dtype == MOE_DT_BF16) ? bf16_bits_to_f32(h[k]) : fp16_bits_to_f32(h[k]);
  }
}

// The same for 8 elements known to lie inside the tensor at a 16-byte aligned address: no bounds checks, one branch
// on the (uniform) dtype.
__device__ __forceinline__ void load8_vec(const void* base, int dtype, int64_t i, float* v) {
  if (dtype == MOE_DT_FP32) {
    const float* p = (const float*)base + i;
    const float4 a = *(const float4*)p, b = *(const float4*)(p + 4);
    v[0] = a.x; v[1] = a.y; v[2] = a.z; v[3] = a.w; v[4] = b.x; v[5] = b.y; v[6] = b.z; v[7] = b.w;
    return;
  }
  const uint4 a = *(const uint4*)((const uint16_t*)base + i);
  const uint32_t w[4] = {a.x, a.y, a.z, a.w};
  if (dtype == MOE_DT_BF16) {
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      v[2 * k] = __uint_as_float(w[k] << 16);
      v[2 * k + 1] = __uint_as_float(w[k] & 0xffff0000u);
    }
  } else {
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      v[2 * k] = fp16_bits_to_f32((uint16_t)(w[k] & 0xffffu));
      v[2 * k + 1] = fp16_bits_to_f32((uint16_t)(w[k] >> 16));
    }
  }
}

// MODE 0: per-row scale appended to the row ([H+4] record).  MODE 1: static scale.
template <int MODE>
__global__ __launch_bounds__(RQ_THREADS) void rmsnorm_quant_fp8_kernel(
    const void* __restrict__ x, int x_dtype, const void* __restrict__ gamma, int gamma_dtype,
    const float* __restrict__ static_scale, uint8_t* __restrict__ out, int64_t H, int64_t out_stride, float eps,
    float lower_bound, int do_norm, int vec_ok) {
  __shared__ float red[16];
  __shared__ double redd[16];
  const int64_t row = blockIdx.x;
  const int es = (x_dtype == MOE_DT_FP32) ? 4 : 2;
  const void* xr = (const uint8_t*)x + row * H * es;
  const int nchunk = (int)((H + RQ_THREADS * 8 - 1) / (RQ_THREADS * 8));

  float v[RQ_MAX_CHUNKS][8];
  double ss = 0.0;
#pragma unroll
  for (int j = 0; j < RQ_MAX_CHUNKS; ++j) {
    if (j < nchunk) {
      const int64_t i = ((int64_t)j * RQ_THREADS + threadIdx.x) * 8;
      if (i < H) {
        if (vec_ok) load8_vec(xr, x_dtype, i, v[j]);  // H % 8 == 0: the 8 elements lie inside the row
        else load8(xr, x_dtype, i, H, false, v[j]);
      } else {
#pragma unroll
        for (int k = 0; k < 8; ++k) v[j][k] = 0.f;
      }
#pragma unroll
      for (int k = 0; k < 8; ++k) ss += (double)v[j][k] * (double)v[j][k];
    }
  }

  if (do_norm) {
    const float total = (float)block_sum_f64(ss, redd);
    const float mean = total / (float)H;
    const float rms = sqrtf(mean);
    const float inv = 1.0f / (rms + eps);
#pragma unroll
    for (int j = 0; j < RQ_MAX_CHUNKS; ++j) {
      if (j < nchunk) {
        const int64_t i = ((int64_t)j * RQ_THREADS + threadIdx.x) * 8;
        if (i < H) {
          float g[8];
          if (vec_ok) load8_vec(gamma, gamma_dtype, i, g);
          else load8(gamma, gamma_dtype, i, H, false, g);
#pragma unroll
          for (int k = 0; k < 8; ++k) v[j][k] = (v[j][k] * inv) * g[k];
        }
      }
    }
  }

  float qs;  // multiplier applied before the cast
  if (MODE == 0) {
    float am = 0.f;
#pragma unroll
    for (int j = 0; j < RQ_MAX_CHUNKS; ++j)
      if (j < nchunk) {
#pragma unroll
        for (int k = 0; k < 8; ++k) am = fmaxf(am, fabsf(v[j][k]));
      }
    am = block_max(am, red);
    if (lower_bound > 0.f) am = fminf(am, lower_bound);
    float dq = am / 240.0f;
    dq = fmaxf(dq, 1e-6f);  // rmsnorm_quant.py:597-604
    qs = 1.0f / dq;
    if (threadIdx.x == 0) {
      uint32_t bits = __float_as_uint(dq);
      uint8_t* sp = out + row * out_stride + H;
      sp[0] = bits & 0xff; sp[1] = (bits >> 8) & 0xff; sp[2] = (bits >> 16) & 0xff; sp[3] = (bits >> 24) & 0xff;
    }
  } else {
    qs = 1.0f / static_scale[0];
  }

  uint8_t* orow = out + row * out_stride;
  const bool st4 = ((out_stride & 3) == 0) && ((((uintptr_t)out) & 3) == 0);
#pragma unroll
  for (int j = 0; j < RQ_MAX_CHUNKS; ++j) {
    if (j < nchunk) {
      const int64_t i = ((int64_t)j * RQ_THREADS + threadIdx.x) * 8;
      if (i < H) {
        float q[8];
#pragma unroll
        for (int k = 0; k < 8; ++k) {
          float t = v[j][k];
          if (MODE == 0) {
            if (lower_bound > 0.f) t = fminf(fmaxf(t, -lower_bound), lower_bound);
            q[k] = t * qs;
          } else {
            q[k] = fminf(fmaxf(t * qs, -240.0f), 240.0f);
          }
        }
        const uint32_t lo = pack4_e4m3(q[0], q[1], q[2], q[3]);
        const uint32_t hi = pack4_e4m3(q[4], q[5], q[6], q[7]);
        if (st4 && i + 8 <= H) {
          *(uint32_t*)(orow + i) = lo;
          *(uint32_t*)(orow + i + 4) = hi;
        } else {
#pragma unroll
          for (int k = 0; k < 8; ++k)
            if (i + k < H) orow[i + k] = (uint8_t)(((k < 4 ? lo : hi) >> (8 * (k & 3))) & 0xff);
        }
      }
    }
  }
}

// The common case of the ROW (MODE 0) and STATIC (MODE 1) front ends on their own: bf16 input and gamma, RMSNorm on,
// 16-byte aligned rows of a multiple of 8 elements.  Same arithmetic in the same order as rmsnorm_quant_fp8_kernel (the two are compared
// bit for bit in the tests), without its per-element dtype and bounds decisions, with the row kept packed as loaded
// until it is used (MAXC chunks of 8 elements per thread instead of room for the longest row) and gamma fetched
// with the row, ahead of the first reduction: the general kernel spends its time in the vector ALUs and, at 8
// chunks of unpacked values per thread, runs four workgroups per CU.
template <int MAXC, int MODE>
__global__ __launch_bounds__(RQ_THREADS) __attribute__((amdgpu_waves_per_eu(MAXC <= 2 ? 6 : MAXC <= 4 ? 4 : 3, 8))) void
rmsnorm_quant_row_bf16_kernel(const uint16_t* __restrict__ x, const uint16_t* __restrict__ gamma,
                              const float* __restrict__ static_scale, uint8_t* __restrict__ out, int64_t H, float eps,
                              float lower_bound) {
  __shared__ float red[16];
  __shared__ double redd[16];
  const int64_t row = blockIdx.x;
  const uint16_t* xr = x + row * H;
  uint4 raw[MAXC], graw[MAXC];
#pragma unroll
  for (int j = 0; j < MAXC; ++j) {
    const int64_t i = ((int64_t)j * RQ_THREADS + threadIdx.x) * 8;
    raw[j] = make_uint4(0, 0, 0, 0);
    if (i < H) raw[j] = *(const uint4*)(xr + i);
  }
#pragma unroll
  for (int j = 0; j < MAXC; ++j) {
    const int64_t i = ((int64_t)j * RQ_THREADS + threadIdx.x) * 8;
    graw[j] = make_uint4(0, 0, 0, 0);
    if (i < H) graw[j] = *(const uint4*)(gamma + i);
  }
  double ss = 0.0;
#pragma unroll
  for (int j = 0; j < MAXC; ++j) {
    const uint32_t w[4] = {raw[j].x, raw[j].y, raw[j].z, raw[j].w};
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      const double lo = (double)bf16_lo(w[k]), hi = (double)bf16_hi(w[k]);
      ss = fma(lo, lo, ss);  // the products are exact in double, so fusing changes nothing
      ss = fma(hi, hi, ss);
    }
  }
  const float total = (float)block_sum_f64(ss, redd);
  const float inv = 1.0f / (sqrtf(total / (float)H) + eps);
  float v[MAXC][8];
  float am = 0.f;
#pragma unroll
  for (int j = 0; j < MAXC; ++j) {
    const uint32_t w[4] = {raw[j].x, raw[j].y, raw[j].z, raw[j].w};
    const uint32_t g[4] = {graw[j].x, graw[j].y, graw[j].z, graw[j].w};
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      v[j][2 * k] = (bf16_lo(w[k]) * inv) * bf16_lo(g[k]);
      v[j][2 * k + 1] = (bf16_hi(w[k]) * inv) * bf16_hi(g[k]);
      if (MODE == 0) am = fmaxf(am, fmaxf(fabsf(v[j][2 * k]), fabsf(v[j][2 * k + 1])));
    }
  }
  const bool clip = MODE == 0 && lower_bound > 0.f;  // uniform
  float qs;
  uint8_t* orow = out + row * (MODE == 0 ? H + 4 : H);
  if (MODE == 0) {
    am = block_max(am, red);
    if (clip) am = fminf(am, lower_bound);
    const float dq = fmaxf(am / 240.0f, 1e-6f);  // rmsnorm_quant.py:597-604
    qs = 1.0f / dq;
    if (threadIdx.x == 0) *(uint32_t*)(orow + H) = __float_as_uint(dq);  // H % 8 == 0: the record's scale is 4-byte aligned
  } else {
    qs = 1.0f / static_scale[0];
  }
#pragma unroll
  for (int j = 0; j < MAXC; ++j) {
    const int64_t i = ((int64_t)j * RQ_THREADS + threadIdx.x) * 8;
    if (i < H) {
      float q[8];
#pragma unroll
      for (int k = 0; k < 8; ++k) {
        if (MODE == 0) q[k] = (clip ? fminf(fmaxf(v[j][k], -lower_bound), lower_bound) : v[j][k]) * qs;
        else q[k] = fminf(fmaxf(v[j][k] * qs, -240.0f), 240.0f);
      }
      *(uint32_t*)(orow + i) = pack4_e4m3(q[0], q[1], q[2], q[3]);
      *(uint32_t*)(orow + i + 4) = pack4_e4m3(q[4], q[5], q[6], q[7]);
    }
  }
}

// MXFP8 front end.  Thread t of the row's workgroup owns MX blocks blk = t and t + 256
// (blk = tile*16 + p8 covers k' in [blk*32, blk*32+32)); its 32 inputs are four runs of 8
// contiguous elements at h = q*(H/4) + tile*128 + p8*8 + r.
constexpr int MXQ_MAX_BLK = RQ_MAX_H / 32 / RQ_THREADS;  // 2

// Eight 16-bit elements (bf16 or fp16) as loaded, widened.
__device__ __forceinline__ void unpack8(const uint4& a, int dtype, float* v) {
  const uint32_t w[4] = {a.x, a.y, a.z, a.w};
#pragma unroll
  for (int k = 0; k < 4; ++k) {
    if (dtype == MOE_DT_BF16) {
      v[2 * k] = bf16_lo(w[k]);
      v[2 * k + 1] = bf16_hi(w[k]);
    } else {
      v[2 * k] = fp16_bits_to_f32((uint16_t)(w[k] & 0xffffu));
      v[2 * k + 1] = fp16_bits_to_f32((uint16_t)(w[k] >> 16));
    }
  }
}

// Fused residual add of the MXFP8 front end (rmsnorm_mx_quantize_tkg.py:29-40,214-232): hidden = input + residual,
// rounded to the input type (the reference adds into a buffer of the residual's type; its golden adds the two arrays
// in their own type, test_rmsnorm_mx_quantize_tkg.py:104-117), kept as the row that is normalised and written out
// as output_residual.  Eight packed 16-bit values at a time.
__device__ __forceinline__ uint4 add8_16(const uint4& a, const uint4& b, int dtype) {
  float x[8], y[8];
  unpack8(a, dtype, x);
  unpack8(b, dtype, y);
  uint32_t w[4];
#pragma unroll
  for (int k = 0; k < 4; ++k) {
    const float s0 = x[2 * k] + y[2 * k], s1 = x[2 * k + 1] + y[2 * k + 1];
    if (dtype == MOE_DT_BF16) {
      w[k] = pack2_bf16(s0, s1);
    } else {
      const _Float16 h0 = (_Float16)s0, h1 = (_Float16)s1;  // round to nearest even
      w[k] = (uint32_t)__builtin_bit_cast(uint16_t, h0) | ((uint32_t)__builtin_bit_cast(uint16_t, h1) << 16);
    }
  }
  return make_uint4(w[0], w[1], w[2], w[3]);
}

// MAXB = MX blocks per thread (1 for H <= 32 * RQ_THREADS).  A row is one load round trip, one reduction and one
// store, so the rows in flight per CU are what fills the memory pipeline, and registers decide how many those are:
// 16-bit inputs (X16) stay packed as loaded (16 registers per MX block instead of 32) and the normalised values,
// which are bf16 by definition, are kept as bf16 pairs.
template <int MAXB, bool X16>
__global__ __launch_bounds__(RQ_THREADS) __attribute__((amdgpu_waves_per_eu(MAXB == 1 ? (X16 ? 6 : 5) : 3, 8))) void rmsnorm_quant_mx_kernel(
    const void* __restrict__ x, int x_dtype, const void* __restrict__ residual, void* __restrict__ out_res,
    const void* __restrict__ gamma, int gamma_dtype, uint8_t* __restrict__ out_q, uint8_t* __restrict__ out_scale,
    uint16_t* __restrict__ out_norm, int64_t rows, int64_t H, float eps, float hidden_actual, int do_norm, int layout,
    int tpr) {
  __shared__ double redd[16];
  // tpr = threads per row (64, 128 or 256): short rows share a workgroup, RQ_THREADS / tpr of them
  const int tpr_lg = (tpr == 64) ? 6 : ((tpr == 128) ? 7 : 8);
  const int lt = threadIdx.x & (tpr - 1);
  const int64_t row_raw = ((int64_t)blockIdx.x << (8 - tpr_lg)) + (threadIdx.x >> tpr_lg);
  const bool row_ok = row_raw < rows;
  const int64_t row = row_ok ? row_raw : rows - 1;
  const int es = X16 ? 2 : 4;
  const void* xr = (const uint8_t*)x + row * H * es;
  const void* rr = residual ? (const uint8_t*)residual + row * H * es : nullptr;
  void* orr = out_res ? (uint8_t*)out_res + row * H * es : nullptr;
  const int nblk = row_ok ? (int)(H / 32) : 0;  // threads of a row past the end own no block
  const int nT = (int)(H / 512);
  const int64_t Hq = H / 4;

  uint4 raw[MAXB][X16 ? 4 : 8];  // the thread's inputs as loaded: [block][q] (fp32: [block][2 q + half])
  double ss = 0.0;
#pragma unroll
  for (int j = 0; j < MAXB; ++j) {
    const int blk = j * tpr + lt;
    if (blk < nblk) {
      const int tile = blk >> 4, p8 = blk & 15;
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const int64_t i = q * Hq + tile * 128 + p8 * 8;
        float t[8];
        if constexpr (X16) {
          raw[j][q] = *(const uint4*)((const uint16_t*)xr + i);
          if (rr) {
            raw[j][q] = add8_16(raw[j][q], *(const uint4*)((const uint16_t*)rr + i), x_dtype);
            if (orr) *(uint4*)((uint16_t*)orr + i) = raw[j][q];
          }
          unpack8(raw[j][q], x_dtype, t);
        } else {
          raw[j][2 * q] = *(const uint4*)((const float*)xr + i);
          raw[j][2 * q + 1] = *(const uint4*)((const float*)xr + i + 4);
          __builtin_memcpy(t, &raw[j][2 * q], 32);
          if (rr) {
            float rv[8];
            __builtin_memcpy(rv, (const float*)rr + i, 32);
#pragma unroll
            for (int r = 0; r < 8; ++r) t[r] += rv[r];
            __builtin_memcpy(&raw[j][2 * q], t, 32);
            if (orr) __builtin_memcpy((float*)orr + i, t, 32);
          }
        }
#pragma unroll
        for (int r = 0; r < 8; ++r) ss += (double)t[r] * (double)t[r];
      }
    }
  }
  float inv = 1.0f;
  if (do_norm) {
    const float total = (float)group_sum_f64(ss, redd, tpr);
    const float rms = sqrtf(total / hidden_actual + eps);
    inv = 1.0f / rms;
  }
#pragma unroll
  for (int j = 0; j < MAXB; ++j) {
    const int blk = j * tpr + lt;
    if (blk < nblk) {
      const int tile = blk >> 4, p8 = blk & 15;
      float am = 0.f;
      uint32_t nv[4][4];  // normalised values, rounded to bf16: [q][pair of r]
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        float t[8], g[8];
        if constexpr (X16) unpack8(raw[j][q], x_dtype, t);
        else __builtin_memcpy(t, &raw[j][2 * q], 32);
        if (do_norm) load8_vec(gamma, gamma_dtype, q * Hq + tile * 128 + p8 * 8, g);
#pragma unroll
        for (int r = 0; r < 8; r += 2) {
          float t0 = t[r], t1 = t[r + 1];
          if (do_norm) {
            t0 = (t0 * inv) * g[r];
            t1 = (t1 * inv) * g[r + 1];
          }
          const uint32_t u = pack2_bf16(t0, t1);
          nv[q][r >> 1] = u;
          am = fmaxf(am, fmaxf(fabsf(bf16_lo(u)), fabsf(bf16_hi(u))));
        }
      }
      if (out_norm != nullptr) {
#pragma unroll
        for (int q = 0; q < 4; ++q)
#pragma unroll
          for (int r = 0; r < 8; ++r) {
            const int64_t p = p8 * 8 + r, h1 = (int64_t)q * nT + tile;
            out_norm[(p * rows + row) * (H / 128) + h1] = (uint16_t)((r & 1) ? (nv[q][r >> 1] >> 16) : (nv[q][r >> 1] & 0xffffu));
          }
      }
      const uint32_t sb = mx_scale_byte(am);
      const float is = mx_inv_scale(sb);
      uint32_t d[8];
#pragma unroll
      for (int r = 0; r < 8; ++r) {
        float e[4];
#pragma unroll
        for (int q = 0; q < 4; ++q) e[q] = ((r & 1) ? bf16_hi(nv[q][r >> 1]) : bf16_lo(nv[q][r >> 1])) * is;
        d[r] = pack4_e4m3(clip448(e[0]), clip448(e[1]), clip448(e[2]), clip448(e[3]));
      }
      if (layout == MOE_MX_LAYOUT_TOKEN_MAJOR) {
        uint4* o = (uint4*)(out_q + row * H + (int64_t)blk * 32);
        o[0] = make_uint4(d[0], d[1], d[2], d[3]);
        o[1] = make_uint4(d[4], d[5], d[6], d[7]);
        out_scale[row * nblk + blk] = (uint8_t)sb;
      } else {
        uint32_t* o = (uint32_t*)out_q;
#pragma unroll
        for (int r = 0; r < 8; ++r) o[((int64_t)(p8 * 8 + r) * nT + tile) * rows + row] = d[r];
        const int srow = (layout == MOE_MX_LAYOUT_REF_DENSE) ? p8 : ((p8 >> 2) * 32 + (p8 & 3));
        out_scale[((int64_t)srow * nT + tile) * rows + row] = (uint8_t)sb;
      }
    }
  }
}

// The common case of the MXFP8 front end on its own: bf16 input and gamma, RMSNorm on, token-major output and no
// copy of the normalised values.  Same results as rmsnorm_quant_mx_kernel, with the arithmetic per element cut to
// what this case needs, because at ~20 vector instructions per element the general kernel is bound by the vector
// ALUs and not by memory:
//  - the block's amax is taken on the packed bf16 bit patterns (sign masked off, 16-bit unsigned max: magnitudes of
//    finite bf16 values order like their bit patterns),
//  - quantisation is v_cvt_scalef32_pk_fp8_bf16: two bf16 values divided by the power of two in the scale operand's
//    exponent field and rounded to e4m3 (nearest even), one instruction per pair.  It differs from "multiply, clip
//    to +-448, convert" in one respect only: a quotient that rounds above 448 gives NaN (0x7f / 0xff) instead of
//    +-448; nan_to_max() turns those bytes into 0x7e / 0xfe.  (Checked over every finite bf16 value against every
//    scale byte whose block can hold it.)
//  - gamma is fetched with the row, ahead of the reduction, so the barrier hides its latency.
__device__ __forceinline__ uint32_t nan_to_max(uint32_t d) {
  // a byte is 0x7f / 0xff exactly when its low seven bits are all set: adding 1 to them carries into bit 7
  const uint32_t m = ((d & 0x7f7f7f7fu) + 0x01010101u) & 0x80808080u;
  return d - (m >> 7);
}

template <int MAXB>
__global__ __launch_bounds__(RQ_THREADS) __attribute__((amdgpu_waves_per_eu(MAXB == 1 ? 6 : 3, 8))) void
rmsnorm_quant_mx_bf16_kernel(const uint16_t* __restrict__ x, const uint16_t* __restrict__ residual,
                             uint16_t* __restrict__ out_res, const uint16_t* __restrict__ gamma,
                             uint8_t* __restrict__ out_q, uint8_t* __restrict__ out_scale, int64_t rows, int64_t H,
                             float eps, float hidden_actual, int tpr) {
  typedef unsigned short v2u16 __attribute__((ext_vector_type(2)));
  typedef short v2s16 __attribute__((ext_vector_type(2)));
  typedef __bf16 v2bf16 __attribute__((ext_vector_type(2)));
  __shared__ double redd[16];
  const int tpr_lg = (tpr == 64) ? 6 : ((tpr == 128) ? 7 : 8);
  const int lt = threadIdx.x & (tpr - 1);
  const int nblk_row = (int)(H / 32);
  const int64_t Hq = H / 4;
  const int64_t row_raw = ((int64_t)blockIdx.x << (8 - tpr_lg)) + (threadIdx.x >> tpr_lg);
  const int64_t row = row_raw < rows ? row_raw : rows - 1;
  const int nblk = row_raw < rows ? nblk_row : 0;  // threads of a row past the end own no block
  const uint16_t* xr = x + row * H;

  uint4 raw[MAXB][4], graw[MAXB][4];
#pragma unroll
  for (int j = 0; j < MAXB; ++j) {
    const int blk = j * tpr + lt;
    if (blk < nblk) {
#pragma unroll
      for (int q = 0; q < 4; ++q) raw[j][q] = *(const uint4*)(xr + q * Hq + blk * 8);  // tile*128 + p8*8 == blk*8
    }
  }
  if (residual != nullptr) {  // hidden = bf16(input + residual): the row that is normalised and written back
#pragma unroll
    for (int j = 0; j < MAXB; ++j) {
      const int blk = j * tpr + lt;
      if (blk < nblk) {
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          raw[j][q] = add8_16(raw[j][q], *(const uint4*)(residual + row * H + q * Hq + blk * 8), MOE_DT_BF16);
          if (out_res != nullptr) *(uint4*)(out_res + row * H + q * Hq + blk * 8) = raw[j][q];
        }
      }
    }
  }
#pragma unroll
  for (int j = 0; j < MAXB; ++j) {
    const int blk = j * tpr + lt;
    if (blk < nblk) {
#pragma unroll
      for (int q = 0; q < 4; ++q) graw[j][q] = *(const uint4*)(gamma + q * Hq + blk * 8);
    }
  }
  {
    double ss = 0.0;
#pragma unroll
    for (int j = 0; j < MAXB; ++j) {
      if (j * tpr + lt < nblk) {
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const uint32_t w[4] = {raw[j][q].x, raw[j][q].y, raw[j][q].z, raw[j][q].w};
#pragma unroll
          for (int k = 0; k < 4; ++k) {
            const double lo = (double)bf16_lo(w[k]), hi = (double)bf16_hi(w[k]);
            ss = fma(lo, lo, ss);  // the products are exact in double, so fusing changes nothing
            ss = fma(hi, hi, ss);
          }
        }
      }
    }
    const float inv = 1.0f / sqrtf((float)group_sum_f64(ss, redd, tpr) / hidden_actual + eps);
#pragma unroll
    for (int j = 0; j < MAXB; ++j) {
      const int blk = j * tpr + lt;
      if (blk < nblk) {
        uint32_t nv[4][4];  // normalised values, rounded to bf16: [q][pair of r]
        v2u16 mx = {0, 0};
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const uint32_t w[4] = {raw[j][q].x, raw[j][q].y, raw[j][q].z, raw[j][q].w};
          const uint32_t g[4] = {graw[j][q].x, graw[j][q].y, graw[j][q].z, graw[j][q].w};
#pragma unroll
          for (int k = 0; k < 4; ++k) {
            const uint32_t u =
                pack2_bf16((bf16_lo(w[k]) * inv) * bf16_lo(g[k]), (bf16_hi(w[k]) * inv) * bf16_hi(g[k]));
            nv[q][k] = u;
            mx = __builtin_elementwise_max(mx, __builtin_bit_cast(v2u16, u & 0x7fff7fffu));
          }
        }
        const uint32_t am = mx.x > mx.y ? mx.x : mx.y;    // bf16 bits of the block's amax
        const int e8 = (int)(am >> 7) - 8;                // its biased exponent, less 8
        const uint32_t sb = (uint32_t)(e8 < 0 ? 0 : e8);  // mx_scale_byte()
        const float scale = __uint_as_float(sb << 23);    // 2^(sb - 127): only the exponent field is read
        uint32_t d[8];
#pragma unroll
        for (int k = 0; k < 4; ++k) {
          v2s16 w01 = {0, 0}, w23 = {0, 0};
          w01 = __builtin_amdgcn_cvt_scalef32_pk_fp8_bf16(w01, __builtin_bit_cast(v2bf16, nv[0][k]), scale, false);
          w01 = __builtin_amdgcn_cvt_scalef32_pk_fp8_bf16(w01, __builtin_bit_cast(v2bf16, nv[1][k]), scale, true);
          w23 = __builtin_amdgcn_cvt_scalef32_pk_fp8_bf16(w23, __builtin_bit_cast(v2bf16, nv[2][k]), scale, false);
          w23 = __builtin_amdgcn_cvt_scalef32_pk_fp8_bf16(w23, __builtin_bit_cast(v2bf16, nv[3][k]), scale, true);
          const uint32_t a = __builtin_bit_cast(uint32_t, w01), b = __builtin_bit_cast(uint32_t, w23);
          // a = (q0 r, q0 r+1, q1 r, q1 r+1), b the same for q2, q3: regroup by r
          d[2 * k] = nan_to_max(__builtin_amdgcn_perm(b, a, 0x06040200u));
          d[2 * k + 1] = nan_to_max(__builtin_amdgcn_perm(b, a, 0x07050301u));
        }
        uint4* o = (uint4*)(out_q + row * H + (int64_t)blk * 32);
        o[0] = make_uint4(d[0], d[1], d[2], d[3]);
        o[1] = make_uint4(d[4], d[5], d[6], d[7]);
        out_scale[row * nblk + blk] = (uint8_t)sb;
      }
    }
  }
}

static bool valid_in_dtype(int d) { return d == MOE_DT_BF16 || d == MOE_DT_FP16 || d == MOE_DT_FP32; }

}  // namespace moe

using namespace moe;

template <int MODE>
static void launch_bf16_front_end(const void* x, const void* gamma, const float* static_scale, void* out, int64_t rows,
                                  int64_t H, float eps, float lower_bound, hipStream_t stream) {
  auto launch = [&](auto kernel) {
    hipLaunchKernelGGL(kernel, dim3((unsigned)rows), dim3(RQ_THREADS), 0, stream, (const uint16_t*)x,
                       (const uint16_t*)gamma, static_scale, (uint8_t*)out, H, eps, lower_bound);
  };
  const int64_t chunks = (H + RQ_THREADS * 8 - 1) / (RQ_THREADS * 8);
  if (chunks <= 1) launch(rmsnorm_quant_row_bf16_kernel<1, MODE>);
  else if (chunks <= 2) launch(rmsnorm_quant_row_bf16_kernel<2, MODE>);
  else if (chunks <= 4) launch(rmsnorm_quant_row_bf16_kernel<4, MODE>);
  else launch(rmsnorm_quant_row_bf16_kernel<8, MODE>);
}

extern "C" int moe_rmsnorm_quant_fp8_row(const void* x, int x_dtype, const void* gamma, int gamma_dtype, void* out,
                                         int64_t rows, int64_t H, float eps, float lower_bound, int do_norm,
                                         void* stream) {
  if (!x || !out || rows < 0 || H <= 0 || !valid_in_dtype(x_dtype)) return MOE_E_BAD_ARG;
  if (do_norm && (!gamma || !valid_in_dtype(gamma_dtype))) return MOE_E_BAD_ARG;
  if (lower_bound < 0.f || eps < 0.f) return MOE_E_BAD_ARG;
  if (H > RQ_MAX_H) return MOE_E_BAD_SHAPE;
  if (rows == 0) return MOE_OK;
  const int vec_ok = (H % 8 == 0) && (((uintptr_t)x & 15) == 0) && (!do_norm || ((uintptr_t)gamma & 15) == 0);
  if (vec_ok && do_norm && x_dtype == MOE_DT_BF16 && gamma_dtype == MOE_DT_BF16 && (((uintptr_t)out & 3) == 0)) {
    launch_bf16_front_end<0>(x, gamma, nullptr, out, rows, H, eps, lower_bound, (hipStream_t)stream);
    MOE_CHECK_LAUNCH();
    return MOE_OK;
  }
  hipLaunchKernelGGL(rmsnorm_quant_fp8_kernel<0>, dim3((unsigned)rows), dim3(RQ_THREADS), 0, (hipStream_t)stream, x,
                     x_dtype, gamma, gamma_dtype, (const float*)nullptr, (uint8_t*)out, H, H + 4, eps, lower_bound,
                     do_norm, vec_ok);
  MOE_CHECK_LAUNCH();
  return MOE_OK;
}

extern "C" int moe_rmsnorm_quant_fp8_static(const void* x, int x_dtype, const void* gamma, int gamma_dtype,
                                            const float* input_dequant_scale, void* out, int64_t rows, int64_t H,
                                            float eps, int do_norm, void* stream) {
  if (!x || !out || !input_dequant_scale || rows < 0 || H <= 0 || !valid_in_dtype(x_dtype)) return MOE_E_BAD_ARG;
  if (do_norm && (!gamma || !valid_in_dtype(gamma_dtype))) return MOE_E_BAD_ARG;
  if (eps < 0.f) return MOE_E_BAD_ARG;
  if (H > RQ_MAX_H) return MOE_E_BAD_SHAPE;
  if (rows == 0) return MOE_OK;
  const int vec_ok = (H % 8 == 0) && (((uintptr_t)x & 15) == 0) && (!do_norm || ((uintptr_t)gamma & 15) == 0);
  if (vec_ok && do_norm && x_dtype == MOE_DT_BF16 && gamma_dtype == MOE_DT_BF16 && (((uintptr_t)out & 3) == 0)) {
    launch_bf16_front_end<1>(x, gamma, input_dequant_scale, out, rows, H, eps, 0.f, (hipStream_t)stream);
    MOE_CHECK_LAUNCH();
    return MOE_OK;
  }
  hipLaunchKernelGGL(rmsnorm_quant_fp8_kernel<1>, dim3((unsigned)rows), dim3(RQ_THREADS), 0, (hipStream_t)stream, x,
                     x_dtype, gamma, gamma_dtype, input_dequant_scale, (uint8_t*)out, H, H, eps, 0.f, do_norm, vec_ok);
  MOE_CHECK_LAUNCH();
  return MOE_OK;
}

extern "C" int moe_rmsnorm_quant_mxfp8(const void* x, int x_dtype, const void* residual, void* out_residual,
                                       const void* gamma, int gamma_dtype, void* out_q, void* out_scale,
                                       void* out_norm, int64_t rows, int64_t H, float eps, int64_t hidden_actual,
                                       int do_norm, int layout, void* stream) {
  if (!x || !out_q || !out_scale || rows < 0 || H <= 0 || !valid_in_dtype(x_dtype)) return MOE_E_BAD_ARG;
  // the sum is needed by the caller's residual stream: the reference requires output_residual with residual
  // (norm_tkg_utils.py:473-476)
  if ((residual != nullptr) != (out_residual != nullptr)) return MOE_E_BAD_ARG;
  if (residual && ((((uintptr_t)residual) & 15) != 0 || (((uintptr_t)out_residual) & 15) != 0)) return MOE_E_BAD_ARG;
  if (do_norm && (!gamma || !valid_in_dtype(gamma_dtype))) return MOE_E_BAD_ARG;
  if (layout < 0 || layout > 2 || eps < 0.f) return MOE_E_BAD_ARG;
  if (H % 512 != 0 || H > RQ_MAX_H) return MOE_E_BAD_SHAPE;
  if (((uintptr_t)x & 15) != 0 || ((uintptr_t)out_q & 15) != 0 || (do_norm && ((uintptr_t)gamma & 15) != 0))
    return MOE_E_BAD_ARG;
  if (rows == 0) return MOE_OK;
  const float ha = (float)(hidden_actual > 0 ? hidden_actual : H);
  const bool x16 = x_dtype != MOE_DT_FP32;
  const int nblk = (int)(H / 32);
  const int tpr = nblk <= 64 ? 64 : (nblk <= 128 ? 128 : RQ_THREADS);
  const int rpw = RQ_THREADS / tpr;  // rows per workgroup
  const dim3 grid((unsigned)((rows + rpw - 1) / rpw)), block(RQ_THREADS);
  auto launch = [&](auto kernel) {
    hipLaunchKernelGGL(kernel, grid, block, 0, (hipStream_t)stream, x, x_dtype, residual, out_residual, gamma,
                       gamma_dtype, (uint8_t*)out_q, (uint8_t*)out_scale, (uint16_t*)out_norm, rows, H, eps, ha, do_norm,
                       layout, tpr);
  };
  const bool fast = x_dtype == MOE_DT_BF16 && do_norm && gamma_dtype == MOE_DT_BF16 && !out_norm &&
                    layout == MOE_MX_LAYOUT_TOKEN_MAJOR;
  if (fast) {
    auto launch_fast = [&](auto kernel) {
      hipLaunchKernelGGL(kernel, grid, block, 0, (hipStream_t)stream, (const uint16_t*)x, (const uint16_t*)residual,
                         (uint16_t*)out_residual, (const uint16_t*)gamma, (uint8_t*)out_q, (uint8_t*)out_scale, rows, H,
                         eps, ha, tpr);
    };
    if (H <= 32 * RQ_THREADS) launch_fast(rmsnorm_quant_mx_bf16_kernel<1>);
    else launch_fast(rmsnorm_quant_mx_bf16_kernel<MXQ_MAX_BLK>);
  } else if (H <= 32 * RQ_THREADS) {
    if (x16) launch(rmsnorm_quant_mx_kernel<1, true>);
    else launch(rmsnorm_quant_mx_kernel<1, false>);
  } else {
    if (x16) launch(rmsnorm_quant_mx_kernel<MXQ_MAX_BLK, true>);
    else launch(rmsnorm_quant_mx_kernel<MXQ_MAX_BLK, false>);
  }
  MOE_CHECK_LAUNCH();
  return MOE_OK;
}
