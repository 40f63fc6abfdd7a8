// Shared device/host helpers for the gfx950 MoE kernels.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "moe_gfx950.h"

#define MOE_CHECK_LAUNCH()                           \
  do {                                               \
    hipError_t e__ = hipGetLastError();              \
    if (e__ != hipSuccess) return MOE_E_LAUNCH;      \
  } while (0)

namespace moe {

constexpr int WAVE = 64;

typedef int v8i __attribute__((ext_vector_type(8)));
typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v2i __attribute__((ext_vector_type(2)));
typedef float v4f __attribute__((ext_vector_type(4)));
typedef __bf16 v8bf __attribute__((ext_vector_type(8)));

// ---- bf16 <-> fp32 (bit level, round-to-nearest-even) ---------------------------------
__device__ __forceinline__ float bf16_bits_to_f32(uint16_t b) { return __uint_as_float(((uint32_t)b) << 16); }

__device__ __forceinline__ uint16_t f32_to_bf16_bits(float f) {
  uint32_t u = __float_as_uint(f);
  if ((u & 0x7fffffffu) > 0x7f800000u) return 0x7fc0;  // NaN
  u += 0x7fffu + ((u >> 16) & 1u);
  return (uint16_t)(u >> 16);
}

__device__ __forceinline__ float round_to_bf16(float f) { return bf16_bits_to_f32(f32_to_bf16_bits(f)); }

// Two values rounded to bf16 (round to nearest even) with the hardware's packed conversion: a in the low half.
__device__ __forceinline__ uint32_t pack2_bf16(float a, float b) {
  typedef __bf16 v2bf_t __attribute__((ext_vector_type(2)));
  typedef float v2f_t __attribute__((ext_vector_type(2)));
  const v2bf_t h = __builtin_convertvector((v2f_t){a, b}, v2bf_t);
  return __builtin_bit_cast(uint32_t, h);
}
__device__ __forceinline__ float bf16_lo(uint32_t u) { return __uint_as_float(u << 16); }
__device__ __forceinline__ float bf16_hi(uint32_t u) { return __uint_as_float(u & 0xffff0000u); }

__device__ __forceinline__ float fp16_bits_to_f32(uint16_t b) {
  _Float16 h;
  __builtin_memcpy(&h, &b, 2);
  return (float)h;
}

// Generic scalar load of element i of a tensor of runtime dtype.
__device__ __forceinline__ float load_as_f32(const void* p, int dtype, int64_t i) {
  if (dtype == MOE_DT_BF16) return bf16_bits_to_f32(((const uint16_t*)p)[i]);
  if (dtype == MOE_DT_FP16) return fp16_bits_to_f32(((const uint16_t*)p)[i]);
  return ((const float*)p)[i];
}

// ---- fp8 e4m3fn (OCP) -----------------------------------------------------------------
// Packs two floats (already clipped by the caller) to two e4m3fn bytes, RNE.
__device__ __forceinline__ uint32_t pack4_e4m3(float a, float b, float c, float d) {
  int r = __builtin_amdgcn_cvt_pk_fp8_f32(a, b, 0, false);
  r = __builtin_amdgcn_cvt_pk_fp8_f32(c, d, r, true);
  return (uint32_t)r;
}

// Exact decode of one e4m3fn byte.
__device__ __forceinline__ float e4m3_to_f32(uint32_t byte) {
  uint32_t s = (byte & 0x80u) << 24;
  uint32_t em = byte & 0x7fu;
  float v;
  if ((em >> 3) == 0) {
    v = (float)em * 0.001953125f;  // subnormal: m * 2^-9
  } else {
    v = __uint_as_float((em << 20) + (120u << 23));  // rebias 7 -> 127
  }
  return __uint_as_float(__float_as_uint(v) | s);
}

// ---- reductions ------------------------------------------------------------------------
__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
  return v;
}
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, 64));
  return v;
}

// Block-wide sum / max over blockDim.x threads (multiple of 64, <= 1024). `red` holds 16 floats.
__device__ __forceinline__ float block_sum(float v, float* red) {
  v = wave_sum(v);
  const int w = threadIdx.x >> 6, nw = blockDim.x >> 6;
  __syncthreads();
  if ((threadIdx.x & 63) == 0) red[w] = v;
  __syncthreads();
  float t = 0.f;
  for (int i = 0; i < nw; ++i) t += red[i];
  return t;
}
// Block-wide sum in double precision (`red` holds 16 doubles).
__device__ __forceinline__ double block_sum_f64(double v, double* red) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
  const int w = threadIdx.x >> 6, nw = blockDim.x >> 6;
  __syncthreads();
  if ((threadIdx.x & 63) == 0) red[w] = v;
  __syncthreads();
  double t = 0.0;
  for (int i = 0; i < nw; ++i) t += red[i];
  return t;
}
// The same over groups of `group` consecutive threads (64, 128 or 256 of a 256-thread workgroup): every thread gets
// the sum of its group.
__device__ __forceinline__ double group_sum_f64(double v, double* red, int group) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
  const int w = threadIdx.x >> 6, gw = group >> 6;  // gw is 1, 2 or 4
  __syncthreads();
  if ((threadIdx.x & 63) == 0) red[w] = v;
  __syncthreads();
  const int w0 = w & ~(gw - 1);
  double t = 0.0;
  for (int i = 0; i < gw; ++i) t += red[w0 + i];
  return t;
}
__device__ __forceinline__ float block_max(float v, float* red) {
  v = wave_max(v);
  const int w = threadIdx.x >> 6, nw = blockDim.x >> 6;
  __syncthreads();
  if ((threadIdx.x & 63) == 0) red[w] = v;
  __syncthreads();
  float t = red[0];
  for (int i = 1; i < nw; ++i) t = fmaxf(t, red[i]);
  return t;
}

// Exclusive prefix sum of v over the workgroup (blockDim.x a multiple of 64, at most 1024): shuffles
// inside a wave, one exchange of the wave totals through `ws` (16 ints).  *total = sum over the workgroup.
__device__ __forceinline__ int block_excl_scan(int v, int* ws, int* total) {
  const int lane = threadIdx.x & 63, w = threadIdx.x >> 6, nw = blockDim.x >> 6;
  int inc = v;
#pragma unroll
  for (int o = 1; o < 64; o <<= 1) {
    const int t = __shfl_up(inc, o, 64);
    if (lane >= o) inc += t;
  }
  __syncthreads();  // `ws` may still be read from a previous call
  if (lane == 63) ws[w] = inc;
  __syncthreads();
  int base = 0, tot = 0;
  for (int i = 0; i < nw; ++i) {
    const int t = ws[i];
    base += (i < w) ? t : 0;
    tot += t;
  }
  *total = tot;
  return base + inc - v;
}

// ---- activation functions (ActFnType, common_types.py:32-36) ---------------------------
// x * sigmoid(k x) with the hardware exp2 and reciprocal (about 1 ulp each): the library expf and
// the IEEE division cost ~100 instructions per element, which made the gate/up epilogue as long
// as half its K loop.  Saturates correctly: exp2 -> inf gives x * 0, exp2 -> 0 gives x.
__device__ __forceinline__ float x_sigmoid(float x, float k) {
  const float e = __builtin_amdgcn_exp2f(x * (-1.44269504088896340736f * k));
  return x * __builtin_amdgcn_rcpf(1.0f + e);
}
__device__ __forceinline__ float act_apply(float x, int kind) {
  switch (kind) {
    case MOE_ACT_SILU:
      return x_sigmoid(x, 1.0f);
    case MOE_ACT_GELU:
      return 0.5f * x * (1.0f + erff(x * 0.70710678118654752440f));
    case MOE_ACT_GELU_TANH: {
      const float c = 0.79788456080286535588f;
      return 0.5f * x * (1.0f + tanhf(c * (x + 0.044715f * x * x * x)));
    }
    default:  // MOE_ACT_SWISH: x * sigmoid(1.702 x)
      return x_sigmoid(x, 1.702f);
  }
}

// E8M0 scale byte for a block whose largest magnitude is amax (e4m3 target, max exponent 8),
// and the exact power-of-two multiplier 2^(127 - scale) that divides by the block scale.
__device__ __forceinline__ uint32_t mx_scale_byte(float amax) {
  int e = (int)((__float_as_uint(amax) >> 23) & 0xffu);
  int s = e - 8;
  return (uint32_t)(s < 0 ? 0 : s);
}
__device__ __forceinline__ float mx_inv_scale(uint32_t sbyte) { return __uint_as_float((254u - sbyte) << 23); }

__device__ __forceinline__ float clip448(float v) { return fminf(fmaxf(v, -448.0f), 448.0f); }

// csrc/build_blocks.hip: address of the current device's built-in scratch, looked up once per device
int build_blocks_static_setup();

}  // namespace moe
