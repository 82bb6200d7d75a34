// numeric.hpp — device-side float codecs shared by the kernels.
//
// kapy.fptofp semantics (lib/Conversion/KgpuToLLVM/ElementwiseOpToLLVM.cpp:536-661): down-casts
// round RN (ties to even) or RZ; casts to fp8 saturate to the largest finite value
// (cvt.rn.satfinite, :238-276).  fp8 is OCP: E4M3FN (bias 7, no inf, NaN 0x7F, max 448) and
// E5M2 (bias 15, IEEE-like).  A register of the elementwise interpreter stores the exactly
// decoded value as an fp32, so a codec here is "round an fp32 to the grid of the small type".
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/kapy_hip.h"

namespace kapy {

__device__ __forceinline__ uint32_t f32_bits(float x) { return __builtin_bit_cast(uint32_t, x); }
__device__ __forceinline__ float bits_f32(uint32_t u) { return __builtin_bit_cast(float, u); }

// ---- bf16 -----------------------------------------------------------------------------------
__device__ __forceinline__ float bf16_to_f32(uint16_t h) { return bits_f32((uint32_t)h << 16); }
__device__ __forceinline__ uint16_t f32_to_bf16_rn(float x) {
  uint32_t u = f32_bits(x);
  if ((u & 0x7FFFFFFFu) > 0x7F800000u) return (uint16_t)((u >> 16) | 0x0040u);  // quiet the NaN
  return (uint16_t)((u + 0x7FFFu + ((u >> 16) & 1u)) >> 16);
}
__device__ __forceinline__ uint16_t f32_to_bf16_rz(float x) {
  uint32_t u = f32_bits(x);
  if ((u & 0x7FFFFFFFu) > 0x7F800000u) return (uint16_t)((u >> 16) | 0x0040u);
  return (uint16_t)(u >> 16);
}

// two fp32 -> one 32-bit word of two bf16 / f16, round-to-nearest-even (v_cvt_pk_bf16_f32 / v_cvt_pk_f16_f32)
__device__ __forceinline__ uint32_t pack2_bf16_rn(float lo, float hi) {
  typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
  bf16x2_t h;
  h[0] = (__bf16)lo;
  h[1] = (__bf16)hi;
  return __builtin_bit_cast(uint32_t, h);
}
__device__ __forceinline__ uint32_t pack2_f16_rn(float lo, float hi) {
  typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
  half2_t h;
  h[0] = (_Float16)lo;
  h[1] = (_Float16)hi;
  return __builtin_bit_cast(uint32_t, h);
}

// ---- f16 ------------------------------------------------------------------------------------
__device__ __forceinline__ float f16_to_f32(uint16_t h) { return (float)__builtin_bit_cast(_Float16, h); }
__device__ __forceinline__ uint16_t f32_to_f16_rn(float x) { return __builtin_bit_cast(uint16_t, (_Float16)x); }

// ---- generic small-float encoder (f16 RZ, e4m3fn, e5m2) ---------------------------------------
// EB/MB: exponent/mantissa bits; BIAS; IEEE: the all-ones exponent encodes inf/NaN; SAT: overflow
// clamps to the largest finite value instead of becoming inf.
template <int EB, int MB, int BIAS, bool IEEE, bool SAT>
__device__ __forceinline__ uint32_t encode_small(float x, bool rn) {
  constexpr uint32_t kSign = 1u << (EB + MB);
  constexpr uint32_t kExpAll = ((1u << EB) - 1u) << MB;
  constexpr uint32_t kNaN = IEEE ? (kExpAll | (1u << (MB - 1))) : (kExpAll | ((1u << MB) - 1u));
  constexpr uint32_t kMax = IEEE ? (kExpAll - 1u) : (kExpAll | ((1u << MB) - 2u));
  constexpr uint32_t kInf = kExpAll;
  constexpr int kEmin = 1 - BIAS;
  const uint32_t u = f32_bits(x);
  const uint32_t sign = (u >> 31) ? kSign : 0u;
  const uint32_t a = u & 0x7FFFFFFFu;
  if (a > 0x7F800000u) return sign | kNaN;
  if (a == 0x7F800000u) return sign | ((SAT || !IEEE) ? kMax : kInf);
  const int e = (int)(a >> 23) - 127;
  uint32_t r;
  if (e < kEmin) {
    // target subnormal range: count quanta of 2^(emin - MB)
    float q = bits_f32(a) * bits_f32((uint32_t)(127 - (kEmin - MB)) << 23);
    r = (uint32_t)(rn ? __builtin_rintf(q) : __builtin_truncf(q));  // r == 2^MB encodes the smallest normal
  } else {
    constexpr int kDrop = 23 - MB;
    uint32_t t = a;
    if (rn) t += ((1u << (kDrop - 1)) - 1u) + ((a >> kDrop) & 1u);
    t >>= kDrop;                                  // (e+127) << MB | mantissa, carry already propagated
    r = t - ((uint32_t)(127 - BIAS) << MB);
  }
  if (r > kMax) r = (SAT || !IEEE || !rn) ? kMax : kInf;
  return sign | r;
}

template <int EB, int MB, int BIAS, bool IEEE>
__device__ __forceinline__ float decode_small(uint32_t b) {
  const uint32_t sign = (b >> (EB + MB)) & 1u;
  const uint32_t ef = (b >> MB) & ((1u << EB) - 1u);
  const uint32_t m = b & ((1u << MB) - 1u);
  float v;
  if (IEEE && ef == (1u << EB) - 1u) v = m ? __builtin_nanf("") : __builtin_inff();
  else if (!IEEE && ef == (1u << EB) - 1u && m == (1u << MB) - 1u) v = __builtin_nanf("");
  else if (ef == 0) v = (float)m * bits_f32((uint32_t)(127 + 1 - BIAS - MB) << 23);
  else v = bits_f32(((ef + 127 - BIAS) << 23) | (m << (23 - MB)));
  return sign ? -v : v;
}

__device__ __forceinline__ uint16_t f32_to_f16_rz(float x) { return (uint16_t)encode_small<5, 10, 15, true, false>(x, false); }
// fp8 (OCP E4M3FN / E5M2, the formats of gfx950's conversion instructions).  Round-to-nearest-even goes through
// v_cvt_pk_fp8_f32 / v_cvt_pk_bf8_f32; they turn overflow into NaN / infinity where kapy's cast saturates
// (ElementwiseOpToLLVM.cpp:577-661 clamps to the largest finite value), so everything but a NaN is clamped first.
// Round-toward-zero has no instruction and stays with the bit-level encoder.
__device__ __forceinline__ float clamp_keep_nan(float x, float bound) { return x != x ? x : __builtin_amdgcn_fmed3f(x, -bound, bound); }
__device__ __forceinline__ uint8_t f32_to_e4m3(float x, bool rn) {
  if (!rn) return (uint8_t)encode_small<4, 3, 7, false, true>(x, false);
  const float c = clamp_keep_nan(x, 448.0f);
  return (uint8_t)__builtin_amdgcn_cvt_pk_fp8_f32(c, c, 0, false);
}
__device__ __forceinline__ uint8_t f32_to_e5m2(float x, bool rn) {
  if (!rn) return (uint8_t)encode_small<5, 2, 15, true, true>(x, false);
  const float c = clamp_keep_nan(x, 57344.0f);
  return (uint8_t)__builtin_amdgcn_cvt_pk_bf8_f32(c, c, 0, false);
}
// four values to four consecutive bytes, round-to-nearest-even
__device__ __forceinline__ uint32_t pack4_e4m3_rn(float a, float b, float c, float d) {
  int w = __builtin_amdgcn_cvt_pk_fp8_f32(clamp_keep_nan(a, 448.0f), clamp_keep_nan(b, 448.0f), 0, false);
  return (uint32_t)__builtin_amdgcn_cvt_pk_fp8_f32(clamp_keep_nan(c, 448.0f), clamp_keep_nan(d, 448.0f), w, true);
}
__device__ __forceinline__ uint32_t pack4_e5m2_rn(float a, float b, float c, float d) {
  int w = __builtin_amdgcn_cvt_pk_bf8_f32(clamp_keep_nan(a, 57344.0f), clamp_keep_nan(b, 57344.0f), 0, false);
  return (uint32_t)__builtin_amdgcn_cvt_pk_bf8_f32(clamp_keep_nan(c, 57344.0f), clamp_keep_nan(d, 57344.0f), w, true);
}
__device__ __forceinline__ float e4m3_to_f32(uint8_t b) { return __builtin_amdgcn_cvt_f32_fp8((int)b, 0); }
__device__ __forceinline__ float e5m2_to_f32(uint8_t b) { return __builtin_amdgcn_cvt_f32_bf8((int)b, 0); }

// a*b + c on values of element type dtype (held as their fp32 images) with the ONE rounding fma promises.  For f16 that
// has to be the 16-bit instruction: the fp32 fma followed by the rounding to f16 rounds twice and lands on the wrong
// neighbour a few times in a million.  For bf16 (no 16-bit fma on this part) and f32 the fp32 fma serves.
__device__ __forceinline__ float fma_typed(float a, float b, float c, int dtype) {
  if (dtype == KAPY_F16) return (float)__builtin_fmaf16((_Float16)a, (_Float16)b, (_Float16)c);
  float r = __builtin_fmaf(a, b, c);
  // The fp32 result must exist as such: where a cast to f16 follows directly (straight-line compiled programs), the compiler
  // would otherwise fold it into the fma (v_fma_mixlo_f16), which rounds the exact sum once - not what fma-then-truncf means.
  asm volatile("" : "+v"(r));
  return r;
}

// Value of element `idx` of a typed buffer as an fp32 (exact for every supported type but i32).
__device__ __forceinline__ float load_as_f32(const void *p, int dtype, int64_t idx) {
  switch (dtype) {
  case KAPY_F16: return f16_to_f32(((const uint16_t *)p)[idx]);
  case KAPY_BF16: return bf16_to_f32(((const uint16_t *)p)[idx]);
  case KAPY_F32: return ((const float *)p)[idx];
  case KAPY_F8E4M3: return e4m3_to_f32(((const uint8_t *)p)[idx]);
  case KAPY_F8E5M2: return e5m2_to_f32(((const uint8_t *)p)[idx]);
  case KAPY_I8: return (float)((const int8_t *)p)[idx];
  case KAPY_I16: return (float)((const int16_t *)p)[idx];
  default: return (float)((const int32_t *)p)[idx];
  }
}

// Round an fp32 to the grid of `dtype` and return it as an fp32 again.
__device__ __forceinline__ float round_to_dtype(float v, int dtype, bool rn) {
  switch (dtype) {
  case KAPY_F16: return f16_to_f32(rn ? f32_to_f16_rn(v) : f32_to_f16_rz(v));
  case KAPY_BF16: return bf16_to_f32(rn ? f32_to_bf16_rn(v) : f32_to_bf16_rz(v));
  case KAPY_F8E4M3: return e4m3_to_f32(f32_to_e4m3(v, rn));
  case KAPY_F8E5M2: return e5m2_to_f32(f32_to_e5m2(v, rn));
  default: return v;
  }
}

// Store an fp32 that already lies on the grid of `dtype` (or must be rounded RN to it).
__device__ __forceinline__ void store_from_f32(void *p, int dtype, int64_t idx, float v) {
  switch (dtype) {
  case KAPY_F16: ((uint16_t *)p)[idx] = f32_to_f16_rn(v); break;
  case KAPY_BF16: ((uint16_t *)p)[idx] = f32_to_bf16_rn(v); break;
  case KAPY_F32: ((float *)p)[idx] = v; break;
  case KAPY_F8E4M3: ((uint8_t *)p)[idx] = f32_to_e4m3(v, true); break;
  case KAPY_F8E5M2: ((uint8_t *)p)[idx] = f32_to_e5m2(v, true); break;
  case KAPY_I8: ((int8_t *)p)[idx] = (int8_t)v; break;
  case KAPY_I16: ((int16_t *)p)[idx] = (int16_t)v; break;
  default: ((int32_t *)p)[idx] = (int32_t)v; break;
  }
}

}  // namespace kapy
