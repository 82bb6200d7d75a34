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

// ---- integer registers.  A signless iN value travels in the 32 bits of the machines' fp32 container as its sign-extended
// image (i1: 0 or 1); nothing but moves, LDS and these helpers ever touches such a container, so the bits survive.
__device__ __forceinline__ int32_t reg_int(float x) { return __builtin_bit_cast(int32_t, x); }
__device__ __forceinline__ float int_reg(int32_t v) { return __builtin_bit_cast(float, v); }
__device__ __forceinline__ bool dtype_is_int(int dtype) { return dtype == KAPY_I8 || dtype == KAPY_I16 || dtype == KAPY_I32 || dtype == KAPY_I1; }
__device__ __forceinline__ int int_width(int dtype) { return dtype == KAPY_I1 ? 1 : dtype == KAPY_I8 ? 8 : dtype == KAPY_I16 ? 16 : 32; }
// the canonical image of the low bits of v
__device__ __forceinline__ int32_t int_canon(int32_t v, int dtype) {
  return dtype == KAPY_I1 ? (v & 1) : dtype == KAPY_I8 ? (int32_t)(int8_t)v : dtype == KAPY_I16 ? (int32_t)(int16_t)v : v;
}
// the value read as a signed / as an unsigned number of its width
__device__ __forceinline__ int32_t int_signed(int32_t v, int dtype) { return dtype == KAPY_I1 ? -(v & 1) : v; }
__device__ __forceinline__ uint32_t int_unsigned(int32_t v, int dtype) {
  return dtype == KAPY_I1 ? (uint32_t)(v & 1) : dtype == KAPY_I8 ? (uint32_t)(uint8_t)v : dtype == KAPY_I16 ? (uint32_t)(uint16_t)v : (uint32_t)v;
}

// arith.addi ... minui on two values of integer type dtype (BinaryOpConversion, ElementwiseOpToLLVM.cpp:1178-1206): wrapping
// arithmetic; what MLIR leaves undefined is defined here (x / 0 = 0, x % 0 = 0, min / -1 wraps with remainder 0, shifts by
// the width or more give 0, shrsi the sign).
__device__ __forceinline__ int32_t int_binary(int op, int32_t av, int32_t bv, int dtype) {
  const int32_t a = int_signed(av, dtype), b = int_signed(bv, dtype);
  const uint32_t ua = int_unsigned(av, dtype), ub = int_unsigned(bv, dtype);
  const uint32_t width = (uint32_t)int_width(dtype);
  uint32_t r = 0;
  switch (op) {
  case KAPY_EW_ADDI: r = ua + ub; break;
  case KAPY_EW_SUBI: r = ua - ub; break;
  case KAPY_EW_MULI: r = ua * ub; break;
  case KAPY_EW_DIVSI: r = b == 0 ? 0u : b == -1 ? 0u - ua : (uint32_t)(a / b); break;
  case KAPY_EW_DIVUI: r = ub == 0 ? 0u : ua / ub; break;
  case KAPY_EW_FLOORDIVSI:
    if (b == 0) r = 0;
    else if (b == -1) r = 0u - ua;
    else {
      const int32_t q = a / b;
      r = (uint32_t)(q - ((a % b != 0 && ((a < 0) != (b < 0))) ? 1 : 0));
    }
    break;
  case KAPY_EW_CEILDIVSI:
    if (b == 0) r = 0;
    else if (b == -1) r = 0u - ua;
    else {
      const int32_t q = a / b;
      r = (uint32_t)(q + ((a % b != 0 && ((a < 0) == (b < 0))) ? 1 : 0));
    }
    break;
  case KAPY_EW_CEILDIVUI: r = (ub == 0 || ua == 0) ? 0u : (ua - 1) / ub + 1; break;
  case KAPY_EW_REMSI: r = (b == 0 || b == -1) ? 0u : (uint32_t)(a % b); break;
  case KAPY_EW_REMUI: r = ub == 0 ? 0u : ua % ub; break;
  case KAPY_EW_ANDI: r = ua & ub; break;
  case KAPY_EW_ORI: r = ua | ub; break;
  case KAPY_EW_XORI: r = ua ^ ub; break;
  case KAPY_EW_SHLI: r = ub >= width ? 0u : ua << ub; break;
  case KAPY_EW_SHRUI: r = ub >= width ? 0u : ua >> ub; break;
  case KAPY_EW_SHRSI: r = (uint32_t)(a >> (ub >= width ? width - 1 : ub)); break;
  case KAPY_EW_MAXSI: r = (uint32_t)(a > b ? a : b); break;
  case KAPY_EW_MINSI: r = (uint32_t)(a < b ? a : b); break;
  case KAPY_EW_MAXUI: r = ua > ub ? ua : ub; break;
  case KAPY_EW_MINUI: r = ua < ub ? ua : ub; break;
  }
  return int_canon((int32_t)r, dtype);
}
// arith.cmpi with MLIR's predicate numbers
__device__ __forceinline__ int32_t int_compare(int pred, int32_t av, int32_t bv, int dtype) {
  const int32_t a = int_signed(av, dtype), b = int_signed(bv, dtype);
  const uint32_t ua = int_unsigned(av, dtype), ub = int_unsigned(bv, dtype);
  switch (pred) {
  case KAPY_CMPI_EQ: return ua == ub;
  case KAPY_CMPI_NE: return ua != ub;
  case KAPY_CMPI_SLT: return a < b;
  case KAPY_CMPI_SLE: return a <= b;
  case KAPY_CMPI_SGT: return a > b;
  case KAPY_CMPI_SGE: return a >= b;
  case KAPY_CMPI_ULT: return ua < ub;
  case KAPY_CMPI_ULE: return ua <= ub;
  case KAPY_CMPI_UGT: return ua > ub;
  default: return ua >= ub;
  }
}
// arith.cmpf: the ordered predicates are false, the unordered ones true, when an operand is NaN
__device__ __forceinline__ int32_t float_compare(int pred, float a, float b) {
  const bool uno = a != a || b != b;
  switch (pred) {
  case KAPY_CMPF_FALSE: return 0;
  case KAPY_CMPF_OEQ: return a == b;
  case KAPY_CMPF_OGT: return a > b;
  case KAPY_CMPF_OGE: return a >= b;
  case KAPY_CMPF_OLT: return a < b;
  case KAPY_CMPF_OLE: return a <= b;
  case KAPY_CMPF_ONE: return !uno && a != b;
  case KAPY_CMPF_ORD: return !uno;
  case KAPY_CMPF_UEQ: return uno || a == b;
  case KAPY_CMPF_UGT: return uno || a > b;
  case KAPY_CMPF_UGE: return uno || a >= b;
  case KAPY_CMPF_ULT: return uno || a < b;
  case KAPY_CMPF_ULE: return uno || a <= b;
  case KAPY_CMPF_UNE: return uno || a != b;
  case KAPY_CMPF_UNO: return uno;
  default: return 1;
  }
}
// arith.sitofp: one rounding to nearest even from the integer.  f32: the conversion instruction; f16: through f32 (any
// integer the f32 rounding touches, |v| >= 2^24, is beyond f16's range and becomes infinity either way); bf16: rounded
// from the integer's own bits (through f32 a value could be rounded twice).  Returns the fp32 image.
__device__ __forceinline__ float int_to_float(int32_t v, int dtype) {
  if (dtype == KAPY_F32) return (float)v;
  if (dtype == KAPY_F16) return f16_to_f32(f32_to_f16_rn((float)v));
  if (v == 0) return 0.f;
  const uint32_t sign = v < 0 ? 0x80000000u : 0u, mag = v < 0 ? 0u - (uint32_t)v : (uint32_t)v;
  const int lz = __builtin_clz(mag);
  const uint32_t m = mag << lz;                   // bit 31 is the leading one
  uint32_t keep = m >> 24;                        // 1.7 bits of a bf16 significand
  const uint32_t rest = m & 0x00FFFFFFu;
  int exponent = 31 - lz;
  if (rest > 0x00800000u || (rest == 0x00800000u && (keep & 1))) {
    if (++keep == 0x100u) { keep = 0x80u; ++exponent; }
  }
  return bits_f32(sign | ((uint32_t)(exponent + 127) << 23) | ((keep & 0x7Fu) << 16));
}
// arith.fptosi: toward zero; saturating, NaN -> 0 (where MLIR leaves the result undefined), then wrapped to the width
__device__ __forceinline__ int32_t float_to_int(float x, int dtype) {
  const int32_t v = x != x ? 0 : x >= 2147483648.f ? 0x7FFFFFFF : x <= -2147483648.f ? (int32_t)0x80000000u : (int32_t)x;
  return int_canon(v, dtype);
}
// arith.bitcast between a float type and the integer type of its width (containers: fp32 image / sign-extended image)
__device__ __forceinline__ float bitcast_reg(float x, int from, int to) {
  if (from == to || (dtype_is_int(from) && dtype_is_int(to))) return x;
  if (dtype_is_int(to)) {  // float -> int
    switch (from) {
    case KAPY_F32: return x;
    case KAPY_F16: return int_reg((int32_t)(int16_t)f32_to_f16_rn(x));
    case KAPY_BF16: return int_reg((int32_t)(int16_t)f32_to_bf16_rn(x));
    case KAPY_F8E4M3: return int_reg((int32_t)(int8_t)f32_to_e4m3(x, true));
    default: return int_reg((int32_t)(int8_t)f32_to_e5m2(x, true));
    }
  }
  const int32_t v = reg_int(x);
  switch (to) {
  case KAPY_F32: return x;
  case KAPY_F16: return f16_to_f32((uint16_t)v);
  case KAPY_BF16: return bf16_to_f32((uint16_t)v);
  case KAPY_F8E4M3: return e4m3_to_f32((uint8_t)v);
  default: return e5m2_to_f32((uint8_t)v);
  }
}

// The conversions with one operand whose result type differs from (or, absi, equals) the operand's: math.absi, arith.trunci /
// extsi / extui, sitofp, fptosi, bitcast, on containers (x of type `from`, the result of type `to`).
__device__ __forceinline__ float convert_reg(int op, float x, int from, int to) {
  switch (op) {
  case KAPY_EW_ABSI: {
    const int32_t v = int_signed(reg_int(x), to);
    return int_reg(int_canon(v < 0 ? (int32_t)(0u - (uint32_t)v) : v, to));
  }
  case KAPY_EW_TRUNCI: return int_reg(int_canon(reg_int(x), to));
  case KAPY_EW_EXTSI: return int_reg(int_canon(int_signed(reg_int(x), from), to));
  case KAPY_EW_EXTUI: return int_reg(int_canon((int32_t)int_unsigned(reg_int(x), from), to));
  case KAPY_EW_SITOFP: return int_to_float(int_signed(reg_int(x), from), to);
  case KAPY_EW_FPTOSI: return int_reg(float_to_int(x, to));
  default: return bitcast_reg(x, from, to);
  }
}
__device__ __forceinline__ int dtype_elem_bytes(int dtype) {
  return (dtype == KAPY_F32 || dtype == KAPY_I32) ? 4 : (dtype == KAPY_F16 || dtype == KAPY_BF16 || dtype == KAPY_I16) ? 2 : 1;
}

// Value of element `idx` of a typed buffer in the machines' container: the fp32 image of a float, the sign-extended image
// (in the container's bits) of an integer.
__device__ __forceinline__ float load_as_f32(const void *p, int dtype, int64_t idx) {
  switch (dtype) {
  case KAPY_F16: return f16_to_f32(((const uint16_t *)p)[idx]);
  case KAPY_BF16: return bf16_to_f32(((const uint16_t *)p)[idx]);
  case KAPY_F32: return ((const float *)p)[idx];
  case KAPY_F8E4M3: return e4m3_to_f32(((const uint8_t *)p)[idx]);
  case KAPY_F8E5M2: return e5m2_to_f32(((const uint8_t *)p)[idx]);
  case KAPY_I8: return int_reg((int32_t)((const int8_t *)p)[idx]);
  case KAPY_I16: return int_reg((int32_t)((const int16_t *)p)[idx]);
  case KAPY_I1: return int_reg((int32_t)(((const uint8_t *)p)[idx] & 1));
  default: return int_reg(((const int32_t *)p)[idx]);
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
  case KAPY_I8: ((int8_t *)p)[idx] = (int8_t)reg_int(v); break;
  case KAPY_I16: ((int16_t *)p)[idx] = (int16_t)reg_int(v); break;
  case KAPY_I1: ((uint8_t *)p)[idx] = (uint8_t)(reg_int(v) & 1); break;
  default: ((int32_t *)p)[idx] = reg_int(v); break;
  }
}

}  // namespace kapy
