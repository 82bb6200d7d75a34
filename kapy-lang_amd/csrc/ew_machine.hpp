// ew_machine.hpp — device side of the stack machine that elementwise programs run on, shared by the
// translation units that instantiate its kernels (elementwise.hip: one vector of 8 elements per lane;
// elementwise_row.hip: whole rows resident per workgroup, for programs with a reduce).
#pragma once
#include <math.h>
#include <stdint.h>

#include "common.hpp"
#include "numeric.hpp"

namespace kapy {

constexpr int kMaxRegs = 16;
constexpr int kMaxInst = 48;
constexpr int kMaxInputs = 8;
constexpr int kMaxPost = 40;
enum PostKind { kPushIn = 100, kPushImm = 101, kCast = 102, kStore = 103, kRevSub = 104, kRevDiv = 105, kSaveTmp = 106, kPushTmp = 107, kPick = 108, kPushU = 109 };
enum InKind { kInFull = 0, kInRow = 1 /* [1 x n] */, kInCol = 2 /* [m x 1] */, kInScalar = 3 };
// bits of PostOp::slot above the slot number (row machine only)
enum SlotFlags { kSlotMask = 3, kUniformResult = 4, kUniformRight = 8, kSameOperand = 16 };  // bits 8-9: the per-row value a step names
struct PostOp {
  int16_t op, a, dtype, rmode;
  int32_t slot;  // which of the three values holds the result (and the left operand), plus SlotFlags
  float imm;
};
struct StackIn {
  const char *base;
  int64_t stride0;
  int32_t dtype, kind;
};
struct StackProgram {
  PostOp post[kMaxPost];
  StackIn in[kMaxInputs];
  char *out;
  int64_t out_stride0;
  int32_t n_post, n_ins, out_dtype, rows, vec_per_row;
  int32_t n_tmps;  // row machine only: values used more than once, parked in LDS
  int32_t width;   // elements per row when the last vector of a row is partial (ragged kernels), else 0
};

namespace {

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

// 0.5*v*(1+tanh(u)) with u = sqrt(2/pi)*(v+0.044715*v^3) equals v*sigmoid(2u) = v / (1 + 2^(-2u*log2 e)):
// no cancellation for v << 0, and only three slow-rate operations per element (exp2, rcp and
// their operand prep).  The constants fold -2*log2(e)*sqrt(2/pi) into the cubic.
__device__ __forceinline__ float gelu_tanh_f32(float v) {
  constexpr float kC1 = -2.0f * 1.4426950408889634f * 0.7978845608028654f;
  constexpr float kC3 = kC1 * 0.044715f;
  float t = v * (kC1 + kC3 * v * v);
  return v * __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(t));
}

// LEAN: without the operations whose code needs many registers (sin, cos): the register-capped 16-bit stack kernel
template <bool LEAN = false>
__device__ __forceinline__ float apply_unary(int op, float a) {
  switch (op) {
  case KAPY_EW_NEGF: return -a;
  case KAPY_EW_ABSF: return fabsf(a);
  case KAPY_EW_EXP: return expf(a);
  case KAPY_EW_EXP2: return exp2f(a);
  case KAPY_EW_LOG: return logf(a);
  case KAPY_EW_LOG2: return log2f(a);
  case KAPY_EW_SQRT: return sqrtf(a);
  case KAPY_EW_RSQRT: return 1.0f / sqrtf(a);
  case KAPY_EW_TANH: return tanhf(a);
  case KAPY_EW_ERF: return erff(a);
  case KAPY_EW_GELU_TANH: return gelu_tanh_f32(a);
  case KAPY_EW_FLOOR: return floorf(a);
  case KAPY_EW_CEIL: return ceilf(a);
  case KAPY_EW_SIN:
    if constexpr (!LEAN) return sinf(a);
    break;
  case KAPY_EW_COS:
    if constexpr (!LEAN) return cosf(a);
    break;
  }
  return a;
}

// arith.maximumf / minimumf: NaN if either operand is NaN.
__device__ __forceinline__ float max_nan(float a, float b) { return (a != a || b != b) ? __builtin_nanf("") : fmaxf(a, b); }
__device__ __forceinline__ float min_nan(float a, float b) { return (a != a || b != b) ? __builtin_nanf("") : fminf(a, b); }
// arith.maxnumf / minnumf: a NaN operand is ignored (NaN only if both are); -0 orders below +0 as above.
__device__ __forceinline__ float max_num(float a, float b) { return a != a ? b : b != b ? a : fmaxf(a, b); }
__device__ __forceinline__ float min_num(float a, float b) { return a != a ? b : b != b ? a : fminf(a, b); }
// arith.remf: a - trunc(a / b) * b computed exactly, sign of a (the frem the reference's BinaryOpConversion emits)
__device__ __forceinline__ float rem_f(float a, float b) { return fmodf(a, b); }

// One instruction of the register machines (interpreter, column machine) for one element: everything but loads, stores and
// reduces.  Register r of the lane is lane_regs[r * STRIDE]; I.dtype is the result's type (written by the host), and for the
// ops whose operand type differs from it (cmpi, the integer casts, sitofp, bitcast) the host has put the operand's type
// into I.rmode; (i, j) is the element's position (kapy.arange).
template <int STRIDE>
__device__ __forceinline__ float machine_step(const kapy_ew_inst &I, const float *lane_regs, int32_t i, int32_t j) {
  const int dt = I.dtype;
  auto R = [&](int r) { return lane_regs[r * STRIDE]; };
  switch (I.op) {
  case KAPY_EW_SPLAT: return dtype_is_int(dt) ? int_reg(int_canon(I.a, dt)) : round_to_dtype(I.imm, dt, true);
  case KAPY_EW_ARANGE: return int_reg(I.a + (I.b ? j : i));
  case KAPY_EW_FPTOFP: return round_to_dtype(R(I.a), dt, I.rmode != KAPY_RZ);
  case KAPY_EW_SELECT: return (reg_int(R(I.a)) & 1) ? R(I.b) : R(I.c);
  case KAPY_EW_CMPI: return int_reg(int_compare(I.c, reg_int(R(I.a)), reg_int(R(I.b)), I.rmode));
  case KAPY_EW_CMPF: return int_reg(float_compare(I.c, R(I.a), R(I.b)));
  case KAPY_EW_ABSI: case KAPY_EW_TRUNCI: case KAPY_EW_EXTSI: case KAPY_EW_EXTUI: case KAPY_EW_SITOFP: case KAPY_EW_FPTOSI: case KAPY_EW_BITCAST:
    return convert_reg(I.op, R(I.a), I.rmode, dt);
  default: break;
  }
  if (I.op >= KAPY_EW_ADDI && I.op <= KAPY_EW_MINUI) return int_reg(int_binary(I.op, reg_int(R(I.a)), reg_int(R(I.b)), dt));
  const float a = R(I.a);
  float r;
  switch (I.op) {
  case KAPY_EW_ADDF: r = __fadd_rn(a, R(I.b)); break;
  case KAPY_EW_SUBF: r = __fsub_rn(a, R(I.b)); break;
  case KAPY_EW_MULF: r = __fmul_rn(a, R(I.b)); break;
  case KAPY_EW_DIVF: r = __fdiv_rn(a, R(I.b)); break;
  case KAPY_EW_FMA: r = fma_typed(a, R(I.b), R(I.c), dt); break;
  case KAPY_EW_MAXIMUMF: r = max_nan(a, R(I.b)); break;
  case KAPY_EW_MINIMUMF: r = min_nan(a, R(I.b)); break;
  case KAPY_EW_MAXNUMF: r = max_num(a, R(I.b)); break;
  case KAPY_EW_MINNUMF: r = min_num(a, R(I.b)); break;
  case KAPY_EW_REMF: r = rem_f(a, R(I.b)); break;
  default: r = apply_unary(I.op, a);
  }
  return dt != KAPY_F32 ? round_to_dtype(r, dt, true) : r;
}

// ---------------------------------------------------------------------------------------------
// Stack machine: any program whose expression tree needs at most three live values, on 8
// consecutive elements per lane in registers.  The host unfolds the SSA program into postfix form
// (a value used twice is simply evaluated twice: every op is pure) and gives every step the stack
// depth it works at, so the three values are three fixed register arrays chosen by a uniform branch:
// no register is ever indexed at run time and nothing is shuffled.  Values are fp32 images of the typed value, rounded to the
// result type after every arithmetic op exactly as the register machine does.
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

__device__ __forceinline__ void widen16x8(u32x4 v, int dtype, float f[8]) {
#pragma unroll
  for (int w = 0; w < 4; ++w) {
    const uint32_t word = v[w];
    if (dtype == KAPY_BF16) {
      f[2 * w] = bits_f32(word << 16);
      f[2 * w + 1] = bits_f32(word & 0xFFFF0000u);
    } else {
      f[2 * w] = f16_to_f32((uint16_t)word);
      f[2 * w + 1] = f16_to_f32((uint16_t)(word >> 16));
    }
  }
}
// The ragged end of a row of 16-bit elements: only the first `valid` (1..7) elements of the vector at p exist; a whole
// 16-byte access would reach past the view (and possibly past its allocation), so they move one by one.
__device__ __forceinline__ u32x4 load16_partial(const char *p, int valid) {
  u32x4 v = {0, 0, 0, 0};
#pragma unroll
  for (int e = 0; e < 8; ++e)
    if (e < valid) v[e >> 1] |= (uint32_t)((const uint16_t *)p)[e] << (16 * (e & 1));
  return v;
}
__device__ __forceinline__ void store16_partial(char *p, u32x4 v, int valid) {
#pragma unroll
  for (int e = 0; e < 8; ++e)
    if (e < valid) ((uint16_t *)p)[e] = (uint16_t)(v[e >> 1] >> (16 * (e & 1)));
}

// The 8 elements of vector jv of row i of a full-extent operand, as they lie in memory (16, 32 or 8 bytes).
struct Raw8 {
  u32x4 lo, hi;
};
__device__ __forceinline__ Raw8 fetch8(const StackIn &g, int32_t i, int32_t jv, bool streaming) {
  const int eb = dtype_elem_bytes(g.dtype);
  const char *ptr = g.base + ((g.kind == kInRow ? 0 : i * g.stride0) + (int64_t)jv * 8) * eb;
  Raw8 r;
  r.lo = r.hi = u32x4{0, 0, 0, 0};
  if (eb == 2) r.lo = streaming ? __builtin_nontemporal_load((const u32x4 *)ptr) : *(const u32x4 *)ptr;
  else if (eb == 4) {
    r.lo = streaming ? __builtin_nontemporal_load((const u32x4 *)ptr) : *(const u32x4 *)ptr;
    r.hi = streaming ? __builtin_nontemporal_load((const u32x4 *)ptr + 1) : *((const u32x4 *)ptr + 1);
  } else {
    const u32x2 v = *(const u32x2 *)ptr;
    r.lo[0] = v[0];
    r.lo[1] = v[1];
  }
  return r;
}
__device__ __forceinline__ void widen8(const Raw8 &r, int dtype, float f[8]) {
  if (dtype == KAPY_F16 || dtype == KAPY_BF16) widen16x8(r.lo, dtype, f);
  else if (dtype == KAPY_I16) {  // integers: the sign-extended image in the container's bits
#pragma unroll
    for (int e = 0; e < 8; ++e) f[e] = int_reg((int32_t)(int16_t)(r.lo[e >> 1] >> (16 * (e & 1))));
  } else if (dtype == KAPY_I8 || dtype == KAPY_I1) {
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const int32_t byte = (int32_t)(int8_t)(r.lo[e >> 2] >> (8 * (e & 3)));
      f[e] = int_reg(dtype == KAPY_I1 ? (byte & 1) : byte);
    }
  } else if (dtype == KAPY_F32 || dtype == KAPY_I32) {
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const uint32_t a = r.lo[e], b = r.hi[e];
      f[e] = bits_f32(a);
      f[4 + e] = bits_f32(b);
    }
  } else {
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const uint32_t word = r.lo[e >> 2];
      const uint8_t byte = (uint8_t)(word >> (8 * (e & 3)));
      f[e] = dtype == KAPY_F8E4M3 ? e4m3_to_f32(byte) : e5m2_to_f32(byte);
    }
  }
}
template <bool NARROW>
__device__ __forceinline__ void load8(const StackIn &g, int32_t i, int32_t jv, float f[8]) {
  if (g.kind == kInCol || g.kind == kInScalar) {
    const float v = load_as_f32(g.base, g.dtype, g.kind == kInCol ? i * g.stride0 : 0);
#pragma unroll
    for (int e = 0; e < 8; ++e) f[e] = v;
    return;
  }
  if (NARROW) {
    const char *ptr = g.base + ((g.kind == kInRow ? 0 : i * g.stride0) + (int64_t)jv * 8) * 2;
    widen16x8(g.kind == kInFull ? __builtin_nontemporal_load((const u32x4 *)ptr) : *(const u32x4 *)ptr, g.dtype, f);
  } else widen8(fetch8(g, i, jv, g.kind == kInFull), g.dtype, f);
}
template <bool NARROW>
__device__ __forceinline__ void round8(float f[8], int dtype, bool rn) {
  switch (dtype) {
  case KAPY_F32: return;
  case KAPY_F16:
    if (rn) {
#pragma unroll
      for (int e = 0; e < 8; ++e) f[e] = (float)(_Float16)f[e];
    } else {
#pragma unroll
      for (int e = 0; e < 8; ++e) f[e] = f16_to_f32(f32_to_f16_rz(f[e]));
    }
    return;
  case KAPY_BF16:
    if (rn) {
#pragma unroll
      for (int e = 0; e < 8; ++e) f[e] = (float)(__bf16)f[e];
    } else {
#pragma unroll
      for (int e = 0; e < 8; ++e) f[e] = bf16_to_f32(f32_to_bf16_rz(f[e]));
    }
    return;
  default:
    if (!NARROW) {
#pragma unroll
      for (int e = 0; e < 8; ++e) f[e] = round_to_dtype(f[e], dtype, rn);
    }
  }
}
template <bool NARROW>
__device__ __forceinline__ void store8(char *out, int dtype, int64_t elem, const float f[8]) {
  if (NARROW || dtype == KAPY_F16 || dtype == KAPY_BF16) {
    u32x4 v;
#pragma unroll
    for (int w = 0; w < 4; ++w) v[w] = dtype == KAPY_F16 ? pack2_f16_rn(f[2 * w], f[2 * w + 1]) : pack2_bf16_rn(f[2 * w], f[2 * w + 1]);
    __builtin_nontemporal_store(v, (u32x4 *)(out + elem * 2));
  } else if (dtype == KAPY_I16) {
    u32x4 v;
#pragma unroll
    for (int w = 0; w < 4; ++w) v[w] = (f32_bits(f[2 * w]) & 0xFFFFu) | (f32_bits(f[2 * w + 1]) << 16);
    __builtin_nontemporal_store(v, (u32x4 *)(out + elem * 2));
  } else if (dtype == KAPY_I8 || dtype == KAPY_I1) {
    const uint32_t mask = dtype == KAPY_I1 ? 1u : 0xFFu;
    u32x2 v;
#pragma unroll
    for (int w = 0; w < 2; ++w)
      v[w] = (f32_bits(f[4 * w]) & mask) | ((f32_bits(f[4 * w + 1]) & mask) << 8) | ((f32_bits(f[4 * w + 2]) & mask) << 16) | ((f32_bits(f[4 * w + 3]) & mask) << 24);
    *(u32x2 *)(out + elem) = v;
  } else if (dtype == KAPY_F32 || dtype == KAPY_I32) {
    u32x4 lo, hi;
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      lo[e] = f32_bits(f[e]);
      hi[e] = f32_bits(f[4 + e]);
    }
    __builtin_nontemporal_store(lo, (u32x4 *)(out + elem * 4));
    __builtin_nontemporal_store(hi, (u32x4 *)(out + elem * 4) + 1);
  } else {
    u32x2 v;
    v[0] = dtype == KAPY_F8E4M3 ? pack4_e4m3_rn(f[0], f[1], f[2], f[3]) : pack4_e5m2_rn(f[0], f[1], f[2], f[3]);
    v[1] = dtype == KAPY_F8E4M3 ? pack4_e4m3_rn(f[4], f[5], f[6], f[7]) : pack4_e5m2_rn(f[4], f[5], f[6], f[7]);
    *(u32x2 *)(out + elem) = v;
  }
}

// q[e] = x[e] / y[e], correctly rounded.  When every operand of every lane is zero or of middling magnitude (2^-60 ..
// 2^60: nothing on the way can overflow or go subnormal) the quotient comes from the sequence at the core of the IEEE
// division without its scaling, special-case and mode-switching steps: the reciprocal refined once, the quotient
// corrected twice by its exact remainder.  Anything else (tiny, huge, infinite, NaN) takes the full division.
__device__ __forceinline__ void div8(const float (&x)[8], const float (&y)[8], float (&q)[8]) {
  bool plain = true;
#pragma unroll
  for (int e = 0; e < 8; ++e) {
    const float ax = fabsf(x[e]), ay = fabsf(y[e]);
    plain = plain && ay >= 0x1p-60f && ay <= 0x1p60f && ax <= 0x1p60f && (ax >= 0x1p-60f || ax == 0.f);
  }
  if (__builtin_amdgcn_ballot_w64(!plain) == 0) {
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const float r0 = __builtin_amdgcn_rcpf(y[e]);
      const float r1 = __builtin_fmaf(__builtin_fmaf(-y[e], r0, 1.0f), r0, r0);
      const float q0 = x[e] * r1;
      const float q1 = __builtin_fmaf(__builtin_fmaf(-q0, y[e], x[e]), r1, q0);
      const float q2 = __builtin_fmaf(__builtin_fmaf(-q1, y[e], x[e]), r1, q1);  // the second correction: without it one quotient in ~10^5 is an ulp off
      q[e] = x[e] == 0.f ? q0 : q2;  // a zero dividend: the corrections add a +0 remainder, which would turn a -0 quotient into +0
    }
  } else {
#pragma unroll
    for (int e = 0; e < 8; ++e) q[e] = __fdiv_rn(x[e], y[e]);
  }
}

// x[e] = op(x[e]) for a unary op whose result has element type dtype (rounding to that type is the caller's).
template <bool NARROW, bool LEAN = false>
__device__ __forceinline__ void unary8(int op, int dtype, float (&x)[8]) {
  if (NARROW && op == KAPY_EW_EXP && dtype == KAPY_F32) {
    // exp(x) = 2^hi * (1 + lo*ln2), hi + lo = x*log2(e) with lo the product's rounding error: within 2 ulp of fp32,
    // far inside the 16-bit rounding every result of a 16-bit program ends in.  2^hi is already 0 or infinite where
    // exp(x) leaves the fp32 range; infinite x would make lo inf - inf, so lo is dropped there.
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const float hi = x[e] * 1.44269504088896341f;
      float lo = __builtin_fmaf(x[e], 1.44269504088896341f, -hi);
      lo = fabsf(x[e]) < 3e38f ? lo : 0.f;
      const float pw = __builtin_amdgcn_exp2f(hi);
      x[e] = pw > 3e38f ? pw : __builtin_fmaf(pw, lo * 0.693147180559945309f, pw);
    }
    return;
  }
#pragma unroll
  for (int e = 0; e < 8; ++e) x[e] = apply_unary<LEAN>(op, x[e]);
}

// One step with its result (and left operand) in value D, the right operand in value D+1 and the
// third operand of an fma in value D+2; D is a template parameter so that no register is indexed.
// NARROW: every operand, every intermediate type and the result are f16 / bf16 / f32-from-16-bit
// (no fp8, no fp32 in memory): the common case, and it needs far fewer registers.
// LEAN: without remf, sin and cos (see apply_unary); the host sends programs that hold one of them to a build with them.
template <int D, bool NARROW, bool RAGGED = false, bool LEAN = false>
__device__ __forceinline__ void stack_step(const StackProgram &P, const PostOp &I, int32_t i, int32_t jv, float (&v)[3][8]) {
  constexpr int R = D + 1 < 3 ? D + 1 : 2, T = D + 2 < 3 ? D + 2 : 2;
  float *x = v[D];
  const float *y = v[R], *z = v[T];
  switch (I.op) {
  case kPushIn:
    if (RAGGED && NARROW && P.in[I.a].kind <= kInRow && (jv + 1) * 8 > P.width) {
      const StackIn &g = P.in[I.a];
      widen16x8(load16_partial(g.base + ((g.kind == kInRow ? 0 : i * g.stride0) + (int64_t)jv * 8) * 2, P.width - jv * 8), g.dtype, x);
      return;
    }
    load8<NARROW>(P.in[I.a], i, jv, x);
    return;
  case kPushImm: {
    const float c = round_to_dtype(I.imm, I.dtype, true);
#pragma unroll
    for (int e = 0; e < 8; ++e) x[e] = c;
    return;
  }
  case kPick:  // a copy of a value lower on the stack (I.a < D)
    if (D > 0) {
#pragma unroll
      for (int e = 0; e < 8; ++e) x[e] = (D == 2 && I.a == 1) ? v[1][e] : v[0][e];
    }
    return;
  case kStore:
    if (RAGGED && NARROW && (jv + 1) * 8 > P.width) {
      u32x4 v;
#pragma unroll
      for (int w = 0; w < 4; ++w) v[w] = P.out_dtype == KAPY_F16 ? pack2_f16_rn(x[2 * w], x[2 * w + 1]) : pack2_bf16_rn(x[2 * w], x[2 * w + 1]);
      store16_partial(P.out + ((int64_t)i * P.out_stride0 + (int64_t)jv * 8) * 2, v, P.width - jv * 8);
      return;
    }
    store8<NARROW>(P.out, P.out_dtype, (int64_t)i * P.out_stride0 + (int64_t)jv * 8, x);
    return;
  case kCast: round8<NARROW>(x, I.dtype, I.rmode != KAPY_RZ); return;
  case KAPY_EW_ADDF:
#pragma unroll
    for (int e = 0; e < 8; ++e) x[e] = __fadd_rn(x[e], y[e]);
    break;
  case KAPY_EW_SUBF:
#pragma unroll
    for (int e = 0; e < 8; ++e) x[e] = __fsub_rn(x[e], y[e]);
    break;
  case kRevSub:
#pragma unroll
    for (int e = 0; e < 8; ++e) x[e] = __fsub_rn(y[e], x[e]);
    break;
  case KAPY_EW_MULF:
#pragma unroll
    for (int e = 0; e < 8; ++e) x[e] = __fmul_rn(x[e], y[e]);
    break;
  case KAPY_EW_DIVF:
    { float a8[8], b8[8];
#pragma unroll
      for (int e = 0; e < 8; ++e) { a8[e] = x[e]; b8[e] = y[e]; }
      div8(a8, b8, *(float (*)[8])x); }
    break;
  case kRevDiv:
    { float a8[8], b8[8];
#pragma unroll
      for (int e = 0; e < 8; ++e) { a8[e] = y[e]; b8[e] = x[e]; }
      div8(a8, b8, *(float (*)[8])x); }
    break;
  case KAPY_EW_MAXIMUMF:
#pragma unroll
    for (int e = 0; e < 8; ++e) x[e] = max_nan(x[e], y[e]);
    break;
  case KAPY_EW_MINIMUMF:
#pragma unroll
    for (int e = 0; e < 8; ++e) x[e] = min_nan(x[e], y[e]);
    break;
  case KAPY_EW_MAXNUMF:
#pragma unroll
    for (int e = 0; e < 8; ++e) x[e] = max_num(x[e], y[e]);
    break;
  case KAPY_EW_MINNUMF:
#pragma unroll
    for (int e = 0; e < 8; ++e) x[e] = min_num(x[e], y[e]);
    break;
  case KAPY_EW_REMF:
    if constexpr (!LEAN) {
#pragma unroll
      for (int e = 0; e < 8; ++e) x[e] = rem_f(x[e], y[e]);
    }
    break;
  case KAPY_EW_FMA:
#pragma unroll
    for (int e = 0; e < 8; ++e) x[e] = fma_typed(x[e], y[e], z[e], I.dtype);
    break;
  default: unary8<NARROW, LEAN>(I.op, I.dtype, *(float (*)[8])x);
  }
  if (I.dtype != KAPY_F32) round8<NARROW>(x, I.dtype, true);
}

template <bool NARROW, bool RAGGED = false, bool LEAN = false>
__device__ __forceinline__ void stack_run(const StackProgram &P) {
  const int64_t slot = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (slot >= (int64_t)P.rows * P.vec_per_row) return;
  const int32_t i = (int32_t)(slot / P.vec_per_row), jv = (int32_t)(slot - (int64_t)i * P.vec_per_row);
  float v[3][8];
#pragma unroll
  for (int d = 0; d < 3; ++d)
#pragma unroll
    for (int e = 0; e < 8; ++e) v[d][e] = 0.f;
  for (int pc = 0; pc < P.n_post; ++pc) {
    const PostOp I = P.post[pc];
    switch (I.slot) {
    case 0: stack_step<0, NARROW, RAGGED, LEAN>(P, I, i, jv, v); break;
    case 1: stack_step<1, NARROW, RAGGED, LEAN>(P, I, i, jv, v); break;
    default: stack_step<2, NARROW, RAGGED, LEAN>(P, I, i, jv, v);
    }
  }
}

}  // namespace
}  // namespace kapy
