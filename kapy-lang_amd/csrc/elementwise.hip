// elementwise.hip — fused elementwise programs over whole views.
//
// Reference: the per-lane, per-element application of arith/math ops by
// lib/Conversion/KgpuToLLVM/ElementwiseOpToLLVM.cpp (generic conversion :424-534, fptofp
// :536-661, bf16 single-rounding arithmetic :771-892, exp :1039-1073, extern-lib calls
// :1100-1166) fed by ld_global / broadcast / splat and drained by st_global.  In the reference
// a fused chain is one straight-line kernel body; here the host recognises the common chain
//     out = cast( act( x * splat(scale) + bias ) )
// and runs it in one pass with 16-byte accesses (affine_act_kernel); any other program runs on a
// small register machine (interpreter_kernel) whose register file lives in LDS.
#include <math.h>
#include <string.h>

#include <type_traits>
#include <vector>

#include "common.hpp"
#include <functional>
#include "numeric.hpp"

namespace kapy {
namespace {

constexpr int kMaxRegs = 16;
constexpr int kMaxInst = 48;
constexpr int kMaxInputs = 8;

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

struct DevView {
  const char *base;  // address of view element (0,0)
  int64_t stride0, stride1;
  int32_t ext0, ext1;
  int32_t dtype;
  uint32_t pad;
};

struct Program {
  kapy_ew_inst inst[kMaxInst];
  int32_t n_inst;
  int32_t n_ins;
  DevView in[kMaxInputs];
  DevView out;
};

// 0.5*v*(1+tanh(u)) with u = sqrt(2/pi)*(v+0.044715*v^3) equals v*sigmoid(2u) = v / (1 + 2^(-2u*log2 e)):
// no cancellation for v << 0, and only three slow-rate operations per element (exp2, rcp and
// their operand prep).  The constants fold -2*log2(e)*sqrt(2/pi) into the cubic.
__device__ __forceinline__ float gelu_tanh_f32(float v) {
  constexpr float kC1 = -2.0f * 1.4426950408889634f * 0.7978845608028654f;
  constexpr float kC3 = kC1 * 0.044715f;
  float t = v * (kC1 + kC3 * v * v);
  return v * __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(t));
}

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
  }
  return a;
}

// arith.maximumf / minimumf: NaN if either operand is NaN.
__device__ __forceinline__ float max_nan(float a, float b) { return (a != a || b != b) ? __builtin_nanf("") : fmaxf(a, b); }
__device__ __forceinline__ float min_nan(float a, float b) { return (a != a || b != b) ? __builtin_nanf("") : fminf(a, b); }

// ---------------------------------------------------------------------------------------------
// Register machine: one output element per lane per pass; register r of lane t is regs[r][t], so
// every access is conflict-free.  Values are fp32 images of the register's dtype.
__global__ __launch_bounds__(256) void interpreter_kernel(Program P, int j_fastest) {
  __shared__ float regs[kMaxRegs][256];
  const int tid = threadIdx.x;
  const int64_t total = (int64_t)P.out.ext0 * P.out.ext1;
  const int64_t t = (int64_t)blockIdx.x * 256 + tid;
  const bool active = t < total;
  int32_t i = 0, j = 0;
  if (active) {
    if (j_fastest) { i = (int32_t)(t / P.out.ext1); j = (int32_t)(t - (int64_t)i * P.out.ext1); }
    else { j = (int32_t)(t / P.out.ext0); i = (int32_t)(t - (int64_t)j * P.out.ext0); }
  }
  // The host has written every instruction's result dtype into I.dtype.
  for (int k = 0; k < P.n_inst; ++k) {
    const kapy_ew_inst I = P.inst[k];
    float r = 0.f;
    const int dt = I.dtype;
    switch (I.op) {
    case KAPY_EW_LD_GLOBAL: {
      const DevView &g = P.in[I.a];
      int32_t gi = g.ext0 == 1 ? 0 : i, gj = g.ext1 == 1 ? 0 : j;
      if (active && gi < g.ext0 && gj < g.ext1) r = load_as_f32(g.base, g.dtype, gi * g.stride0 + gj * g.stride1);
      else {
        uint32_t w = I.c == KAPY_PAD_ZERO ? 0u : g.pad;
        r = load_as_f32(&w, g.dtype, 0);
      }
      break;
    }
    case KAPY_EW_SPLAT:
      r = round_to_dtype(I.imm, dt, true);
      break;
    case KAPY_EW_FPTOFP:
      r = round_to_dtype(regs[I.a][tid], dt, I.rmode != KAPY_RZ);
      break;
    case KAPY_EW_ST_GLOBAL:
      if (active) store_from_f32((void *)P.out.base, P.out.dtype, i * P.out.stride0 + j * P.out.stride1, regs[I.a][tid]);
      continue;
    default: {
      const float a = regs[I.a][tid];
      switch (I.op) {
      case KAPY_EW_ADDF: r = __fadd_rn(a, regs[I.b][tid]); break;
      case KAPY_EW_SUBF: r = __fsub_rn(a, regs[I.b][tid]); break;
      case KAPY_EW_MULF: r = __fmul_rn(a, regs[I.b][tid]); break;
      case KAPY_EW_DIVF: r = __fdiv_rn(a, regs[I.b][tid]); break;
      case KAPY_EW_FMA: r = __fmaf_rn(a, regs[I.b][tid], regs[I.c][tid]); break;
      case KAPY_EW_MAXIMUMF: r = max_nan(a, regs[I.b][tid]); break;
      case KAPY_EW_MINIMUMF: r = min_nan(a, regs[I.b][tid]); break;
      default: r = apply_unary(I.op, a);
      }
      if (dt != KAPY_F32) r = round_to_dtype(r, dt, true);
    }
    }
    regs[I.dst][tid] = r;  // regs[*][tid] is private to the lane: no barrier needed
  }
}

// ---------------------------------------------------------------------------------------------
// Stack machine: any program whose expression tree needs at most three live values, on 8
// consecutive elements per lane in registers.  The host unfolds the SSA program into postfix form
// (a value used twice is simply evaluated twice: every op is pure) and gives every step the stack
// depth it works at, so the three values are three fixed register arrays chosen by a uniform branch:
// no register is ever indexed at run time and nothing is shuffled.  Values are fp32 images of the typed value, rounded to the
// result type after every arithmetic op exactly as the register machine does.
constexpr int kMaxPost = 40;
enum PostKind { kPushIn = 100, kPushImm = 101, kCast = 102, kStore = 103, kRevSub = 104, kRevDiv = 105, kSaveTmp = 106, kPushTmp = 107, kPick = 108 };
enum InKind { kInFull = 0, kInRow = 1 /* [1 x n] */, kInCol = 2 /* [m x 1] */, kInScalar = 3 };
struct PostOp {
  int16_t op, a, dtype, rmode;
  int32_t slot;  // which of the three values holds the result (and the left operand)
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
};
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
// The 8 elements of vector jv of row i of a full-extent operand, as they lie in memory (16, 32 or 8 bytes).
struct Raw8 {
  u32x4 lo, hi;
};
__device__ __forceinline__ Raw8 fetch8(const StackIn &g, int32_t i, int32_t jv, bool streaming) {
  const int eb = g.dtype == KAPY_F32 ? 4 : (g.dtype == KAPY_F16 || g.dtype == KAPY_BF16) ? 2 : 1;
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
  else if (dtype == KAPY_F32) {
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
  } else if (dtype == KAPY_F32) {
    u32x4 lo, hi;
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      lo[e] = f32_bits(f[e]);
      hi[e] = f32_bits(f[4 + e]);
    }
    __builtin_nontemporal_store(lo, (u32x4 *)(out + elem * 4));
    __builtin_nontemporal_store(hi, (u32x4 *)(out + elem * 4) + 1);
  } else {
    u32x2 v = {0, 0};
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const uint32_t byte = dtype == KAPY_F8E4M3 ? f32_to_e4m3(f[e], true) : f32_to_e5m2(f[e], true);
      v[e >> 2] |= byte << (8 * (e & 3));
    }
    *(u32x2 *)(out + elem) = v;
  }
}

// One step with its result (and left operand) in value D, the right operand in value D+1 and the
// third operand of an fma in value D+2; D is a template parameter so that no register is indexed.
// NARROW: every operand, every intermediate type and the result are f16 / bf16 / f32-from-16-bit
// (no fp8, no fp32 in memory): the common case, and it needs far fewer registers.
template <int D, bool NARROW>
__device__ __forceinline__ void stack_step(const StackProgram &P, const PostOp &I, int32_t i, int32_t jv, float (&v)[3][8]) {
  constexpr int R = D + 1 < 3 ? D + 1 : 2, T = D + 2 < 3 ? D + 2 : 2;
  float *x = v[D];
  const float *y = v[R], *z = v[T];
  switch (I.op) {
  case kPushIn: load8<NARROW>(P.in[I.a], i, jv, x); return;
  case kPushImm: {
    const float c = round_to_dtype(I.imm, I.dtype, true);
#pragma unroll
    for (int e = 0; e < 8; ++e) x[e] = c;
    return;
  }
  case kStore: store8<NARROW>(P.out, P.out_dtype, (int64_t)i * P.out_stride0 + (int64_t)jv * 8, x); return;
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
#pragma unroll
    for (int e = 0; e < 8; ++e) x[e] = __fdiv_rn(x[e], y[e]);
    break;
  case kRevDiv:
#pragma unroll
    for (int e = 0; e < 8; ++e) x[e] = __fdiv_rn(y[e], x[e]);
    break;
  case KAPY_EW_MAXIMUMF:
#pragma unroll
    for (int e = 0; e < 8; ++e) x[e] = max_nan(x[e], y[e]);
    break;
  case KAPY_EW_MINIMUMF:
#pragma unroll
    for (int e = 0; e < 8; ++e) x[e] = min_nan(x[e], y[e]);
    break;
  case KAPY_EW_FMA:
#pragma unroll
    for (int e = 0; e < 8; ++e) x[e] = __fmaf_rn(x[e], y[e], z[e]);
    break;
  default:
#pragma unroll
    for (int e = 0; e < 8; ++e) x[e] = apply_unary(I.op, x[e]);
  }
  if (I.dtype != KAPY_F32) round8<NARROW>(x, I.dtype, true);
}

template <bool NARROW>
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
    case 0: stack_step<0, NARROW>(P, I, i, jv, v); break;
    case 1: stack_step<1, NARROW>(P, I, i, jv, v); break;
    default: stack_step<2, NARROW>(P, I, i, jv, v);
    }
  }
}

// Throughput of this kernel follows the number of resident waves (each lane walks its program one
// dependent step at a time), so the 16-bit-only form is held to 64 registers: 8 waves per SIMD.
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(8, 8))) void stack_kernel_narrow(StackProgram P) { stack_run<true>(P); }
__global__ __launch_bounds__(256) void stack_kernel_any(StackProgram P) { stack_run<false>(P); }

// ---------------------------------------------------------------------------------------------
// Row machine: programs with a reduce along the rows (softmax, layer norm ...).  A workgroup owns
// one row and keeps it on chip for the whole program, so HBM sees one read of every operand and one
// write of the result.  Lane t holds CH chunks of 8 elements, chunk c at vector c*THREADS + t of the
// row; a step of the stack machine runs on every chunk; a reduce folds the lane's chunks, then the
// wave with a butterfly of bpermutes, then the workgroup's waves through LDS, and leaves the result
// in every element.  Values needed more than once are parked in LDS as fp32 and read back by the
// lane that wrote them.
template <int KIND>
__device__ __forceinline__ float fold(float a, float b) { return KIND == 0 ? a + b : max_nan(a, b); }

template <int D, int CH, int THREADS, bool NARROW>
__device__ __forceinline__ void row_step(const StackProgram &P, const PostOp &I, int32_t i, int pc, float (&v)[CH][3][8], float *lds) {
  const int tid = threadIdx.x;
  constexpr int WAVES = THREADS / 64;
  if (I.op == KAPY_EW_REDUCE_SUM || I.op == KAPY_EW_REDUCE_MAX) {
    const bool sum = I.op == KAPY_EW_REDUCE_SUM;
    float acc = sum ? 0.f : -__builtin_inff();
#pragma unroll
    for (int c = 0; c < CH; ++c) {
      if (c * THREADS + tid < P.vec_per_row) {
        float part;
        if (sum) part = ((v[c][D][0] + v[c][D][1]) + (v[c][D][2] + v[c][D][3])) + ((v[c][D][4] + v[c][D][5]) + (v[c][D][6] + v[c][D][7]));
        else part = max_nan(max_nan(max_nan(v[c][D][0], v[c][D][1]), max_nan(v[c][D][2], v[c][D][3])),
                            max_nan(max_nan(v[c][D][4], v[c][D][5]), max_nan(v[c][D][6], v[c][D][7])));
        acc = sum ? acc + part : max_nan(acc, part);
      }
    }
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) {
      const float other = __shfl_xor(acc, off, 64);
      acc = sum ? acc + other : max_nan(acc, other);
    }
    if (WAVES > 1) {
      // the exchange area alternates with the step's parity, so that a wave still reading the previous
      // reduce's partials cannot meet the next reduce's writes: one barrier per reduce
      float *red = lds + (pc & 1) * WAVES;
      if ((tid & 63) == 0) red[tid >> 6] = acc;
      __syncthreads();
      acc = red[0];
#pragma unroll
      for (int w = 1; w < WAVES; ++w) acc = sum ? acc + red[w] : max_nan(acc, red[w]);
    }
    acc = round_to_dtype(acc, I.dtype, true);
#pragma unroll
    for (int c = 0; c < CH; ++c)
#pragma unroll
      for (int e = 0; e < 8; ++e) v[c][D][e] = acc;
    return;
  }
  if (I.op == kPick) {  // a copy of a value lower on the stack (I.a < D)
    if (D > 0) {
#pragma unroll
      for (int c = 0; c < CH; ++c)
#pragma unroll
        for (int e = 0; e < 8; ++e) v[c][D][e] = (D == 2 && I.a == 1) ? v[c][1][e] : v[c][0][e];
    }
    return;
  }
  float *tmps = lds + 32;
#pragma unroll
  for (int c = 0; c < CH; ++c) {
    const int32_t jv = c * THREADS + tid;
    const bool active = jv < P.vec_per_row;
    if (I.op == kSaveTmp || I.op == kPushTmp) {
      float4 *slot = (float4 *)(tmps + ((int64_t)I.a * P.vec_per_row + jv) * 8);
      if (active) {
        if (I.op == kSaveTmp) {
          slot[0] = float4{v[c][D][0], v[c][D][1], v[c][D][2], v[c][D][3]};
          slot[1] = float4{v[c][D][4], v[c][D][5], v[c][D][6], v[c][D][7]};
        } else {
          const float4 lo = slot[0], hi = slot[1];
          v[c][D][0] = lo.x; v[c][D][1] = lo.y; v[c][D][2] = lo.z; v[c][D][3] = lo.w;
          v[c][D][4] = hi.x; v[c][D][5] = hi.y; v[c][D][6] = hi.z; v[c][D][7] = hi.w;
        }
      }
    } else if (I.op == kPushIn || I.op == kStore) {
      if (active) stack_step<D, NARROW>(P, I, i, jv, v[c]);
    } else stack_step<D, NARROW>(P, I, i, jv, v[c]);
  }
}

template <int CH, int THREADS, bool NARROW>
__global__ __launch_bounds__(THREADS) void row_kernel(StackProgram P) {
  extern __shared__ float row_lds[];
  const int32_t i = blockIdx.x;
  float v[CH][3][8];
#pragma unroll
  for (int c = 0; c < CH; ++c)
#pragma unroll
    for (int d = 0; d < 3; ++d)
#pragma unroll
      for (int e = 0; e < 8; ++e) v[c][d][e] = 0.f;
  for (int pc = 0; pc < P.n_post; ++pc) {
    const PostOp I = P.post[pc];
    switch (I.slot) {
    case 0: row_step<0, CH, THREADS, NARROW>(P, I, i, pc, v, row_lds); break;
    case 1: row_step<1, CH, THREADS, NARROW>(P, I, i, pc, v, row_lds); break;
    default: row_step<2, CH, THREADS, NARROW>(P, I, i, pc, v, row_lds);
    }
  }
}

template <bool NARROW>
int launch_row_kernel(const StackProgram &P, hipStream_t s) {
  const int vpr = P.vec_per_row;
  // few chunks per lane keep the three values of the stack within 64 to 128 registers; long rows take 1024 lanes
  const int threads = vpr <= 64 ? 64 : vpr <= 512 ? 256 : 1024;
  const int ch = (vpr + threads - 1) / threads;
  const size_t lds = (32 + (size_t)P.n_tmps * vpr * 8) * sizeof(float);  // 32 floats: the reduce exchange of up to 16 waves, twice
  if (lds > 160 * 1024) return fail(KAPY_ERR_UNSUPPORTED, "elementwise: the program keeps %d row values of %d elements alive, more than fits the LDS", P.n_tmps, vpr * 8);
  dim3 grid((unsigned)P.rows);
#define KAPY_ROW(CH_, TH_)                                                                                         \
  do {                                                                                                             \
    if (lds > 48 * 1024) KAPY_HIP_CHECK(hipFuncSetAttribute((const void *)row_kernel<CH_, TH_, NARROW>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds)); \
    row_kernel<CH_, TH_, NARROW><<<grid, TH_, lds, s>>>(P);                                                        \
  } while (0)
  if (threads == 64) KAPY_ROW(1, 64);
  else if (threads == 256) { if (ch == 1) KAPY_ROW(1, 256); else KAPY_ROW(2, 256); }
  else { if (ch == 1) KAPY_ROW(1, 1024); else if (ch == 2) KAPY_ROW(2, 1024); else KAPY_ROW(4, 1024); }
#undef KAPY_ROW
  KAPY_HIP_CHECK(hipGetLastError());
  return KAPY_OK;
}

// ---------------------------------------------------------------------------------------------
// out[i,j] = cast_out( act( f32(x[i,j]) * scale + f32(bias) ) ), x/out contiguous along j.
enum BiasMode { kNoBias = 0, kBiasRow = 1 /* bias[0,j] */, kBiasCol = 2 /* bias[i,0] */, kBiasFull = 3 };

struct AffineActParams {
  const char *x, *bias;
  char *out;
  int64_t x_stride0, out_stride0, bias_stride0;  // elements
  int32_t rows, vec_per_row;
  int32_t has_scale, bias_mode, act;  // act: a unary kapy_ew_op, or -1
  float scale;
};

// Two 16-bit elements of a 32-bit word <-> two fp32.  For f16 the widening is left as a plain cast
// so that the compiler can fold it into v_fma_mix_f32 (conversion + multiply + add in one
// instruction), and the narrowing pairs up into v_cvt_pk_f16_f32; bf16 widens with a shift and
// narrows with v_cvt_pk_bf16_f32.  All narrowing is round-to-nearest-even.
typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
struct Bf16Tag {};
template <typename T> struct Pair;
template <> struct Pair<_Float16> {
  static __device__ __forceinline__ void widen(uint32_t word, float &lo, float &hi) {
    half2_t h = __builtin_bit_cast(half2_t, word);
    lo = (float)h[0];
    hi = (float)h[1];
  }
  static __device__ __forceinline__ uint32_t narrow(float lo, float hi) {
    half2_t h;
    h[0] = (_Float16)lo;
    h[1] = (_Float16)hi;
    return __builtin_bit_cast(uint32_t, h);
  }
};
template <> struct Pair<Bf16Tag> {
  static __device__ __forceinline__ void widen(uint32_t word, float &lo, float &hi) {
    lo = bits_f32(word << 16);
    hi = bits_f32(word & 0xFFFF0000u);
  }
  static __device__ __forceinline__ uint32_t narrow(float lo, float hi) {
    bf16x2_t h;
    h[0] = (__bf16)lo;
    h[1] = (__bf16)hi;
    return __builtin_bit_cast(uint32_t, h);
  }
};

template <typename T>
__device__ __forceinline__ void unpack8(u32x4 v, float f[8]) {
#pragma unroll
  for (int w = 0; w < 4; ++w) {
    const uint32_t word = v[w];  // bit_cast needs a scalar object, not a vector-element lvalue
    Pair<T>::widen(word, f[2 * w], f[2 * w + 1]);
  }
}
template <typename T>
__device__ __forceinline__ u32x4 pack8(const float f[8]) {
  u32x4 v;
#pragma unroll
  for (int w = 0; w < 4; ++w) v[w] = Pair<T>::narrow(f[2 * w], f[2 * w + 1]);
  return v;
}

// One element of the fused chain.  x*scale + bias is written as a plain expression: the compiler
// may contract it into one FMA (for f16 inputs the mixed-precision v_fma_mix_f32), i.e. one
// rounding where mulf-then-addf has two; the difference is at most half an ulp of fp32, five
// orders of magnitude inside the 2-ulp tolerance of the 16-bit result.
template <int ACT>
__device__ __forceinline__ float affine_act(float x, float scale, float bias, int act) {
  float v = x * scale + bias;
  if (ACT == KAPY_EW_GELU_TANH) return gelu_tanh_f32(v);
  if (ACT >= 0) return apply_unary(act, v);
  return v;
}

// 16-bit in, 16-bit out (same type), 8 elements per 16-byte vector, UNROLL vectors per lane.
#ifndef KAPY_EW_UNROLL
#define KAPY_EW_UNROLL 2
#endif
#ifndef KAPY_EW_NT
#define KAPY_EW_NT 1
#endif
template <typename T, int ACT>
__global__ __launch_bounds__(256) void affine_act_kernel(AffineActParams p) {
  constexpr int UNROLL = KAPY_EW_UNROLL;
  const uint32_t total = (uint32_t)p.rows * (uint32_t)p.vec_per_row;
  const uint32_t first = blockIdx.x * (256 * UNROLL) + threadIdx.x;
  const float scale = p.has_scale ? p.scale : 1.0f;
  u32x4 xv[UNROLL], bv[UNROLL];
  int32_t row[UNROLL], col[UNROLL];
#pragma unroll
  for (int u = 0; u < UNROLL; ++u) {
    uint32_t slot = first + u * 256;
    row[u] = -1;
    if (slot < total) {
      row[u] = (int32_t)(slot / (uint32_t)p.vec_per_row);
      col[u] = (int32_t)(slot - (uint32_t)row[u] * (uint32_t)p.vec_per_row) * 8;
      const u32x4 *xp = (const u32x4 *)(p.x + ((int64_t)row[u] * p.x_stride0 + col[u]) * 2);
      xv[u] = KAPY_EW_NT ? __builtin_nontemporal_load(xp) : *xp;
      if (p.bias_mode == kBiasRow) bv[u] = *(const u32x4 *)(p.bias + (int64_t)col[u] * 2);
      else if (p.bias_mode == kBiasFull) bv[u] = *(const u32x4 *)(p.bias + ((int64_t)row[u] * p.bias_stride0 + col[u]) * 2);
      else if (p.bias_mode == kBiasCol) {
        uint32_t h = *(const uint16_t *)(p.bias + (int64_t)row[u] * p.bias_stride0 * 2);
        h |= h << 16;
        bv[u] = u32x4{h, h, h, h};
      }
    }
  }
#pragma unroll
  for (int u = 0; u < UNROLL; ++u) {
    if (row[u] < 0) continue;
    float f[8], b[8];
    unpack8<T>(xv[u], f);
    if (p.bias_mode != kNoBias) unpack8<T>(bv[u], b);
#pragma unroll
    for (int e = 0; e < 8; ++e) f[e] = affine_act<ACT>(f[e], scale, p.bias_mode != kNoBias ? b[e] : 0.f, p.act);
    u32x4 *op = (u32x4 *)(p.out + ((int64_t)row[u] * p.out_stride0 + col[u]) * 2);
    if (KAPY_EW_NT) __builtin_nontemporal_store(pack8<T>(f), op);
    else *op = pack8<T>(f);
  }
}

// Same chain when the bias is broadcast along rows (bias[0, j]) or absent: a lane keeps one
// 8-column chunk and walks ROWS consecutive rows, so its bias vector is fetched and widened once
// and no index division is needed.  Grid: x over column chunks, y over groups of ROWS rows.
#ifndef KAPY_EW_ROWS
#define KAPY_EW_ROWS 2
#endif
template <typename T, int ACT>
__global__ __launch_bounds__(256) void affine_act_cols_kernel(AffineActParams p) {
  constexpr int ROWS = KAPY_EW_ROWS;
  const int32_t chunk = blockIdx.x * 256 + threadIdx.x;
  if (chunk >= p.vec_per_row) return;
  const int32_t col = chunk * 8, row0 = blockIdx.y * ROWS;
  const float scale = p.has_scale ? p.scale : 1.0f;
  float b[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
  if (p.bias_mode == kBiasRow) unpack8<T>(*(const u32x4 *)(p.bias + (int64_t)col * 2), b);
  u32x4 xv[ROWS];
#pragma unroll
  for (int u = 0; u < ROWS; ++u)
    if (row0 + u < p.rows) {
      const u32x4 *xp = (const u32x4 *)(p.x + ((int64_t)(row0 + u) * p.x_stride0 + col) * 2);
      xv[u] = KAPY_EW_NT ? __builtin_nontemporal_load(xp) : *xp;
    }
#pragma unroll
  for (int u = 0; u < ROWS; ++u) {
    if (row0 + u >= p.rows) break;
    float f[8];
    unpack8<T>(xv[u], f);
#pragma unroll
    for (int e = 0; e < 8; ++e) f[e] = affine_act<ACT>(f[e], scale, b[e], p.act);
    u32x4 *op = (u32x4 *)(p.out + ((int64_t)(row0 + u) * p.out_stride0 + col) * 2);
    if (KAPY_EW_NT) __builtin_nontemporal_store(pack8<T>(f), op);
    else *op = pack8<T>(f);
  }
}

// ---------------------------------------------------------------------------------------------
// Host side: verification (the op verifiers of the reference), pattern matching, launch.
struct Node {
  int kind;  // kapy_ew_op
  int a = -1, b = -1, c = -1;
  int dtype = -1, rmode = KAPY_RN, input = -1;
  float imm = 0.f;
};

int verify_program(const kapy_ew_inst *prog, int n_inst, const kapy_global *const *ins, int n_ins, const kapy_global *out,
                   int result_dtype[kMaxInst]) {
  if (!prog || n_inst <= 0) return fail(KAPY_ERR_INVALID, "elementwise: empty program");
  if (n_inst > kMaxInst) return fail(KAPY_ERR_UNSUPPORTED, "elementwise: more than %d instructions", kMaxInst);
  if (n_ins < 0 || n_ins > kMaxInputs) return fail(KAPY_ERR_UNSUPPORTED, "elementwise: more than %d inputs", kMaxInputs);
  int rc = check_global(out, "elementwise result");
  if (rc) return rc;
  for (int k = 0; k < n_ins; ++k) {
    if (!ins || (rc = check_global(ins[k], "elementwise operand"))) return rc ? rc : fail(KAPY_ERR_INVALID, "elementwise: null operand list");
    if (ins[k]->start0 < 0 || ins[k]->start1 < 0) return fail(KAPY_ERR_INVALID, "elementwise: negative view start");
  }
  if (out->start0 < 0 || out->start1 < 0) return fail(KAPY_ERR_INVALID, "elementwise: negative view start");
  int reg_dtype[kMaxRegs];
  for (int r = 0; r < kMaxRegs; ++r) reg_dtype[r] = -1;
  const int64_t o0 = extent0(out), o1 = extent1(out);
  bool has_store = false;
  auto reg_ok = [&](int r) { return r >= 0 && r < kMaxRegs && reg_dtype[r] >= 0; };
  for (int k = 0; k < n_inst; ++k) {
    const kapy_ew_inst &I = prog[k];
    if (I.op < 0 || I.op >= KAPY_EW_NUM_OPS) return fail(KAPY_ERR_INVALID, "elementwise: unknown op %d at %d", I.op, k);
    if (I.op != KAPY_EW_ST_GLOBAL && (I.dst < 0 || I.dst >= kMaxRegs))
      return fail(KAPY_ERR_INVALID, "elementwise: result register out of range at %d", k);
    switch (I.op) {
    case KAPY_EW_LD_GLOBAL: {
      if (I.a < 0 || I.a >= n_ins) return fail(KAPY_ERR_INVALID, "elementwise: ld_global of unknown operand at %d", k);
      if (I.c < 0 || I.c > 3) return fail(KAPY_ERR_INVALID, "elementwise: unknown padding option at %d", k);
      int64_t e0 = extent0(ins[I.a]), e1 = extent1(ins[I.a]);
      if ((e0 != o0 && e0 != 1) || (e1 != o1 && e1 != 1))
        return fail(KAPY_ERR_VERIFY, "broadcast: source shape must be 1 on the axes it is broadcast along");
      reg_dtype[I.dst] = ins[I.a]->dtype;
      break;
    }
    case KAPY_EW_SPLAT:
      if (I.dtype != KAPY_F16 && I.dtype != KAPY_BF16 && I.dtype != KAPY_F32)
        return fail(KAPY_ERR_VERIFY, "splat: only f16, bf16 and f32 splats are supported");
      reg_dtype[I.dst] = I.dtype;
      break;
    case KAPY_EW_FPTOFP: {
      if (!reg_ok(I.a)) return fail(KAPY_ERR_INVALID, "elementwise: use of undefined register at %d", k);
      int sd = reg_dtype[I.a], dd = I.dtype;
      if (!is_float(sd) || !is_float(dd)) return fail(KAPY_ERR_VERIFY, "fptofp: operands must have float element type");
      bool down = dtype_bytes(dd) < dtype_bytes(sd);
      if (down && I.rmode != KAPY_RN && I.rmode != KAPY_RZ) return fail(KAPY_ERR_VERIFY, "fptofp: rounding mode is required for down cast");
      if (sd == KAPY_BF16 && is_f8(dd) && I.rmode == KAPY_RZ)
        return fail(KAPY_ERR_VERIFY, "fptofp: unsupported rounding mode when convert bf16 to f8");
      if (is_f8(sd) && is_f8(dd)) return fail(KAPY_ERR_VERIFY, "fptofp: convert f8 to f8 is not supported");
      reg_dtype[I.dst] = dd;
      break;
    }
    case KAPY_EW_FMA:
      if (!reg_ok(I.a) || !reg_ok(I.b) || !reg_ok(I.c)) return fail(KAPY_ERR_INVALID, "elementwise: use of undefined register at %d", k);
      if (reg_dtype[I.a] != reg_dtype[I.b] || reg_dtype[I.a] != reg_dtype[I.c])
        return fail(KAPY_ERR_VERIFY, "elementwise: operands must have the same element type at %d", k);
      reg_dtype[I.dst] = reg_dtype[I.a];
      break;
    case KAPY_EW_ADDF: case KAPY_EW_SUBF: case KAPY_EW_MULF: case KAPY_EW_DIVF: case KAPY_EW_MAXIMUMF: case KAPY_EW_MINIMUMF:
      if (!reg_ok(I.a) || !reg_ok(I.b)) return fail(KAPY_ERR_INVALID, "elementwise: use of undefined register at %d", k);
      if (reg_dtype[I.a] != reg_dtype[I.b])
        return fail(KAPY_ERR_VERIFY, "elementwise: operands must have the same element type at %d", k);
      reg_dtype[I.dst] = reg_dtype[I.a];
      break;
    case KAPY_EW_ST_GLOBAL:
      if (!reg_ok(I.a)) return fail(KAPY_ERR_INVALID, "elementwise: use of undefined register at %d", k);
      if (reg_dtype[I.a] != out->dtype) return fail(KAPY_ERR_VERIFY, "st_global: source and target must have the same element type");
      has_store = true;
      break;
    case KAPY_EW_REDUCE_SUM: case KAPY_EW_REDUCE_MAX:
      if (!reg_ok(I.a)) return fail(KAPY_ERR_INVALID, "elementwise: use of undefined register at %d", k);
      if (I.b != 0 && I.b != 1) return fail(KAPY_ERR_VERIFY, "reduce: axis must be 0 or 1");
      reg_dtype[I.dst] = reg_dtype[I.a];
      break;
    default:
      if (!reg_ok(I.a)) return fail(KAPY_ERR_INVALID, "elementwise: use of undefined register at %d", k);
      reg_dtype[I.dst] = reg_dtype[I.a];
    }
    if (result_dtype) result_dtype[k] = I.op == KAPY_EW_ST_GLOBAL ? out->dtype : reg_dtype[I.dst];
    if (I.op != KAPY_EW_ST_GLOBAL && I.op != KAPY_EW_LD_GLOBAL && I.op != KAPY_EW_FPTOFP) {
      int d = reg_dtype[I.dst];
      if (d != KAPY_F16 && d != KAPY_BF16 && d != KAPY_F32)
        return fail(KAPY_ERR_VERIFY, "elementwise: arithmetic needs f16, bf16 or f32 operands at %d", k);
    }
  }
  if (!has_store) return fail(KAPY_ERR_INVALID, "elementwise: program has no st_global");
  return KAPY_OK;
}

uint32_t padding_word_of(int32_t dtype, int32_t padding);

// Symbolic evaluation into a DAG, then a structural match of
//   st( fptofp_rn[T]( act?( addf( mulf(extf(ld x), splat s), extf(ld bias) ) ) ) )   (operands in either order;
//   the scale and the bias optional; fma(x, s, bias) is NOT matched: it rounds once, mulf+addf twice).
bool match_affine_act(const kapy_ew_inst *prog, int n_inst, const kapy_global *const *ins, const kapy_global *out,
                      AffineActParams *p, int *elem_dtype) {
  std::vector<Node> nodes;
  int reg[kMaxRegs];
  for (int r = 0; r < kMaxRegs; ++r) reg[r] = -1;
  int stored = -1, n_store = 0;
  for (int k = 0; k < n_inst; ++k) {
    const kapy_ew_inst &I = prog[k];
    Node n;
    n.kind = I.op;
    switch (I.op) {
    case KAPY_EW_LD_GLOBAL: n.input = I.a; if (I.c != KAPY_PAD_ZERO) return false; break;
    case KAPY_EW_SPLAT: n.imm = I.imm; n.dtype = I.dtype; break;
    case KAPY_EW_FPTOFP: n.a = reg[I.a]; n.dtype = I.dtype; n.rmode = I.rmode; break;
    case KAPY_EW_ST_GLOBAL: stored = reg[I.a]; ++n_store; continue;
    case KAPY_EW_FMA: n.a = reg[I.a]; n.b = reg[I.b]; n.c = reg[I.c]; break;
    case KAPY_EW_ADDF: case KAPY_EW_SUBF: case KAPY_EW_MULF: case KAPY_EW_DIVF: case KAPY_EW_MAXIMUMF: case KAPY_EW_MINIMUMF:
      n.a = reg[I.a]; n.b = reg[I.b]; break;
    default: n.a = reg[I.a];
    }
    nodes.push_back(n);
    reg[I.dst] = (int)nodes.size() - 1;
  }
  if (n_store != 1 || stored < 0) return false;
  const int T = out->dtype;
  if (T != KAPY_F16 && T != KAPY_BF16) return false;
  auto is_kind = [&](int id, int kind) { return id >= 0 && nodes[id].kind == kind; };
  // x: extf(ld in) with in of the output's type and full extent
  auto as_input_f32 = [&](int id) -> int {
    if (!is_kind(id, KAPY_EW_FPTOFP) || nodes[id].dtype != KAPY_F32) return -1;
    int s = nodes[id].a;
    return is_kind(s, KAPY_EW_LD_GLOBAL) ? nodes[s].input : -1;
  };
  auto as_splat_f32 = [&](int id, float *v) {
    if (!is_kind(id, KAPY_EW_SPLAT) || nodes[id].dtype != KAPY_F32) return false;
    *v = nodes[id].imm;
    return true;
  };
  int cur = stored;
  if (!is_kind(cur, KAPY_EW_FPTOFP) || nodes[cur].dtype != T || nodes[cur].rmode != KAPY_RN) return false;
  cur = nodes[cur].a;
  if (cur < 0) return false;
  p->act = -1;
  int k = nodes[cur].kind;
  if (k >= KAPY_EW_NEGF && k <= KAPY_EW_GELU_TANH) {
    p->act = k;
    cur = nodes[cur].a;
    if (cur < 0) return false;
  }
  int x_in = -1, bias_in = -1;
  p->has_scale = 0;
  p->scale = 1.f;
  auto match_scaled = [&](int id) -> int {  // mulf(x, s) | mulf(s, x) | x
    if (is_kind(id, KAPY_EW_MULF)) {
      float s;
      int xa = as_input_f32(nodes[id].a), xb = as_input_f32(nodes[id].b);
      if (xa >= 0 && as_splat_f32(nodes[id].b, &s)) { p->has_scale = 1; p->scale = s; return xa; }
      if (xb >= 0 && as_splat_f32(nodes[id].a, &s)) { p->has_scale = 1; p->scale = s; return xb; }
      return -1;
    }
    return as_input_f32(id);
  };
  if (is_kind(cur, KAPY_EW_ADDF)) {
    int l = nodes[cur].a, r = nodes[cur].b;
    int xl = match_scaled(l);
    if (xl >= 0 && as_input_f32(r) >= 0) { x_in = xl; bias_in = as_input_f32(r); }
    else {
      p->has_scale = 0;
      int xr = match_scaled(r);
      if (xr >= 0 && as_input_f32(l) >= 0) { x_in = xr; bias_in = as_input_f32(l); }
      else return false;
    }
  } else {
    x_in = match_scaled(cur);
    if (x_in < 0) return false;
  }
  const kapy_global *x = ins[x_in];
  if (x->dtype != T || x->stride1 != 1 || out->stride1 != 1) return false;
  const int64_t o0 = extent0(out), o1 = extent1(out);
  if (extent0(x) != o0 || extent1(x) != o1 || o1 % 8 != 0) return false;
  if (vector_bytes(x, 1) != 16 || vector_bytes(out, 1) != 16) return false;
  if (o0 * (o1 / 8) >= (int64_t(1) << 31) - 1024) return false;
  p->bias_mode = kNoBias;
  p->bias = nullptr;
  p->bias_stride0 = 0;
  if (bias_in >= 0) {
    const kapy_global *b = ins[bias_in];
    if (b->dtype != T) return false;
    int64_t b0 = extent0(b), b1 = extent1(b);
    if (b1 == o1 && b->stride1 == 1 && vector_bytes(b, 1) == 16) p->bias_mode = (b0 == 1 && o0 != 1) ? kBiasRow : kBiasFull;
    else if (b1 == 1 && o1 != 1 && b0 == o0) p->bias_mode = kBiasCol;
    else return false;
    p->bias = view_base(b);
    p->bias_stride0 = b->stride0;
  }
  p->x = view_base(x);
  p->out = (char *)view_base(out);
  p->x_stride0 = x->stride0;
  p->out_stride0 = out->stride0;
  p->rows = (int32_t)o0;
  p->vec_per_row = (int32_t)(o1 / 8);
  *elem_dtype = T;
  return true;
}

// does any ld_global of input `input` ask for a padding pattern other than zero?
bool prog_padding_nonzero(const kapy_ew_inst *prog, int n_inst, int input) {
  for (int k = 0; k < n_inst; ++k)
    if (prog[k].op == KAPY_EW_LD_GLOBAL && prog[k].a == input && prog[k].c != KAPY_PAD_ZERO) return true;
  return false;
}
// Postfix form of the program for the stack machine; false when the program does not fit it
// (a tree deeper than three values, more than kMaxPost steps after unfolding shared values,
// operands that are not full / row / column / scalar views readable 8 at a time, padding).
bool build_stack_program(const kapy_ew_inst *prog, int n_inst, const int *result_dtype, const kapy_global *const *ins, int n_ins,
                         const kapy_global *out, StackProgram *P, bool row_mode = false) {
  struct N {
    int op, a = -1, b = -1, c = -1, dtype = -1, rmode = KAPY_RN, input = -1;
    float imm = 0.f;
  };
  std::vector<N> nodes;
  int reg[kMaxRegs];
  for (int r = 0; r < kMaxRegs; ++r) reg[r] = -1;
  int stored = -1, n_store = 0;
  for (int k = 0; k < n_inst; ++k) {
    const kapy_ew_inst &I = prog[k];
    N n;
    n.op = I.op;
    n.dtype = result_dtype[k];
    n.rmode = I.rmode;
    n.imm = I.imm;
    switch (I.op) {
    case KAPY_EW_LD_GLOBAL: n.input = I.a; break;
    case KAPY_EW_SPLAT: break;
    case KAPY_EW_ST_GLOBAL: stored = reg[I.a]; ++n_store; continue;
    case KAPY_EW_FMA: n.a = reg[I.a]; n.b = reg[I.b]; n.c = reg[I.c]; break;
    case KAPY_EW_ADDF: case KAPY_EW_SUBF: case KAPY_EW_MULF: case KAPY_EW_DIVF: case KAPY_EW_MAXIMUMF: case KAPY_EW_MINIMUMF:
      n.a = reg[I.a]; n.b = reg[I.b]; break;
    default: n.a = reg[I.a];
    }
    nodes.push_back(n);
    reg[I.dst] = (int)nodes.size() - 1;
  }
  if (n_store != 1 || stored < 0) return false;
  // a reduce needs the row machine, and there only along the rows
  for (const N &n : nodes)
    if (n.op == KAPY_EW_REDUCE_SUM || n.op == KAPY_EW_REDUCE_MAX)
      if (!row_mode) return false;
  if (row_mode)
    for (int k = 0; k < n_inst; ++k)
      if ((prog[k].op == KAPY_EW_REDUCE_SUM || prog[k].op == KAPY_EW_REDUCE_MAX) && prog[k].b != 1) return false;
  // the result: rows contiguous, 8 elements at a time
  const int64_t o0 = extent0(out), o1 = extent1(out);
  const int ob = dtype_bytes(out->dtype);
  if (!is_float(out->dtype) || out->stride1 != 1 || o1 % 8 != 0 || ((uintptr_t)view_base(out) % (8 * ob)) || (out->stride0 * ob) % (8 * ob)) return false;
  if (o0 * (o1 / 8) >= (int64_t(1) << 31) - 1024) return false;
  if (row_mode && o1 / 8 > 4096) return false;
  for (int k = 0; k < n_ins; ++k) {
    const kapy_global *g = ins[k];
    StackIn &in = P->in[k];
    in.base = view_base(g);
    in.stride0 = g->stride0;
    in.dtype = g->dtype;
    if (!is_float(g->dtype)) return false;
    const int64_t e0 = extent0(g), e1 = extent1(g);
    const int eb = dtype_bytes(g->dtype);
    const bool vec_ok = g->stride1 == 1 && ((uintptr_t)in.base % (8 * eb)) == 0 && (g->stride0 * eb) % (8 * eb) == 0;
    if (e0 == o0 && e1 == o1 && vec_ok) in.kind = kInFull;
    else if (e0 == 1 && e1 == o1 && vec_ok) in.kind = kInRow;
    else if (e1 == 1 && e0 == o0) in.kind = kInCol;
    else if (e0 == 1 && e1 == 1) in.kind = kInScalar;
    else return false;
  }
  // depth of the stack an expression needs when the deeper operand is evaluated first
  std::vector<int> need(nodes.size(), 0);
  for (size_t id = 0; id < nodes.size(); ++id) {
    const N &n = nodes[id];
    if (n.op == KAPY_EW_LD_GLOBAL || n.op == KAPY_EW_SPLAT) need[id] = 1;
    else if (n.op == KAPY_EW_FMA) need[id] = std::max(need[n.a], std::max(need[n.b] + 1, need[n.c] + 2));
    else if (n.b >= 0) need[id] = std::min(std::max(need[n.a], need[n.b] + 1), std::max(need[n.b], need[n.a] + 1));
    else need[id] = need[n.a];
  }
  if (need[stored] > 3) return false;
  // row machine: a value with several uses is computed once.  A later use that finds the value still on the
  // stack below it copies it from there (kPick); one that does not reads it back from LDS, where the first
  // evaluation parked it.  A first run of the emission finds out which values are ever read back.
  std::vector<int> uses(nodes.size(), 0), tmp_of(nodes.size(), -1);
  std::vector<char> parked(nodes.size(), 0), read_back(nodes.size(), 0);
  int n_tmps = 0;
  if (row_mode) {
    std::vector<char> reached(nodes.size(), 0);
    std::function<void(int)> visit = [&](int id) {
      ++uses[id];
      if (reached[id]) return;
      reached[id] = 1;
      const N &n = nodes[id];
      if (n.a >= 0) visit(n.a);
      if (n.b >= 0) visit(n.b);
      if (n.c >= 0) visit(n.c);
    };
    visit(stored);
  }
  int count = 0;
  bool ok = true, dry = row_mode;
  int holder[3] = {-1, -1, -1};  // which node's value each stack slot holds
  auto push = [&](int op, int a, int dtype, int rmode, int slot, float imm) {
    if (count >= kMaxPost || slot > 2) { ok = false; return; }
    P->post[count++] = PostOp{(int16_t)op, (int16_t)a, (int16_t)dtype, (int16_t)rmode, slot, imm};
  };
  // evaluate node id into value d (values d+1, d+2 are free to use)
  std::function<void(int, int)> emit_node;
  std::function<void(int, int)> emit = [&](int id, int d) {
    if (!ok) return;
    if (d > 2) { ok = false; return; }
    const bool shared_value = row_mode && uses[id] > 1 && nodes[id].op != KAPY_EW_SPLAT;
    if (shared_value) {
      for (int below = 0; below < d; ++below)
        if (holder[below] == id) {
          push(kPick, below, nodes[id].dtype, 0, d, 0.f);
          holder[d] = id;
          return;
        }
      if (parked[id]) {
        read_back[id] = 1;
        if (!dry) push(kPushTmp, tmp_of[id], nodes[id].dtype, 0, d, 0.f);
        else push(kPushTmp, 0, nodes[id].dtype, 0, d, 0.f);
        holder[d] = id;
        return;
      }
    }
    emit_node(id, d);
    if (d + 1 < 3) holder[d + 1] = -1;
    if (d + 2 < 3) holder[d + 2] = -1;
    holder[d] = id;
    if (shared_value) {
      parked[id] = 1;
      if (dry || tmp_of[id] >= 0) push(kSaveTmp, dry ? 0 : tmp_of[id], nodes[id].dtype, 0, d, 0.f);
    }
  };
  emit_node = [&](int id, int d) {
    if (!ok) return;
    const N &n = nodes[id];
    switch (n.op) {
    case KAPY_EW_LD_GLOBAL:
      if (prog_padding_nonzero(prog, n_inst, n.input)) { ok = false; return; }
      push(kPushIn, n.input, n.dtype, 0, d, 0.f);
      return;
    case KAPY_EW_SPLAT: push(kPushImm, 0, n.dtype, 0, d, n.imm); return;
    case KAPY_EW_FPTOFP: emit(n.a, d); push(kCast, 0, n.dtype, n.rmode, d, 0.f); return;
    case KAPY_EW_FMA: emit(n.a, d); emit(n.b, d + 1); emit(n.c, d + 2); push(KAPY_EW_FMA, 0, n.dtype, 0, d, 0.f); return;
    case KAPY_EW_ADDF: case KAPY_EW_SUBF: case KAPY_EW_MULF: case KAPY_EW_DIVF: case KAPY_EW_MAXIMUMF: case KAPY_EW_MINIMUMF: {
      const bool a_first = std::max(need[n.a], need[n.b] + 1) <= std::max(need[n.b], need[n.a] + 1);
      if (a_first) { emit(n.a, d); emit(n.b, d + 1); push(n.op, 0, n.dtype, 0, d, 0.f); }
      else {
        emit(n.b, d); emit(n.a, d + 1);
        push(n.op == KAPY_EW_SUBF ? kRevSub : n.op == KAPY_EW_DIVF ? kRevDiv : n.op, 0, n.dtype, 0, d, 0.f);
      }
      return;
    }
    default: emit(n.a, d); push(n.op, 0, n.dtype, 0, d, 0.f);
    }
  };
  emit(stored, 0);
  push(kStore, 0, out->dtype, 0, 0, 0.f);
  if (!ok) return false;
  if (row_mode) {  // again, parking only what the first run read back
    for (size_t id = 0; id < nodes.size(); ++id)
      if (read_back[id]) tmp_of[id] = n_tmps++;
    count = 0;
    dry = false;
    std::fill(parked.begin(), parked.end(), 0);
    holder[0] = holder[1] = holder[2] = -1;
    emit(stored, 0);
    push(kStore, 0, out->dtype, 0, 0, 0.f);
    if (!ok) return false;
  }
  P->n_post = count;
  P->n_ins = n_ins;
  P->out = (char *)view_base(out);
  P->out_stride0 = out->stride0;
  P->out_dtype = out->dtype;
  P->rows = (int32_t)o0;
  P->vec_per_row = (int32_t)(o1 / 8);
  P->n_tmps = n_tmps;
  return true;
}

uint32_t padding_word_of(int32_t dtype, int32_t padding) {
  static const uint32_t f32[4] = {0, 0x7FC00000u, 0x7F800000u, 0xFF800000u};
  static const uint32_t f16[4] = {0, 0x7E00u, 0x7C00u, 0xFC00u};
  static const uint32_t bf16[4] = {0, 0x7FC0u, 0x7F80u, 0xFF80u};
  static const uint32_t e4m3[4] = {0, 0x7Fu, 0x7Eu, 0xFEu};
  static const uint32_t e5m2[4] = {0, 0x7Eu, 0x7Cu, 0xFCu};
  switch (dtype) {
  case KAPY_F32: return f32[padding];
  case KAPY_F16: return f16[padding];
  case KAPY_BF16: return bf16[padding];
  case KAPY_F8E4M3: return e4m3[padding];
  case KAPY_F8E5M2: return e5m2[padding];
  }
  return 0;
}

DevView to_dev(const kapy_global *g) {
  DevView v;
  v.base = view_base(g);
  v.stride0 = g->stride0;
  v.stride1 = g->stride1;
  v.ext0 = (int32_t)extent0(g);
  v.ext1 = (int32_t)extent1(g);
  v.dtype = g->dtype;
  v.pad = 0;
  return v;
}

}  // namespace
}  // namespace kapy

using namespace kapy;

extern "C" {

int kapy_elementwise(const kapy_ew_inst *prog, int32_t n_inst, const kapy_global *const *ins, int32_t n_ins,
                     const kapy_global *out, void *stream) {
  int result_dtype[kMaxInst];
  int rc = verify_program(prog, n_inst, ins, n_ins, out, result_dtype);
  if (rc) return rc;
  rc = ensure_device();
  if (rc) return rc;
  const int64_t o0 = extent0(out), o1 = extent1(out);
  if (o0 <= 0 || o1 <= 0) return KAPY_OK;
  hipStream_t s = (hipStream_t)stream;

  bool has_reduce = false;
  for (int k = 0; k < n_inst; ++k) has_reduce |= prog[k].op == KAPY_EW_REDUCE_SUM || prog[k].op == KAPY_EW_REDUCE_MAX;
  if (has_reduce) {
    StackProgram SP;
    memset(&SP, 0, sizeof SP);
    if (!build_stack_program(prog, n_inst, result_dtype, ins, n_ins, out, &SP, true))
      return fail(KAPY_ERR_UNSUPPORTED, "elementwise: a program with a reduce needs axis 1, contiguous rows of a multiple of 8 and at most 32768 "
                                        "elements, zero padding, full / row / column / scalar operands and at most three values in flight");
    bool narrow = out->dtype == KAPY_F16 || out->dtype == KAPY_BF16;
    for (int k = 0; k < n_ins; ++k) narrow = narrow && (ins[k]->dtype == KAPY_F16 || ins[k]->dtype == KAPY_BF16);
    for (int k = 0; k < n_inst; ++k) narrow = narrow && !is_f8(result_dtype[k]);
    return narrow ? launch_row_kernel<true>(SP, s) : launch_row_kernel<false>(SP, s);
  }

  AffineActParams ap;
  int T = -1;
  if (match_affine_act(prog, n_inst, ins, out, &ap, &T)) {
    uint32_t slots = (uint32_t)ap.rows * (uint32_t)ap.vec_per_row;
    const bool cols = (ap.bias_mode == kBiasRow || ap.bias_mode == kNoBias) && (ap.rows + KAPY_EW_ROWS - 1) / KAPY_EW_ROWS <= 65535;
    dim3 grid = cols ? dim3((ap.vec_per_row + 255) / 256, (ap.rows + KAPY_EW_ROWS - 1) / KAPY_EW_ROWS)
                     : dim3((slots + 256 * KAPY_EW_UNROLL - 1) / (256 * KAPY_EW_UNROLL));
#define KAPY_LAUNCH_AFFINE(TT, AA)                                                     \
  do {                                                                                 \
    if (cols) affine_act_cols_kernel<TT, AA><<<grid, 256, 0, s>>>(ap);                 \
    else affine_act_kernel<TT, AA><<<grid, 256, 0, s>>>(ap);                           \
  } while (0)
    if (T == KAPY_F16) {
      if (ap.act == KAPY_EW_GELU_TANH) KAPY_LAUNCH_AFFINE(_Float16, KAPY_EW_GELU_TANH);
      else if (ap.act < 0) KAPY_LAUNCH_AFFINE(_Float16, -1);
      else KAPY_LAUNCH_AFFINE(_Float16, 0);
    } else {
      if (ap.act == KAPY_EW_GELU_TANH) KAPY_LAUNCH_AFFINE(Bf16Tag, KAPY_EW_GELU_TANH);
      else if (ap.act < 0) KAPY_LAUNCH_AFFINE(Bf16Tag, -1);
      else KAPY_LAUNCH_AFFINE(Bf16Tag, 0);
    }
#undef KAPY_LAUNCH_AFFINE
    KAPY_HIP_CHECK(hipGetLastError());
    return KAPY_OK;
  }

  {
    StackProgram SP;
    memset(&SP, 0, sizeof SP);
    if (build_stack_program(prog, n_inst, result_dtype, ins, n_ins, out, &SP)) {
      const int64_t slots = (int64_t)SP.rows * SP.vec_per_row;
      bool narrow = out->dtype == KAPY_F16 || out->dtype == KAPY_BF16;
      for (int k = 0; k < n_ins; ++k) narrow = narrow && (ins[k]->dtype == KAPY_F16 || ins[k]->dtype == KAPY_BF16);
      for (int k = 0; k < n_inst; ++k) narrow = narrow && !is_f8(result_dtype[k]);
      if (narrow) stack_kernel_narrow<<<dim3((unsigned)((slots + 255) / 256)), 256, 0, s>>>(SP);
      else stack_kernel_any<<<dim3((unsigned)((slots + 255) / 256)), 256, 0, s>>>(SP);
      KAPY_HIP_CHECK(hipGetLastError());
      return KAPY_OK;
    }
  }

  Program P;
  memset(&P, 0, sizeof P);
  P.n_inst = n_inst;
  P.n_ins = n_ins;
  for (int k = 0; k < n_inst; ++k) {
    P.inst[k] = prog[k];
    P.inst[k].dtype = result_dtype[k];
  }
  for (int k = 0; k < n_ins; ++k) P.in[k] = to_dev(ins[k]);
  // padding pattern per input: taken from the (single) ld_global that names it
  for (int k = 0; k < n_inst; ++k)
    if (prog[k].op == KAPY_EW_LD_GLOBAL) P.in[prog[k].a].pad = padding_word_of(ins[prog[k].a]->dtype, prog[k].c);
  P.out = to_dev(out);
  int64_t total = o0 * o1;
  int j_fastest = out->stride1 <= out->stride0;
  dim3 grid((unsigned)((total + 255) / 256));
  interpreter_kernel<<<grid, 256, 0, s>>>(P, j_fastest);
  KAPY_HIP_CHECK(hipGetLastError());
  return KAPY_OK;
}

int kapy_fptofp(const kapy_global *src, const kapy_global *dst, int32_t rmode, void *stream) {
  int rc = check_global(src, "fptofp source");
  if (!rc) rc = check_global(dst, "fptofp result");
  if (rc) return rc;
  if (extent0(src) != extent0(dst) || extent1(src) != extent1(dst))
    return fail(KAPY_ERR_VERIFY, "fptofp: source and result must have the same shape");
  kapy_ew_inst prog[3] = {{KAPY_EW_LD_GLOBAL, 0, 0, 0, 0, 0, KAPY_RN, 0.f},
                          {KAPY_EW_FPTOFP, 1, 0, 0, 0, dst->dtype, rmode, 0.f},
                          {KAPY_EW_ST_GLOBAL, 0, 1, 0, 0, 0, KAPY_RN, 0.f}};
  const kapy_global *ins[1] = {src};
  return kapy_elementwise(prog, 3, ins, 1, dst, stream);
}

}  // extern "C"
