// ew_row_machine.hpp — device side and launcher of the row machine (see elementwise_row.hip), a template over the
// kernel's mode so that the light, 16-bit and general kernels are built in translation units of their own.
#pragma once
#include "ew_machine.hpp"

namespace kapy {
namespace {

constexpr int kUSlots = 4;  // per-row values

// The per-row values: four named registers (an array indexed by a run-time value would be moved to scratch memory).
struct PerRow {
  float u0, u1, u2, u3;
};
// (v_cndmask chains; the empty asm keeps the optimiser from folding them back into an indexed access)
__device__ __forceinline__ float get_u(const PerRow &u, int k) {
  float r = u.u3;
  asm volatile("" : "+v"(r));
  r = k == 2 ? u.u2 : r;
  asm volatile("" : "+v"(r));
  r = k == 1 ? u.u1 : r;
  asm volatile("" : "+v"(r));
  r = k == 0 ? u.u0 : r;
  return r;
}
__device__ __forceinline__ void set_u(PerRow &u, int k, float r) {
  asm volatile("" : "+v"(u.u0), "+v"(u.u1), "+v"(u.u2), "+v"(u.u3));
  u.u0 = k == 0 ? r : u.u0;
  u.u1 = k == 1 ? r : u.u1;
  u.u2 = k == 2 ? r : u.u2;
  u.u3 = k == 3 ? r : u.u3;
  asm volatile("" : "+v"(u.u0), "+v"(u.u1), "+v"(u.u2), "+v"(u.u3));
}

enum RowMode { kModeLight = 0, kModeNarrow = 1, kModeAny = 2 };

// A step on one per-row value (left operand and result x, then y, z).  One element per row: full-precision routines
// cost nothing here.
__device__ __forceinline__ float scalar_step(const StackProgram &P, const PostOp &I, int32_t i, float x, float y, float z) {
  float r;
  switch (I.op) {
  case kPushIn: {
    const StackIn &g = P.in[I.a];
    return load_as_f32(g.base, g.dtype, g.kind == kInCol ? (int64_t)i * g.stride0 : 0);
  }
  case kPushImm: return round_to_dtype(I.imm, I.dtype, true);
  case kCast: return round_to_dtype(x, I.dtype, I.rmode != KAPY_RZ);
  case KAPY_EW_ADDF: r = __fadd_rn(x, y); break;
  case KAPY_EW_SUBF: r = __fsub_rn(x, y); break;
  case kRevSub: r = __fsub_rn(y, x); break;
  case KAPY_EW_MULF: r = __fmul_rn(x, y); break;
  case KAPY_EW_DIVF: r = __fdiv_rn(x, y); break;
  case kRevDiv: r = __fdiv_rn(y, x); break;
  case KAPY_EW_MAXIMUMF: r = max_nan(x, y); break;
  case KAPY_EW_MINIMUMF: r = min_nan(x, y); break;
  case KAPY_EW_MAXNUMF: r = max_num(x, y); break;
  case KAPY_EW_MINNUMF: r = min_num(x, y); break;
  case KAPY_EW_FMA: r = fma_typed(x, y, z, I.dtype); break;
  default: r = apply_unary(I.op, x);
  }
  return I.dtype != KAPY_F32 ? round_to_dtype(r, I.dtype, true) : r;
}

// The ops of the light kernel, in place on row value D of every chunk: 16-bit memory types, round-to-nearest casts,
// and arithmetic whose hardware forms are exact or within an fp32 ulp or two, which the final 16-bit rounding hides.
// The right operand is the next row value, the step's per-row value or the left operand itself, chosen once per
// step.  The host sends a program here only if every row step is one of these.
#define KAPY_LIGHT_BINARY(EXPR)                                                    \
  do {                                                                             \
    if (I.slot & kUniformRight) {                                                  \
      _Pragma("unroll") for (int c = 0; c < CH; ++c)                               \
      _Pragma("unroll") for (int e = 0; e < 8; ++e) {                              \
        const float x = v[c][D][e], y = ur;                                        \
        v[c][D][e] = (EXPR);                                                       \
      }                                                                            \
    } else if (I.slot & kSameOperand) {                                            \
      _Pragma("unroll") for (int c = 0; c < CH; ++c)                               \
      _Pragma("unroll") for (int e = 0; e < 8; ++e) {                              \
        const float x = v[c][D][e], y = x;                                         \
        v[c][D][e] = (EXPR);                                                       \
      }                                                                            \
    } else {                                                                       \
      _Pragma("unroll") for (int c = 0; c < CH; ++c)                               \
      _Pragma("unroll") for (int e = 0; e < 8; ++e) {                              \
        const float x = v[c][D][e], y = v[c][R][e];                                \
        v[c][D][e] = (EXPR);                                                       \
      }                                                                            \
    }                                                                              \
  } while (0)
#define KAPY_LIGHT_UNARY(EXPR)                                                     \
  do {                                                                             \
    _Pragma("unroll") for (int c = 0; c < CH; ++c)                                 \
    _Pragma("unroll") for (int e = 0; e < 8; ++e) {                                \
      const float x = v[c][D][e];                                                  \
      v[c][D][e] = (EXPR);                                                         \
    }                                                                              \
  } while (0)

template <int D, int CH, int THREADS, int NS>
__device__ __forceinline__ void light_step(const StackProgram &P, const PostOp &I, int32_t i, float (&v)[CH][NS][8], float ur) {
  constexpr int R = D + 1 < NS ? D + 1 : D, T = D + 2 < NS ? D + 2 : D;
  const int tid = threadIdx.x;
  switch (I.op) {
  case kPushImm: {
    const float c0 = round_to_dtype(I.imm, I.dtype, true);
    KAPY_LIGHT_UNARY((void(x), c0));
    return;
  }
  case kStore:
#pragma unroll
    for (int c = 0; c < CH; ++c) {
      const int32_t jv = c * THREADS + tid;
      if (jv < P.vec_per_row) store8<true>(P.out, P.out_dtype, (int64_t)i * P.out_stride0 + (int64_t)jv * 8, v[c][D]);
    }
    return;
  case kCast: break;  // the rounding below is the cast
  case KAPY_EW_ADDF: KAPY_LIGHT_BINARY(__fadd_rn(x, y)); break;
  case KAPY_EW_SUBF: KAPY_LIGHT_BINARY(__fsub_rn(x, y)); break;
  case kRevSub: KAPY_LIGHT_BINARY(__fsub_rn(y, x)); break;
  case KAPY_EW_MULF: KAPY_LIGHT_BINARY(__fmul_rn(x, y)); break;
  case KAPY_EW_MAXIMUMF: KAPY_LIGHT_BINARY(max_nan(x, y)); break;
  case KAPY_EW_MINIMUMF: KAPY_LIGHT_BINARY(min_nan(x, y)); break;
  case KAPY_EW_FMA:
#pragma unroll
    for (int c = 0; c < CH; ++c)
#pragma unroll
      for (int e = 0; e < 8; ++e) v[c][D][e] = fma_typed(v[c][D][e], v[c][R][e], v[c][T][e], I.dtype);
    break;
  case KAPY_EW_NEGF: KAPY_LIGHT_UNARY(-x); break;
  case KAPY_EW_ABSF: KAPY_LIGHT_UNARY(fabsf(x)); break;
  case KAPY_EW_RSQRT: KAPY_LIGHT_UNARY(__builtin_amdgcn_rsqf(x)); break;
  case KAPY_EW_SQRT: KAPY_LIGHT_UNARY(__builtin_amdgcn_sqrtf(x)); break;
  case KAPY_EW_GELU_TANH: KAPY_LIGHT_UNARY(gelu_tanh_f32(x)); break;
  default: return;
  }
  if (I.dtype != KAPY_F32) {
#pragma unroll
    for (int c = 0; c < CH; ++c) round8<true>(v[c][D], I.dtype, true);
  }
}
#undef KAPY_LIGHT_BINARY
#undef KAPY_LIGHT_UNARY

template <int D, int CH, int THREADS, int NS, int MODE>
__device__ __forceinline__ void row_step(const StackProgram &P, const PostOp &I, int32_t i, int pc, float (&v)[CH][NS][8], PerRow &u,
                                         float *lds) {
  constexpr bool NARROW = MODE != kModeAny, LIGHT = MODE == kModeLight;
  const int tid = threadIdx.x;
  constexpr int WAVES = THREADS / 64;
  const int k = (I.slot >> 8) & 3;
  if (I.op == KAPY_EW_REDUCE_SUM || I.op == KAPY_EW_REDUCE_MAX) {  // row value D -> per-row value k
    const bool sum = I.op == KAPY_EW_REDUCE_SUM;
    float acc = sum ? -0.f : -__builtin_inff();  // -0: the identity of addition, a row of only -0 sums to -0
#pragma unroll
    for (int c = 0; c < CH; ++c) {
      if (c * THREADS + tid < P.vec_per_row) {
        float part;
        if (sum) part = ((v[c][D][0] + v[c][D][1]) + (v[c][D][2] + v[c][D][3])) + ((v[c][D][4] + v[c][D][5]) + (v[c][D][6] + v[c][D][7]));
        else {
          // fmaxf skips a NaN operand, so NaNs are looked for separately
          part = fmaxf(fmaxf(fmaxf(v[c][D][0], v[c][D][1]), fmaxf(v[c][D][2], v[c][D][3])),
                       fmaxf(fmaxf(v[c][D][4], v[c][D][5]), fmaxf(v[c][D][6], v[c][D][7])));
          bool any_nan = false;
#pragma unroll
          for (int e = 0; e < 8; ++e) any_nan |= v[c][D][e] != v[c][D][e];
          if (any_nan) part = __builtin_nanf("");
        }
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
    set_u(u, k, round_to_dtype(acc, I.dtype, true));
    return;
  }
  if (I.slot & kUniformResult) {  // a step on the per-row stack: result and left operand k, then k+1, k+2
    if (I.op == kPick) { set_u(u, k, get_u(u, I.a)); return; }
    set_u(u, k, scalar_step(P, I, i, get_u(u, k), get_u(u, k + 1 < kUSlots ? k + 1 : k), get_u(u, k + 2 < kUSlots ? k + 2 : k)));
    return;
  }
  if (I.op == kPick) {  // a copy of a row value lower on the stack (I.a < D)
    if (D > 0) {
#pragma unroll
      for (int c = 0; c < CH; ++c)
#pragma unroll
        for (int e = 0; e < 8; ++e) v[c][D][e] = (D == 2 && I.a == 1) ? v[c][NS > 1 ? 1 : 0][e] : v[c][0][e];
    }
    return;
  }
  const float ur = get_u(u, k);  // the per-row operand of steps that have one
  if (I.op == kPushU) {
#pragma unroll
    for (int c = 0; c < CH; ++c)
#pragma unroll
      for (int e = 0; e < 8; ++e) v[c][D][e] = ur;
    return;
  }
  if (I.op == KAPY_EW_DIVF && (I.slot & kUniformRight)) {
    // division of the row by one value: x*(1/y) corrected by one Newton step on the remainder, which is the
    // correctly rounded quotient except where it is subnormal; the divisor's reciprocal is computed once.  A very
    // large or very small divisor is brought to the middle of the range together with the dividends (a power of two,
    // exact); zero, infinite and NaN divisors and dividends come out of x*(1/y) as IEEE division has them, and are
    // recognised by the NaN remainder they leave.
    float y = ur;
    const float ay = fabsf(y);
    const float scale = ay > 1e30f ? 0x1p-64f : ay < 1e-30f ? 0x1p64f : 1.0f;
    y *= scale;
    const float rcp = __builtin_amdgcn_rcpf(y);
#pragma unroll
    for (int c = 0; c < CH; ++c) {
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const float x = v[c][D][e] * scale;
        const float q = x * rcp;
        const float rem = __builtin_fmaf(-q, y, x);
        const float q2 = __builtin_fmaf(rem, rcp, q);
        v[c][D][e] = (rem == rem && rem != 0.f) ? q2 : q;  // (a zero remainder: q is exact already, and adding +0 would turn a -0 quotient into +0)
      }
      if (I.dtype != KAPY_F32) round8<NARROW>(v[c][D], I.dtype, true);
    }
    return;
  }
  if (NARROW && I.op == KAPY_EW_EXP && I.dtype == KAPY_F32) {
    // exp(x) = 2^(x*log2(e)) with the product's rounding error carried into a first-order correction: about
    // 2 ulp of fp32, far below the 16-bit rounding that every result of a NARROW program ends in
#pragma unroll
    for (int c = 0; c < CH; ++c) {
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const float x = v[c][D][e];
        const float hi = x * 1.44269504088896341f;
        const float lo = __builtin_fmaf(x, 1.44269504088896341f, -hi) + x * 1.92596299e-8f;
        const float p = __builtin_amdgcn_exp2f(hi);
        // 2^hi is already 0 or infinite where exp(x) leaves the fp32 range (results below 2^-126 become 0)
        v[c][D][e] = p > 3e38f ? p : __builtin_fmaf(p * lo, 0.693147180559945309f, p);
      }
    }
    return;
  }
  if (NARROW && I.op == kPushIn && P.in[I.a].kind <= kInRow) {
    // a full or row operand of 16-bit elements: every chunk's 16 bytes are asked for before any is widened
    const StackIn &g = P.in[I.a];
    u32x4 raw[CH];
#pragma unroll
    for (int c = 0; c < CH; ++c) {
      const int32_t jv = c * THREADS + tid;
      const char *ptr = g.base + ((g.kind == kInRow ? 0 : (int64_t)i * g.stride0) + (int64_t)jv * 8) * 2;
      raw[c] = u32x4{0, 0, 0, 0};
      if (jv < P.vec_per_row) raw[c] = g.kind == kInFull ? __builtin_nontemporal_load((const u32x4 *)ptr) : *(const u32x4 *)ptr;
    }
#pragma unroll
    for (int c = 0; c < CH; ++c) widen16x8(raw[c], g.dtype, v[c][D]);
    return;
  }
  if (LIGHT && I.op != kSaveTmp && I.op != kPushTmp) {
    light_step<D, CH, THREADS, NS>(P, I, i, v, ur);
    return;
  }
  float *tmps = lds + 32;
#pragma unroll
  for (int c = 0; c < CH; ++c) {
    __builtin_amdgcn_sched_barrier(0);  // one chunk's temporaries at a time
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
      continue;
    }
    // the general step: operands gathered into the three positions the stack machine's step works on
    float t[3][8];
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      t[0][e] = v[c][D][e];
      t[1][e] = (I.slot & kUniformRight) ? ur : (I.slot & kSameOperand) ? v[c][D][e] : D + 1 < NS ? v[c][D + 1 < NS ? D + 1 : D][e] : 0.f;
      t[2][e] = D + 2 < NS ? v[c][D + 2 < NS ? D + 2 : D][e] : 0.f;
    }
    if (LIGHT) continue;  // (only the LDS steps above reach this loop in the light kernel)
    if ((I.op != kPushIn && I.op != kStore) || active) stack_step<0, NARROW>(P, I, i, jv, t);
#pragma unroll
    for (int e = 0; e < 8; ++e) v[c][D][e] = t[0][e];
  }
}

template <int CH, int THREADS, int NS, int MODE>
__global__ __launch_bounds__(THREADS) void row_kernel(StackProgram P) {
  extern __shared__ float row_lds[];
  const int32_t i = blockIdx.x;
  float v[CH][NS][8];
  PerRow u = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
  for (int c = 0; c < CH; ++c)
#pragma unroll
    for (int d = 0; d < NS; ++d)
#pragma unroll
      for (int e = 0; e < 8; ++e) v[c][d][e] = 0.f;
  PostOp next = P.post[0];
  for (int pc = 0; pc < P.n_post; ++pc) {
    const PostOp I = next;
    next = P.post[pc + 1 < P.n_post ? pc + 1 : pc];  // fetched while this step runs
    const int d = I.slot & kSlotMask;
    if (NS > 2 && d == 2) row_step<(NS > 2 ? 2 : 0), CH, THREADS, NS, MODE>(P, I, i, pc, v, u, row_lds);
    else if (NS > 1 && d == 1) row_step<(NS > 1 ? 1 : 0), CH, THREADS, NS, MODE>(P, I, i, pc, v, u, row_lds);
    else row_step<0, CH, THREADS, NS, MODE>(P, I, i, pc, v, u, row_lds);
  }
}

template <int MODE>
int launch_row_kernel(const StackProgram &P, int ns, hipStream_t s) {
  constexpr bool NARROW = MODE != kModeAny;
  const int vpr = P.vec_per_row;
  // the smallest workgroup that covers the row with at most four chunks of 8 elements per lane: a step's fixed cost
  // (fetching and decoding it) is then shared by up to 32 elements, and several rows are resident per CU
  // (the kernels that carry the general step are few: short rows share the 256-lane one)
  const int threads = (vpr <= 256 && MODE == kModeLight) ? 64 : vpr <= 1024 ? 256 : 1024;
  const int ch = (vpr + threads - 1) / threads;
  const size_t lds = (32 + (size_t)P.n_tmps * vpr * 8) * sizeof(float);  // 32 floats: the reduce exchange of up to 16 waves, twice
  if (lds > 160 * 1024) return fail(KAPY_ERR_UNSUPPORTED, "elementwise: the program keeps %d row values of %d elements alive, more than fits the LDS", P.n_tmps, vpr * 8);
  dim3 grid((unsigned)P.rows);
#define KAPY_ROW(CH_, TH_, NS_)                                                                                    \
  do {                                                                                                             \
    if (lds > 48 * 1024) KAPY_HIP_CHECK(hipFuncSetAttribute((const void *)row_kernel<CH_, TH_, NS_, MODE>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds)); \
    row_kernel<CH_, TH_, NS_, MODE><<<grid, TH_, lds, s>>>(P);                                                   \
  } while (0)
  // The light kernel exists per chunk count, and for four chunks per stack depth, so that a program that needs one or
  // two row values is not charged the registers of three.  The others always carry four chunks and three values.
#define KAPY_ROW_CH(TH_)                                                                                           \
  do {                                                                                                             \
    if (MODE != kModeLight || (ch > 2 && ns == 3)) KAPY_ROW(4, TH_, 3);                                            \
    else if (ch == 1) KAPY_ROW((MODE == kModeLight ? 1 : 4), TH_, 3);                                              \
    else if (ch == 2) KAPY_ROW((MODE == kModeLight ? 2 : 4), TH_, 3);                                              \
    else if (ns == 2) KAPY_ROW(4, TH_, (MODE == kModeLight ? 2 : 3));                                              \
    else KAPY_ROW(4, TH_, (MODE == kModeLight ? 1 : 3));                                                           \
  } while (0)
  if (threads == 64) { if constexpr (MODE == kModeLight) KAPY_ROW_CH(64); }
  else if (threads == 256) KAPY_ROW_CH(256);
  else KAPY_ROW_CH(1024);
#undef KAPY_ROW_CH
#undef KAPY_ROW
  KAPY_HIP_CHECK(hipGetLastError());
  return KAPY_OK;
}

}  // namespace
}  // namespace kapy
