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
#include <stdlib.h>
#include <string.h>

#include <string>
#include <type_traits>
#include <utility>
#include <vector>

#include "common.hpp"
#include <functional>
#include "numeric.hpp"
#include "ew_machine.hpp"

namespace kapy {
namespace {


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

// (device helpers and the stack machine proper live in ew_machine.hpp)
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
    case KAPY_EW_ST_GLOBAL:
      if (active) store_from_f32((void *)P.out.base, P.out.dtype, i * P.out.stride0 + j * P.out.stride1, regs[I.a][tid]);
      continue;
    default: r = machine_step<256>(I, &regs[0][tid], i, j);
    }
    regs[I.dst][tid] = r;  // regs[*][tid] is private to the lane: no barrier needed
  }
}

// Column machine: a program whose reduces run along axis 0 (ReduceOpToLLVM.cpp:51-172 reduces either axis).  A workgroup
// owns a strip of 64 columns, one per lane, and its waves share out the rows, so a wave's accesses to a row-major operand
// are 64 consecutive elements.  The program runs in phases, one per reduce and a last one that stores: phase p walks all
// rows executing only the instructions reduce p depends on (earlier reduces are per-column values by then), folds the
// operand in fp32 per wave, and the waves' partials are folded in wave order and rounded once to the register's type, as
// kapy_reduce does.  Operands are re-read in every phase (they come from L2 when the strip fits there); nothing but the
// per-column results is kept on chip, so any number of rows is served.
constexpr int kMaxColumnReduces = 4;
struct ColumnPlan {
  int32_t n_phases;                      // reduces + 1
  int32_t stop[kMaxColumnReduces + 1];   // the phase's reduce instruction; n_inst for the storing phase
  uint64_t need[kMaxColumnReduces + 1];  // bit k: the phase executes instruction k
};

template <int WAVES>
__global__ __launch_bounds__(WAVES * 64) void column_program_kernel(Program P, ColumnPlan C) {
  __shared__ float regs[kMaxRegs][WAVES * 64];
  __shared__ float part[WAVES][64];
  __shared__ float red[kMaxColumnReduces][64];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int32_t j = (int32_t)blockIdx.x * 64 + lane;
  const bool in_strip = j < P.out.ext1;
  for (int phase = 0; phase < C.n_phases; ++phase) {
    const bool last = phase == C.n_phases - 1;
    const int stop = C.stop[phase];
    const uint64_t need = C.need[phase];
    const bool sum = !last && P.inst[stop].op == KAPY_EW_REDUCE_SUM;
    float acc = sum ? -0.f : -__builtin_inff();  // -0: the identity of addition, a column of only -0 sums to -0
    for (int32_t i = wave; i < P.out.ext0; i += WAVES) {
      for (int k = 0; k < stop; ++k) {
        if (!((need >> k) & 1)) continue;
        const kapy_ew_inst I = P.inst[k];
        float r = 0.f;
        switch (I.op) {
        case KAPY_EW_LD_GLOBAL: {
          const DevView &g = P.in[I.a];
          const int32_t gi = g.ext0 == 1 ? 0 : i, gj = g.ext1 == 1 ? 0 : j;
          if (in_strip && gi < g.ext0 && gj < g.ext1) r = load_as_f32(g.base, g.dtype, gi * g.stride0 + gj * g.stride1);
          else {
            uint32_t w = I.c == KAPY_PAD_ZERO ? 0u : g.pad;
            r = load_as_f32(&w, g.dtype, 0);
          }
          break;
        }
        case KAPY_EW_REDUCE_SUM: case KAPY_EW_REDUCE_MAX: r = red[I.c][lane]; break;  // I.c: which reduce this is (set by the host)
        case KAPY_EW_ST_GLOBAL:
          if (in_strip) store_from_f32((void *)P.out.base, P.out.dtype, i * P.out.stride0 + j * P.out.stride1, regs[I.a][tid]);
          continue;
        default: r = machine_step<WAVES * 64>(I, &regs[0][tid], i, j);
        }
        regs[I.dst][tid] = r;  // regs[*][tid] is private to the lane
      }
      if (!last) {
        const float x = regs[P.inst[stop].a][tid];
        acc = sum ? acc + x : max_nan(acc, x);
      }
    }
    if (last) break;
    part[wave][lane] = acc;
    __syncthreads();
    if (wave == 0) {
      float total = part[0][lane];
      for (int w = 1; w < WAVES; ++w) total = sum ? total + part[w][lane] : max_nan(total, part[w][lane]);
      red[phase][lane] = round_to_dtype(total, P.inst[stop].dtype, true);
    }
    __syncthreads();
  }
}

// Throughput of this kernel follows the number of resident waves (each lane walks its program one
// dependent step at a time), so the 16-bit-only form is held to 64 registers: 8 waves per SIMD.
// (The operations whose code alone overruns 64 registers - remf, sin, cos - are left out of it; a program that holds one
// runs the same machine without the cap.)
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(8, 8))) void stack_kernel_narrow(StackProgram P) { stack_run<true, false, true>(P); }
__global__ __launch_bounds__(256) void stack_kernel_narrow_heavy(StackProgram P) { stack_run<true>(P); }
__global__ __launch_bounds__(256) void stack_kernel_any(StackProgram P) { stack_run<false>(P); }
// rows whose width is not a multiple of 8 (row starts still 16-byte aligned): the last vector of a row moves element by element
__global__ __launch_bounds__(256) void stack_kernel_narrow_ragged(StackProgram P) { stack_run<true, true>(P); }

// A reduce along axis 0 of a program's value, for the column programs (run_column_program): the stack machine's steps with
// the store replaced by a fold over rows.  A workgroup owns a strip of 8 * LPR columns (LPR lanes x one vector of 8) and a
// chunk of the rows, which its 256 / LPR groups of lanes walk; the groups' partial results meet in LDS and every
// (chunk, column) leaves an fp32 partial result in `lines`, which column_fold_kernel folds in chunk order.
template <int LPR>
__global__ __launch_bounds__(256) void stack_colreduce_kernel(StackProgram P, float *lines, int32_t per_chunk, int32_t sum) {
  constexpr int GROUPS = 256 / LPR, COLS = LPR * 8;
  __shared__ float part[GROUPS][COLS + 1];
  const int cl = threadIdx.x % LPR, rg = threadIdx.x / LPR;
  const int32_t jv = (int32_t)blockIdx.x * LPR + cl;
  const int32_t r_begin = blockIdx.y * per_chunk, r_end = min(P.rows, r_begin + per_chunk);
  float acc[8];
#pragma unroll
  for (int e = 0; e < 8; ++e) acc[e] = sum ? -0.f : -__builtin_inff();  // -0: the identity of addition
  if (jv < P.vec_per_row) {
    for (int32_t i = r_begin + rg; i < r_end; i += GROUPS) {
      float v[3][8];
#pragma unroll
      for (int d = 0; d < 3; ++d)
#pragma unroll
        for (int e = 0; e < 8; ++e) v[d][e] = 0.f;
      for (int pc = 0; pc < P.n_post; ++pc) {
        const PostOp I = P.post[pc];
        if (I.op == kStore) {  // (the value to fold is at the bottom of the stack)
#pragma unroll
          for (int e = 0; e < 8; ++e) acc[e] = sum ? acc[e] + v[0][e] : max_nan(acc[e], v[0][e]);
          continue;
        }
        switch (I.slot) {
        case 0: stack_step<0, false>(P, I, i, jv, v); break;
        case 1: stack_step<1, false>(P, I, i, jv, v); break;
        default: stack_step<2, false>(P, I, i, jv, v);
        }
      }
    }
  }
#pragma unroll
  for (int e = 0; e < 8; ++e) part[rg][cl * 8 + e] = acc[e];
  __syncthreads();
  const int64_t col = (int64_t)blockIdx.x * COLS + threadIdx.x;
  if (threadIdx.x < COLS && col < (int64_t)P.vec_per_row * 8) {
    float t = part[0][threadIdx.x];
#pragma unroll
    for (int g = 1; g < GROUPS; ++g) t = sum ? t + part[g][threadIdx.x] : max_nan(t, part[g][threadIdx.x]);
    lines[(int64_t)blockIdx.y * P.vec_per_row * 8 + col] = t;
  }
}

// `chunks` partial lines of n values folded in chunk order, rounded once to the reduce's type, stored as that type.
__global__ __launch_bounds__(256) void column_fold_kernel(const float *lines, int32_t chunks, int32_t n, int32_t sum, int32_t dtype, void *result) {
  const int32_t col = (int32_t)blockIdx.x * 256 + threadIdx.x;
  if (col >= n) return;
  float t = lines[col];
  for (int32_t c = 1; c < chunks; ++c) {
    const float x = lines[(int64_t)c * n + col];
    t = sum ? t + x : max_nan(t, x);
  }
  store_from_f32(result, dtype, col, t);
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
  int32_t width;                      // elements per row when the last vector of a row is partial, else 0
  int32_t combine;                    // how the second operand meets x*scale: Combine (plain binary programs; kAdd otherwise)
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
enum Combine { kAdd = 0, kSub = 1 /* x - y */, kRevSubtract = 2 /* y - x */, kMul = 3, kMax = 4, kMin = 5 };
template <int ACT>
__device__ __forceinline__ float affine_act(float x, float scale, float bias, int act, int combine) {
  if (ACT == -1 && combine != kAdd) {  // z = x op y on the 16-bit type: the fp32 result rounded once is the type's own
    switch (combine) {
    case kSub: return x - bias;
    case kRevSubtract: return bias - x;
    case kMul: return x * bias;
    case kMax: return max_nan(x, bias);
    default: return min_nan(x, bias);
    }
  }
  float v = x * scale + bias;
  if (ACT == KAPY_EW_GELU_TANH) return gelu_tanh_f32(v);
  if (ACT >= 0) return apply_unary(act, v);
  return v;
}

// 16-bit in, 16-bit out (same type), 8 elements per 16-byte vector, UNROLL vectors per lane.
constexpr int kEwUnroll = 2;    // 16-byte vectors per lane of the flat fused kernels
constexpr bool kEwNt = true;    // non-temporal loads and stores (the operands are streamed once)
// 16 bytes at ptr, or the first `valid` elements of them at the ragged end of a row (RAGGED kernels only)
template <bool RAGGED>
__device__ __forceinline__ u32x4 load_row16(const char *ptr, int valid, bool stream) {
  if (RAGGED && valid < 8) return load16_partial(ptr, valid);
  return stream ? __builtin_nontemporal_load((const u32x4 *)ptr) : *(const u32x4 *)ptr;
}
template <bool RAGGED>
__device__ __forceinline__ void store_row16(char *ptr, u32x4 v, int valid) {
  if (RAGGED && valid < 8) { store16_partial(ptr, v, valid); return; }
  if (kEwNt) __builtin_nontemporal_store(v, (u32x4 *)ptr);
  else *(u32x4 *)ptr = v;
}

template <typename T, int ACT, bool RAGGED>
__global__ __launch_bounds__(256) void affine_act_kernel(AffineActParams p) {
  constexpr int UNROLL = kEwUnroll;
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
      const int valid = RAGGED ? p.width - col[u] : 8;
      xv[u] = load_row16<RAGGED>(p.x + ((int64_t)row[u] * p.x_stride0 + col[u]) * 2, valid, kEwNt);
      if (p.bias_mode == kBiasRow) bv[u] = load_row16<RAGGED>(p.bias + (int64_t)col[u] * 2, valid, false);
      else if (p.bias_mode == kBiasFull) bv[u] = load_row16<RAGGED>(p.bias + ((int64_t)row[u] * p.bias_stride0 + col[u]) * 2, valid, kEwNt);  // (read once, like x)
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
    for (int e = 0; e < 8; ++e) f[e] = affine_act<ACT>(f[e], scale, p.bias_mode != kNoBias ? b[e] : 0.f, p.act, p.combine);
    store_row16<RAGGED>(p.out + ((int64_t)row[u] * p.out_stride0 + col[u]) * 2, pack8<T>(f), RAGGED ? p.width - col[u] : 8);
  }
}

// Same chain when the bias is broadcast along rows (bias[0, j]) or absent: a lane keeps one
// 8-column chunk and walks ROWS consecutive rows, so its bias vector is fetched and widened once
// and no index division is needed.  Grid: x over column chunks, y over groups of ROWS rows.
template <typename T, int ACT, bool RAGGED>
__global__ __launch_bounds__(256) void affine_act_cols_kernel(AffineActParams p) {
  constexpr int ROWS = 2;  // rows in flight per lane
  const int32_t chunk = blockIdx.x * 256 + threadIdx.x;
  if (chunk >= p.vec_per_row) return;
  const int32_t col = chunk * 8, row0 = blockIdx.y * ROWS;
  const float scale = p.has_scale ? p.scale : 1.0f;
  float b[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
  const int valid = RAGGED ? p.width - col : 8;
  if (p.bias_mode == kBiasRow) unpack8<T>(load_row16<RAGGED>(p.bias + (int64_t)col * 2, valid, false), b);
  u32x4 xv[ROWS];
#pragma unroll
  for (int u = 0; u < ROWS; ++u)
    if (row0 + u < p.rows) xv[u] = load_row16<RAGGED>(p.x + ((int64_t)(row0 + u) * p.x_stride0 + col) * 2, valid, kEwNt);
#pragma unroll
  for (int u = 0; u < ROWS; ++u) {
    if (row0 + u >= p.rows) break;
    float f[8];
    unpack8<T>(xv[u], f);
#pragma unroll
    for (int e = 0; e < 8; ++e) f[e] = affine_act<ACT>(f[e], scale, b[e], p.act, p.combine);
    store_row16<RAGGED>(p.out + ((int64_t)(row0 + u) * p.out_stride0 + col) * 2, pack8<T>(f), valid);
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

// `normalised`, if given, receives the program as the kernels are to read it: a copy in which a cast that does not narrow
// (f16 <-> bf16, any widening) rounds to nearest whatever its rounding mode field says - the reference asks for a rounding
// mode on down casts only (Kapy.cpp:272-287), and so does the oracle.
int verify_program(const kapy_ew_inst *prog, int n_inst, const kapy_global *const *ins, int n_ins, const kapy_global *out,
                   int result_dtype[kMaxInst], kapy_ew_inst *normalised = nullptr) {
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
    if (normalised) normalised[k] = I;
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
      if (I.dtype != KAPY_F16 && I.dtype != KAPY_BF16 && I.dtype != KAPY_F32 && !is_int(I.dtype))
        return fail(KAPY_ERR_VERIFY, "splat: only f16, bf16, f32 and integer splats are supported");
      reg_dtype[I.dst] = I.dtype;
      break;
    case KAPY_EW_ARANGE:
      if (I.b != 0 && I.b != 1) return fail(KAPY_ERR_VERIFY, "arange: axis must be 0 or 1");
      reg_dtype[I.dst] = KAPY_I32;
      break;
    case KAPY_EW_SELECT:
      if (!reg_ok(I.a) || !reg_ok(I.b) || !reg_ok(I.c)) return fail(KAPY_ERR_INVALID, "elementwise: use of undefined register at %d", k);
      if (reg_dtype[I.a] != KAPY_I1) return fail(KAPY_ERR_VERIFY, "select: condition must have i1 element type");
      if (reg_dtype[I.b] != reg_dtype[I.c]) return fail(KAPY_ERR_VERIFY, "select: true and false values must have the same element type");
      reg_dtype[I.dst] = reg_dtype[I.b];
      break;
    case KAPY_EW_TRUNCI: case KAPY_EW_EXTSI: case KAPY_EW_EXTUI: case KAPY_EW_SITOFP: case KAPY_EW_FPTOSI: case KAPY_EW_BITCAST: {
      if (!reg_ok(I.a)) return fail(KAPY_ERR_INVALID, "elementwise: use of undefined register at %d", k);
      const int sd = reg_dtype[I.a], dd = I.dtype;
      auto bits = [](int d) { return d == KAPY_I1 ? 1 : 8 * dtype_bytes(d); };
      const bool arith_float_s = sd == KAPY_F16 || sd == KAPY_BF16 || sd == KAPY_F32, arith_float_d = dd == KAPY_F16 || dd == KAPY_BF16 || dd == KAPY_F32;
      if (!dtype_bytes(dd)) return fail(KAPY_ERR_INVALID, "elementwise: unknown element type %d at %d", dd, k);
      if (I.op == KAPY_EW_TRUNCI && !(is_int(sd) && is_int(dd) && bits(dd) < bits(sd)))
        return fail(KAPY_ERR_VERIFY, "trunci: operand and result must be integers, the result narrower");
      if ((I.op == KAPY_EW_EXTSI || I.op == KAPY_EW_EXTUI) && !(is_int(sd) && is_int(dd) && bits(dd) > bits(sd)))
        return fail(KAPY_ERR_VERIFY, "extsi / extui: operand and result must be integers, the result wider");
      if (I.op == KAPY_EW_SITOFP && !(is_int(sd) && arith_float_d)) return fail(KAPY_ERR_VERIFY, "sitofp: an integer operand and an f16, bf16 or f32 result are required");
      if (I.op == KAPY_EW_FPTOSI && !(arith_float_s && is_int(dd) && dd != KAPY_I1)) return fail(KAPY_ERR_VERIFY, "fptosi: an f16, bf16 or f32 operand and an i8, i16 or i32 result are required");
      if (I.op == KAPY_EW_BITCAST && (sd == KAPY_I1 || dd == KAPY_I1 || dtype_bytes(sd) != dtype_bytes(dd)))
        return fail(KAPY_ERR_VERIFY, "bitcast: operand and result must have the same bit width");
      if (normalised) normalised[k].rmode = sd;   // the machines read the operand's type here
      reg_dtype[I.dst] = dd;
      break;
    }
    case KAPY_EW_FPTOFP: {
      if (!reg_ok(I.a)) return fail(KAPY_ERR_INVALID, "elementwise: use of undefined register at %d", k);
      int sd = reg_dtype[I.a], dd = I.dtype;
      if (!is_float(sd) || !is_float(dd)) return fail(KAPY_ERR_VERIFY, "fptofp: operands must have float element type");
      bool down = dtype_bytes(dd) < dtype_bytes(sd);
      if (down && I.rmode != KAPY_RN && I.rmode != KAPY_RZ) return fail(KAPY_ERR_VERIFY, "fptofp: rounding mode is required for down cast");
      if (sd == KAPY_BF16 && is_f8(dd) && I.rmode == KAPY_RZ)
        return fail(KAPY_ERR_VERIFY, "fptofp: unsupported rounding mode when convert bf16 to f8");
      if (is_f8(sd) && is_f8(dd)) return fail(KAPY_ERR_VERIFY, "fptofp: convert f8 to f8 is not supported");
      if (normalised && !down) normalised[k].rmode = KAPY_RN;
      reg_dtype[I.dst] = dd;
      break;
    }
    case KAPY_EW_FMA:
      if (!reg_ok(I.a) || !reg_ok(I.b) || !reg_ok(I.c)) return fail(KAPY_ERR_INVALID, "elementwise: use of undefined register at %d", k);
      if (reg_dtype[I.a] != reg_dtype[I.b] || reg_dtype[I.a] != reg_dtype[I.c])
        return fail(KAPY_ERR_VERIFY, "elementwise: operands must have the same element type at %d", k);
      reg_dtype[I.dst] = reg_dtype[I.a];
      break;
    KAPY_EW_BINARY_CASES: {
      if (!reg_ok(I.a) || !reg_ok(I.b)) return fail(KAPY_ERR_INVALID, "elementwise: use of undefined register at %d", k);
      if (reg_dtype[I.a] != reg_dtype[I.b])
        return fail(KAPY_ERR_VERIFY, "elementwise: operands must have the same element type at %d", k);
      const bool on_ints = (I.op >= KAPY_EW_ADDI && I.op <= KAPY_EW_MINUI) || I.op == KAPY_EW_CMPI;
      if (on_ints && !is_int(reg_dtype[I.a])) return fail(KAPY_ERR_VERIFY, "elementwise: integer op on non-integer operands at %d", k);
      if (I.op == KAPY_EW_CMPI && (I.c < 0 || I.c > KAPY_CMPI_UGE)) return fail(KAPY_ERR_INVALID, "cmpi: unknown predicate %d", I.c);
      if (I.op == KAPY_EW_CMPF && (I.c < 0 || I.c > KAPY_CMPF_TRUE)) return fail(KAPY_ERR_INVALID, "cmpf: unknown predicate %d", I.c);
      if (I.op == KAPY_EW_CMPF && reg_dtype[I.a] != KAPY_F16 && reg_dtype[I.a] != KAPY_BF16 && reg_dtype[I.a] != KAPY_F32)
        return fail(KAPY_ERR_VERIFY, "cmpf: operands must be f16, bf16 or f32");
      if (normalised && (I.op == KAPY_EW_CMPI || I.op == KAPY_EW_CMPF)) normalised[k].rmode = reg_dtype[I.a];
      reg_dtype[I.dst] = (I.op == KAPY_EW_CMPI || I.op == KAPY_EW_CMPF) ? (int)KAPY_I1 : reg_dtype[I.a];
      break;
    }
    case KAPY_EW_ABSI:
      if (!reg_ok(I.a)) return fail(KAPY_ERR_INVALID, "elementwise: use of undefined register at %d", k);
      if (!is_int(reg_dtype[I.a])) return fail(KAPY_ERR_VERIFY, "absi: operand must be an integer");
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
    const bool typed_above = (I.op >= KAPY_EW_ADDI && I.op < KAPY_EW_NUM_OPS) || I.op == KAPY_EW_SPLAT;   // (each checked its own types)
    if (I.op != KAPY_EW_ST_GLOBAL && I.op != KAPY_EW_LD_GLOBAL && I.op != KAPY_EW_FPTOFP && !typed_above) {
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
    KAPY_EW_BINARY_CASES:
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
  int x_in = -1, bias_in = -1;
  p->act = -1;
  p->has_scale = 0;
  p->scale = 1.f;
  p->combine = kAdd;
  // st(op(ld x, ld y)) on the 16-bit type itself (addf: the reference's elementwise_add fixture): the fp32 sum,
  // difference or product of two 16-bit values is exact or rounds harmlessly (operands more than 2^16 apart), so
  // rounding it once to the type gives the type's own correctly rounded result
  const int top = cur >= 0 ? nodes[cur].kind : -1;
  const bool plain_add = (top == KAPY_EW_ADDF || top == KAPY_EW_SUBF || top == KAPY_EW_MULF || top == KAPY_EW_MAXIMUMF || top == KAPY_EW_MINIMUMF) &&
                         is_kind(nodes[cur].a, KAPY_EW_LD_GLOBAL) && is_kind(nodes[cur].b, KAPY_EW_LD_GLOBAL);
  if (plain_add) {
    x_in = nodes[nodes[cur].a].input;
    bias_in = nodes[nodes[cur].b].input;
    bool swapped = false;
    if (extent0(ins[x_in]) != extent0(out) || extent1(ins[x_in]) != extent1(out)) { std::swap(x_in, bias_in); swapped = true; }
    p->combine = top == KAPY_EW_ADDF ? kAdd : top == KAPY_EW_SUBF ? (swapped ? kRevSubtract : kSub) : top == KAPY_EW_MULF ? kMul : top == KAPY_EW_MAXIMUMF ? kMax : kMin;
  }
  if (!plain_add) {
  if (!is_kind(cur, KAPY_EW_FPTOFP) || nodes[cur].dtype != T || nodes[cur].rmode != KAPY_RN) return false;
  cur = nodes[cur].a;
  if (cur < 0) return false;
  int k = nodes[cur].kind;
  if (k >= KAPY_EW_NEGF && k <= KAPY_EW_GELU_TANH) {
    p->act = k;
    cur = nodes[cur].a;
    if (cur < 0) return false;
  }
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
  }
  const kapy_global *x = ins[x_in];
  if (x->dtype != T || x->stride1 != 1 || out->stride1 != 1) return false;
  const int64_t o0 = extent0(out), o1 = extent1(out);
  if (extent0(x) != o0 || extent1(x) != o1) return false;
  if (vector_bytes(x, 1) != 16 || vector_bytes(out, 1) != 16) return false;
  if (o0 * ((o1 + 7) / 8) >= (int64_t(1) << 31) - 1024) return false;
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
  p->vec_per_row = (int32_t)((o1 + 7) / 8);
  p->width = o1 % 8 ? (int32_t)o1 : 0;
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
// `folded`: the final value is folded by a reducing kernel instead of stored, so the rounding a store would perform
// has to be a step of the program.
bool build_stack_program(const kapy_ew_inst *prog, int n_inst, const int *result_dtype, const kapy_global *const *ins, int n_ins,
                         const kapy_global *out, StackProgram *P, bool folded = false) {
  struct N {
    int op, a = -1, b = -1, c = -1, dtype = -1, rmode = KAPY_RN, input = -1;
    float imm = 0.f;
  };
  for (int k = 0; k < n_inst; ++k)
    if (prog[k].op >= KAPY_EW_ADDI || is_int(result_dtype[k])) return false;  // integer registers: the register machines' business
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
    KAPY_EW_BINARY_CASES:
      n.a = reg[I.a]; n.b = reg[I.b]; break;
    default: n.a = reg[I.a];
    }
    nodes.push_back(n);
    reg[I.dst] = (int)nodes.size() - 1;
  }
  if (n_store != 1 || stored < 0) return false;
  for (const N &n : nodes)
    if (n.op == KAPY_EW_REDUCE_SUM || n.op == KAPY_EW_REDUCE_MAX) return false;  // the row machine's business
  // the result: rows contiguous, 8 elements at a time
  const int64_t o0 = extent0(out), o1 = extent1(out);
  const int ob = dtype_bytes(out->dtype);
  if (!is_float(out->dtype) || out->stride1 != 1 || ((uintptr_t)view_base(out) % (8 * ob)) || (out->stride0 * ob) % (8 * ob)) return false;
  if (o1 % 8 != 0) {  // a ragged last vector per row: the 16-bit kernel has a form for it
    bool narrow = out->dtype == KAPY_F16 || out->dtype == KAPY_BF16;
    for (int k = 0; k < n_ins; ++k) narrow = narrow && (ins[k]->dtype == KAPY_F16 || ins[k]->dtype == KAPY_BF16);
    for (int k = 0; k < n_inst; ++k) narrow = narrow && !is_f8(result_dtype[k]);
    if (!narrow) return false;
  }
  if (o0 * ((o1 + 7) / 8) >= (int64_t(1) << 31) - 1024) return false;
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
  // how often each value is used: one with several uses is copied from lower on the stack when it is still there
  // (otherwise it is evaluated again: every op is pure)
  std::vector<int> uses(nodes.size(), 0);
  {
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
  int holder[3] = {-1, -1, -1};  // which node's value each stack slot holds
  int count = 0;
  bool ok = true;
  auto push = [&](int op, int a, int dtype, int rmode, int slot, float imm) {
    if (count >= kMaxPost || slot > 2) { ok = false; return; }
    P->post[count++] = PostOp{(int16_t)op, (int16_t)a, (int16_t)dtype, (int16_t)rmode, slot, imm};
  };
  // evaluate node id into value d (values d+1, d+2 are free to use)
  std::function<void(int, int)> emit_node;
  std::function<void(int, int)> emit = [&](int id, int d) {
    if (!ok) return;
    if (d > 2) { ok = false; return; }
    if (uses[id] > 1 && nodes[id].op != KAPY_EW_SPLAT)
      for (int below = 0; below < d; ++below)
        if (holder[below] == id) {
          push(kPick, below, nodes[id].dtype, 0, d, 0.f);
          holder[d] = id;
          return;
        }
    emit_node(id, d);
    for (int above = d + 1; above < 3; ++above) holder[above] = -1;
    holder[d] = id;
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
    case KAPY_EW_FPTOFP:
      emit(n.a, d);
      // values are fp32 images of typed values: widening to f32 changes nothing; and the store rounds to nearest itself
      if (n.dtype != KAPY_F32 && !(!folded && id == stored && n.dtype == out->dtype && n.rmode != KAPY_RZ)) push(kCast, 0, n.dtype, n.rmode, d, 0.f);
      return;
    case KAPY_EW_FMA: emit(n.a, d); emit(n.b, d + 1); emit(n.c, d + 2); push(KAPY_EW_FMA, 0, n.dtype, 0, d, 0.f); return;
    KAPY_EW_BINARY_CASES: {
      const bool a_first = n.op == KAPY_EW_REMF || std::max(need[n.a], need[n.b] + 1) <= std::max(need[n.b], need[n.a] + 1);  // (remf has no reversed form)
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
  P->n_post = count;
  P->n_ins = n_ins;
  P->out = (char *)view_base(out);
  P->out_stride0 = out->stride0;
  P->out_dtype = out->dtype;
  P->rows = (int32_t)o0;
  P->vec_per_row = (int32_t)((o1 + 7) / 8);
  P->width = o1 % 8 ? (int32_t)o1 : 0;
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


// A program whose reduces all run along axis 0, on the column machine.
bool stream_is_capturing(hipStream_t s);

// The column program as a sequence of launches over the whole device, where its shapes allow: phase p (one per reduce) is an
// elementwise program of its own - the instructions reduce p depends on, with every earlier reduce replaced by a load of
// that reduce's per-column results ([1 x n], in the reduce's type) - whose value is folded over rows instead of stored
// (stack_colreduce_kernel over strips x row chunks, then column_fold_kernel); the last phase is an ordinary
// kapy_elementwise call with the results as row operands.  The results and the partial lines live in the library's own
// workspace array (reduce_scratch_lines: calls that use it must not overlap in time on one GPU).  Returns 1 when the program ran this way, 0 when it does not fit (the caller then runs the one-launch
// column machine, which takes any views), a negative status on failure.
int run_column_phases(const kapy_ew_inst *prog, int n_inst, const int *result_dtype, const kapy_global *const *ins, int n_ins, const kapy_global *out,
                      const ColumnPlan &C, const Program &P, hipStream_t s) {
  const int n_reduce = C.n_phases - 1;
  const int64_t m = extent0(out), n = extent1(out);
  if (n % 8 != 0 || out->stride1 != 1 || n_ins + n_reduce > kMaxInputs || m < 64) return 0;
  // phase programs, built before anything is launched: any that does not fit the stack machine sends the whole call back
  struct Phase {
    kapy_ew_inst inst[kMaxInst + 1];
    int dtype[kMaxInst + 1];
    int n = 0;
  };
  std::vector<Phase> phases(C.n_phases);
  int reduce_dtype[kMaxColumnReduces] = {0, 0, 0, 0};
  for (int k = 0; k < n_inst; ++k)
    if (prog[k].op == KAPY_EW_REDUCE_SUM || prog[k].op == KAPY_EW_REDUCE_MAX) reduce_dtype[P.inst[k].c] = result_dtype[k];
  for (int ph = 0; ph < C.n_phases; ++ph) {
    Phase &F = phases[ph];
    for (int k = 0; k < C.stop[ph]; ++k) {
      if (!((C.need[ph] >> k) & 1)) continue;
      kapy_ew_inst I = prog[k];
      if (I.op == KAPY_EW_REDUCE_SUM || I.op == KAPY_EW_REDUCE_MAX) {
        const int which = P.inst[k].c;
        I = kapy_ew_inst{};
        I.op = KAPY_EW_LD_GLOBAL;
        I.dst = prog[k].dst;
        I.a = n_ins + which;
        I.c = KAPY_PAD_ZERO;
      }
      F.dtype[F.n] = result_dtype[k];
      F.inst[F.n++] = I;
    }
    if (ph < n_reduce) {  // the value the reduce folds, "stored" (the kernel folds it instead)
      kapy_ew_inst St{};
      St.op = KAPY_EW_ST_GLOBAL;
      St.a = prog[C.stop[ph]].a;
      F.dtype[F.n] = reduce_dtype[ph];
      F.inst[F.n++] = St;
    }
  }
  size_t bytes = 0;
  float *block = reduce_scratch_lines(&bytes);
  if (!block) return 0;
  auto give_up = [&](int rc) { return rc; };
  // [results of up to four reduces, 4 bytes per column each][partial lines]
  const int64_t floats = (int64_t)(bytes / sizeof(float)), left = floats / n - kMaxColumnReduces;
  if (left < 1) return give_up(0);
  const int lpr = n >= 256 ? 32 : 8;
  const int64_t strips = (n / 8 + lpr - 1) / lpr, want = 4 * (int64_t)device_cus();
  int64_t chunks = std::max<int64_t>(1, std::min<int64_t>({(want + strips - 1) / strips, m / 64, 256, left}));
  const int32_t per_chunk = (int32_t)((m + chunks - 1) / chunks);
  chunks = (m + per_chunk - 1) / per_chunk;
  float *lines = block + kMaxColumnReduces * n;
  kapy_global views[kMaxInputs];
  const kapy_global *all[kMaxInputs];
  for (int k = 0; k < n_ins; ++k) all[k] = ins[k];
  for (int c = 0; c < n_reduce; ++c) {
    kapy_global &v = views[c];
    v.ptr = block + c * n;
    v.start0 = v.start1 = 0;
    v.end0 = 1;
    v.end1 = v.stride0 = (int32_t)n;
    v.stride1 = 1;
    v.dtype = reduce_dtype[c];
    v.alignment = 16;
    all[n_ins + c] = &v;
  }
  if (strips > 0x7fffffff || n >= (int64_t(1) << 31)) return give_up(0);
  // the reduce phases' stack programs (the value type of a phase is its reduce operand's: a pseudo-result of that type)
  std::vector<StackProgram> SP(n_reduce);
  for (int ph = 0; ph < n_reduce; ++ph) {
    kapy_global pseudo = *out;
    pseudo.ptr = lines;  // (an aligned address; never written)
    pseudo.start0 = pseudo.start1 = 0;
    pseudo.end0 = (int32_t)m;
    pseudo.end1 = pseudo.stride0 = (int32_t)n;
    pseudo.stride1 = 1;
    const Phase &F = phases[ph];
    // the operand's type: that of the instruction that defines the stored register last
    int operand_dtype = -1;
    for (int k = 0; k + 1 < F.n; ++k)
      if (F.inst[k].op != KAPY_EW_ST_GLOBAL && F.inst[k].dst == F.inst[F.n - 1].a) operand_dtype = F.dtype[k];
    if (operand_dtype < 0) return give_up(0);
    pseudo.dtype = operand_dtype;
    if (!build_stack_program(F.inst, F.n, F.dtype, all, n_ins + ph, &pseudo, &SP[ph], true) || SP[ph].width) return give_up(0);
  }
  for (int ph = 0; ph < n_reduce; ++ph) {
    const int sum = prog[C.stop[ph]].op == KAPY_EW_REDUCE_SUM;
    dim3 grid((unsigned)strips, (unsigned)chunks);
    if (lpr == 32) stack_colreduce_kernel<32><<<grid, 256, 0, s>>>(SP[ph], lines, per_chunk, sum);
    else stack_colreduce_kernel<8><<<grid, 256, 0, s>>>(SP[ph], lines, per_chunk, sum);
    column_fold_kernel<<<dim3((unsigned)((n + 255) / 256)), 256, 0, s>>>(lines, (int32_t)chunks, (int32_t)n, sum, reduce_dtype[ph], block + ph * n);
  }
  const Phase &L = phases[n_reduce];
  int rc = kapy_elementwise(L.inst, L.n, all, n_ins + n_reduce, out, (void *)s);
  return rc ? rc : 1;
}

// st(fptofp_rn[T](divf(E, reduce_sum0(E)))), E = exp(subf(F, reduce_max0(F))), F = extf(ld x): the input's index, or -1
int match_column_softmax(const kapy_ew_inst *prog, int n_inst, const int *result_dtype, const kapy_global *out) {
  struct N { int op, a = -1, b = -1, dtype = -1, rmode = KAPY_RN, input = -1, axis = 0; };
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
    switch (I.op) {
    case KAPY_EW_LD_GLOBAL: n.input = I.a; if (I.c != KAPY_PAD_ZERO) return -1; break;
    case KAPY_EW_ST_GLOBAL: stored = reg[I.a]; ++n_store; continue;
    case KAPY_EW_FPTOFP: case KAPY_EW_EXP: n.a = reg[I.a]; break;
    case KAPY_EW_REDUCE_SUM: case KAPY_EW_REDUCE_MAX: n.a = reg[I.a]; n.axis = I.b; break;
    case KAPY_EW_SUBF: case KAPY_EW_DIVF: n.a = reg[I.a]; n.b = reg[I.b]; break;
    default: return -1;
    }
    nodes.push_back(n);
    reg[I.dst] = (int)nodes.size() - 1;
  }
  const int T = out->dtype;
  if (n_store != 1 || stored < 0 || (T != KAPY_F16 && T != KAPY_BF16)) return -1;
  auto is = [&](int id, int op) { return id >= 0 && nodes[id].op == op && (op == KAPY_EW_LD_GLOBAL || nodes[id].dtype == KAPY_F32); };
  const N &st = nodes[stored];
  if (st.op != KAPY_EW_FPTOFP || st.dtype != T || st.rmode == KAPY_RZ || !is(st.a, KAPY_EW_DIVF)) return -1;
  const int e = nodes[st.a].a, rs = nodes[st.a].b;
  if (!is(rs, KAPY_EW_REDUCE_SUM) || nodes[rs].axis != 0 || nodes[rs].a != e || !is(e, KAPY_EW_EXP)) return -1;
  const int sub = nodes[e].a;
  if (!is(sub, KAPY_EW_SUBF)) return -1;
  const int f = nodes[sub].a, rm = nodes[sub].b;
  if (!is(rm, KAPY_EW_REDUCE_MAX) || nodes[rm].axis != 0 || nodes[rm].a != f || !is(f, KAPY_EW_FPTOFP)) return -1;
  const int ld = nodes[f].a;
  if (ld < 0 || nodes[ld].op != KAPY_EW_LD_GLOBAL || nodes[ld].dtype != T) return -1;
  return nodes[ld].input;
}

int run_column_program(const kapy_ew_inst *prog, int n_inst, const int *result_dtype, const kapy_global *const *ins, int n_ins, const kapy_global *out,
                       hipStream_t s) {
  {  // the softmax of every column has kernels of its own
    const int x_in = match_column_softmax(prog, n_inst, result_dtype, out);
    if (x_in >= 0 && x_in < n_ins) {
      const int ran = run_column_softmax(ins[x_in], out, s);
      if (ran != 0) return ran < 0 ? ran : KAPY_OK;
    }
  }
  Program P;
  memset(&P, 0, sizeof P);
  ColumnPlan C;
  memset(&C, 0, sizeof C);
  P.n_inst = n_inst;
  P.n_ins = n_ins;
  // def_of[r]: the instructions the current value of register r is computed from
  uint64_t def_of[kMaxRegs];
  memset(def_of, 0, sizeof def_of);
  int n_reduce = 0;
  uint64_t stores = 0;
  for (int k = 0; k < n_inst; ++k) {
    kapy_ew_inst I = prog[k];
    I.dtype = result_dtype[k];
    uint64_t d = uint64_t(1) << k;
    switch (I.op) {
    case KAPY_EW_LD_GLOBAL: case KAPY_EW_SPLAT: case KAPY_EW_ARANGE: break;
    case KAPY_EW_FMA: case KAPY_EW_SELECT: d |= def_of[I.a] | def_of[I.b] | def_of[I.c]; break;
    KAPY_EW_BINARY_CASES:
      d |= def_of[I.a] | def_of[I.b];
      break;
    case KAPY_EW_REDUCE_SUM: case KAPY_EW_REDUCE_MAX:
      if (n_reduce == kMaxColumnReduces)
        return fail(KAPY_ERR_UNSUPPORTED, "elementwise: a program may hold at most %d reduces along axis 0", kMaxColumnReduces);
      C.stop[n_reduce] = k;
      C.need[n_reduce] = def_of[I.a];  // what the operand is computed from; the reduce itself is the fold after the row loop
      I.c = n_reduce++;
      break;                           // later phases read the per-column result: nothing before it is needed for its sake
    default: d |= def_of[I.a];
    }
    if (I.op == KAPY_EW_ST_GLOBAL) stores |= d;
    else def_of[I.dst] = d;
    P.inst[k] = I;
  }
  C.stop[n_reduce] = n_inst;
  C.need[n_reduce] = stores;
  C.n_phases = n_reduce + 1;
  for (int k = 0; k < n_ins; ++k) P.in[k] = to_dev(ins[k]);
  for (int k = 0; k < n_inst; ++k)
    if (prog[k].op == KAPY_EW_LD_GLOBAL) P.in[prog[k].a].pad = padding_word_of(ins[prog[k].a]->dtype, prog[k].c);
  P.out = to_dev(out);
  {
    const int fast = run_column_phases(prog, n_inst, result_dtype, ins, n_ins, out, C, P, s);
    if (fast != 0) return fast < 0 ? fast : KAPY_OK;
  }
  const int64_t strips = (extent1(out) + 63) / 64;
  if (strips > 0x7fffffff) return fail(KAPY_ERR_UNSUPPORTED, "elementwise: too many columns for a program with reduces along axis 0");
  // many rows: more waves per strip
  if (extent0(out) >= 256) column_program_kernel<8><<<dim3((unsigned)strips), 512, 0, s>>>(P, C);
  else column_program_kernel<4><<<dim3((unsigned)strips), 256, 0, s>>>(P, C);
  KAPY_HIP_CHECK(hipGetLastError());
  return KAPY_OK;
}

// compiling and loading code objects are not stream work: they must not happen while a caller captures the stream into a graph
bool stream_is_capturing(hipStream_t s) {
  hipStreamCaptureStatus status = hipStreamCaptureStatusNone;
  return hipStreamIsCapturing(s, &status) == hipSuccess && status != hipStreamCaptureStatusNone;
}

}  // namespace
}  // namespace kapy

using namespace kapy;

extern "C" {

int kapy_elementwise(const kapy_ew_inst *prog, int32_t n_inst, const kapy_global *const *ins, int32_t n_ins,
                     const kapy_global *out, void *stream) {
  int result_dtype[kMaxInst];
  kapy_ew_inst normalised[kMaxInst];
  const kapy_ew_inst *as_given = prog;
  int rc = verify_program(prog, n_inst, ins, n_ins, out, result_dtype, normalised);
  if (rc) return rc;
  prog = normalised;
  rc = ensure_device();
  if (rc) return rc;
  const int64_t o0 = extent0(out), o1 = extent1(out);
  if (o0 <= 0 || o1 <= 0) return KAPY_OK;
  hipStream_t s = (hipStream_t)stream;

  // a kernel compiled for exactly this program and operand signature, if the caller asked for one
  rc = launch_specialized(prog, n_inst, result_dtype, ins, n_ins, out, s);
  if (rc != 0) return rc < 0 ? rc : KAPY_OK;

  bool has_reduce = false;
  for (int k = 0; k < n_inst; ++k) has_reduce |= prog[k].op == KAPY_EW_REDUCE_SUM || prog[k].op == KAPY_EW_REDUCE_MAX;
  // Integer registers and the ops on them (compare, select, casts, arange) run on the register machines and in compiled
  // kernels; the hand-written float kernels and the stack machines are not tried for such a program.  A program with an
  // arange depends on where an element sits, so it is never re-shaped (transposed problem, one-line form) either.
  bool has_int = is_int(out->dtype), has_arange = false;
  for (int k = 0; k < n_inst; ++k) {
    has_int |= prog[k].op >= KAPY_EW_ADDI || is_int(result_dtype[k]);
    has_arange |= prog[k].op == KAPY_EW_ARANGE;
  }

  // A column-major result: the same program on the transposed problem has a row-major one (every view with its axes
  // swapped - a row operand becomes a column operand and the other way round), which is what the fast kernels are written for.
  // Operands that are column-major too then read along their rows; the others are no worse off than before.
  if (!has_reduce && !has_arange && out->stride0 == 1 && out->stride1 != 1 && o1 > 1 && n_ins <= kMaxInputs) {
    auto swapped = [](const kapy_global *g) {
      kapy_global v = *g;
      std::swap(v.start0, v.start1);
      std::swap(v.end0, v.end1);
      std::swap(v.stride0, v.stride1);
      return v;
    };
    kapy_global views[kMaxInputs], result = swapped(out);
    const kapy_global *ptrs[kMaxInputs];
    for (int k = 0; k < n_ins; ++k) {
      views[k] = swapped(ins[k]);
      ptrs[k] = &views[k];
    }
    return kapy_elementwise(as_given, n_inst, ptrs, n_ins, &result, stream);
  }

  // Rows that are not a whole number of 8-element vectors move element by element (or, 16-bit only, with a ragged last
  // vector per row, and then only from aligned rows).  When the result and every operand are dense matrices of one shape
  // (pitch = width) or single elements, the program does not care where a row ends: it runs once over the first
  // 8 * floor(o0 * o1 / 8) elements as one line, in whole vectors, and once over the up to 7 that remain.
  if (!has_reduce && !has_arange && o0 > 1 && o1 % 8 != 0 && o0 * o1 < (int64_t(1) << 31) - 1024 && n_ins <= kMaxInputs) {
    auto dense = [&](const kapy_global *g) { return g->stride1 == 1 && g->stride0 == o1 && extent0(g) == o0 && extent1(g) == o1; };
    auto single = [](const kapy_global *g) { return extent0(g) == 1 && extent1(g) == 1; };
    bool flat = dense(out);
    for (int k = 0; k < n_ins; ++k) flat = flat && (dense(ins[k]) || single(ins[k]));
    if (flat) {
      const int64_t total = o0 * o1, whole = total / 8 * 8;
      auto line = [&](const kapy_global *g, int64_t first, int64_t count) {
        if (single(g)) return *g;
        kapy_global v = *g;
        v.ptr = (void *)(view_base(g) + first * dtype_bytes(g->dtype));
        v.start0 = v.start1 = 0;
        v.end0 = 1;
        v.end1 = v.stride0 = (int32_t)count;
        v.stride1 = 1;
        v.alignment = 16;
        while (v.alignment > 1 && ((uintptr_t)v.ptr & (uintptr_t)(v.alignment - 1))) v.alignment >>= 1;
        return v;
      };
      for (int part = 0; part < 2; ++part) {
        const int64_t first = part ? whole : 0, count = part ? total - whole : whole;
        if (count == 0) continue;
        kapy_global views[kMaxInputs], result = line(out, first, count);
        const kapy_global *ptrs[kMaxInputs];
        for (int k = 0; k < n_ins; ++k) {
          views[k] = line(ins[k], first, count);
          ptrs[k] = &views[k];
        }
        rc = kapy_elementwise(as_given, n_inst, ptrs, n_ins, &result, stream);
        if (rc) return rc;
      }
      return KAPY_OK;
    }
  }
  if (has_reduce) {
    int along[2] = {0, 0};
    for (int k = 0; k < n_inst; ++k)
      if (prog[k].op == KAPY_EW_REDUCE_SUM || prog[k].op == KAPY_EW_REDUCE_MAX) ++along[prog[k].b];
    if (along[0] && along[1])
      return fail(KAPY_ERR_UNSUPPORTED, "elementwise: the reduces of one program must run along the same axis (reduce the other axis with kapy_reduce first)");
    if (along[0]) return run_column_program(prog, n_inst, result_dtype, ins, n_ins, out, s);
    rc = has_int ? fail(KAPY_ERR_UNSUPPORTED, "elementwise: a program with a reduce along rows and integer registers runs as a compiled kernel only")
                 : run_row_program(prog, n_inst, result_dtype, ins, n_ins, out, s);
    if (rc != KAPY_ERR_UNSUPPORTED) return rc;
    // What the row machine refuses (a width that is not a multiple of 8, more than three row values in flight) a compiled
    // kernel may still serve: compile one now rather than turn the caller away.  Without the runtime compiler, or for a
    // program that fits neither, the row machine's refusal stands.
    const std::string refusal = last_error_buffer();
    if (stream_is_capturing(s))
      return fail(rc, "%s (a kernel compiled for the program could serve it, but nothing is compiled or loaded while the stream is being captured: "
                  "call kapy_elementwise_specialize before the capture)", refusal.c_str());
    if (specialize_program(prog, n_inst, result_dtype, ins, n_ins, out) == KAPY_OK && launch_specialized(prog, n_inst, result_dtype, ins, n_ins, out, s) == 1)
      return KAPY_OK;
    return fail(rc, "%s", refusal.c_str());
  }

  AffineActParams ap;
  int T = -1;
  if (!has_int && match_affine_act(prog, n_inst, ins, out, &ap, &T)) {
    uint32_t slots = (uint32_t)ap.rows * (uint32_t)ap.vec_per_row;
    const bool cols = (ap.bias_mode == kBiasRow || ap.bias_mode == kNoBias) && (ap.rows + 2 - 1) / 2 <= 65535;
    dim3 grid = cols ? dim3((ap.vec_per_row + 255) / 256, (ap.rows + 2 - 1) / 2)
                     : dim3((slots + 256 * kEwUnroll - 1) / (256 * kEwUnroll));
#define KAPY_LAUNCH_AFFINE(TT, AA)                                                     \
  do {                                                                                 \
    if (cols && ap.width) affine_act_cols_kernel<TT, AA, true><<<grid, 256, 0, s>>>(ap);  \
    else if (cols) affine_act_cols_kernel<TT, AA, false><<<grid, 256, 0, s>>>(ap);     \
    else if (ap.width) affine_act_kernel<TT, AA, true><<<grid, 256, 0, s>>>(ap);       \
    else affine_act_kernel<TT, AA, false><<<grid, 256, 0, s>>>(ap);                    \
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

  // A program that no hand-written kernel matches is compiled when it comes back: from its second call with the same operand
  // signature (the first runs on the stepwise machines below, so that no single call takes a compile unasked; a compile is a
  // fraction of a second, the first in a process seconds).  KAPY_EW_AUTO_SPECIALIZE=1: on its first call; =0: never.  Never
  // while the stream is capturing.  A program that cannot be compiled, or a machine without the runtime compiler, goes on below
  // and is not tried again.
  static const int compile_from_call = [] {
    const char *v = getenv("KAPY_EW_AUTO_SPECIALIZE");
    return !v || !v[0] ? 2 : v[0] == '0' ? 0 : v[0] == '1' ? 1 : 2;
  }();
  if (compile_from_call && !stream_is_capturing(s) && unmatched_call_wants_compile(prog, n_inst, result_dtype, ins, n_ins, out, compile_from_call)) {
    if (specialize_program(prog, n_inst, result_dtype, ins, n_ins, out) == KAPY_OK) {
      rc = launch_specialized(prog, n_inst, result_dtype, ins, n_ins, out, s);
      if (rc != 0) return rc < 0 ? rc : KAPY_OK;
    } else {
      unmatched_compile_failed(prog, n_inst, result_dtype, ins, n_ins, out);
    }
  }

  if (!has_int) {
    StackProgram SP;
    memset(&SP, 0, sizeof SP);
    if (build_stack_program(prog, n_inst, result_dtype, ins, n_ins, out, &SP)) {
      const int64_t slots = (int64_t)SP.rows * SP.vec_per_row;
      bool narrow = out->dtype == KAPY_F16 || out->dtype == KAPY_BF16;
      for (int k = 0; k < n_ins; ++k) narrow = narrow && (ins[k]->dtype == KAPY_F16 || ins[k]->dtype == KAPY_BF16);
      for (int k = 0; k < n_inst; ++k) narrow = narrow && !is_f8(result_dtype[k]);
      bool heavy = false;
      for (int k = 0; k < n_inst; ++k) heavy = heavy || prog[k].op == KAPY_EW_REMF || prog[k].op == KAPY_EW_SIN || prog[k].op == KAPY_EW_COS;
      if (narrow && SP.width) stack_kernel_narrow_ragged<<<dim3((unsigned)((slots + 255) / 256)), 256, 0, s>>>(SP);
      else if (narrow && heavy) stack_kernel_narrow_heavy<<<dim3((unsigned)((slots + 255) / 256)), 256, 0, s>>>(SP);
      else if (narrow) stack_kernel_narrow<<<dim3((unsigned)((slots + 255) / 256)), 256, 0, s>>>(SP);
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

int kapy_elementwise_specialize(const kapy_ew_inst *prog, int32_t n_inst, const kapy_global *const *ins, int32_t n_ins, const kapy_global *out) {
  int result_dtype[kMaxInst];
  kapy_ew_inst normalised[kMaxInst];
  int rc = verify_program(prog, n_inst, ins, n_ins, out, result_dtype, normalised);
  if (rc) return rc;
  prog = normalised;
  rc = ensure_device();
  if (rc) return rc;
  // act(x*s + bias) with the GELU or no activation already has a hand-written kernel with the activation compiled in:
  // nothing to gain from another one
  AffineActParams ap;
  int T = -1;
  if (match_affine_act(prog, n_inst, ins, out, &ap, &T) && (ap.act < 0 || ap.act == KAPY_EW_GELU_TANH)) return KAPY_OK;
  return specialize_program(prog, n_inst, result_dtype, ins, n_ins, out);
}

int kapy_elementwise_specialize_stats(int64_t *loaded, int64_t *launches) {
  specialized_stats(loaded, launches);
  return KAPY_OK;
}

int kapy_elementwise_source(const kapy_ew_inst *prog, int32_t n_inst, const kapy_global *const *ins, int32_t n_ins, const kapy_global *out,
                            char *source, int64_t capacity, int64_t *source_bytes, int64_t *code_bytes) {
  int result_dtype[kMaxInst];
  kapy_ew_inst normalised[kMaxInst];
  int rc = verify_program(prog, n_inst, ins, n_ins, out, result_dtype, normalised);
  if (rc) return rc;
  prog = normalised;
  return specialized_source(prog, n_inst, result_dtype, ins, n_ins, out, source, capacity, source_bytes, code_bytes);
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
