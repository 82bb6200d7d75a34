// elementwise_jit.cpp — specialised kernels for elementwise programs.
//
// The reference compiles every function once to device code and launches that
// (python/src/passes.cc:141-261: translate_mlir_to_llvm, translate_llvm_to_ptx); the machines of
// elementwise.hip instead walk a program step by step on the device, which costs vector-ALU issue slots per step.
// kapy_elementwise_specialize closes that gap for programs the hand-written kernels do not match: it writes the
// program out as straight-line HIP over the same device helpers the machines use (the text of numeric.hpp and
// ew_machine.hpp is embedded at build time, so rounding and special cases are the machines' own), compiles it for
// gfx950 with the runtime compiler (libhiprtc, opened on first use; absent => KAPY_ERR_UNSUPPORTED and the machines keep
// serving), loads the code object and keeps it in a process-wide table keyed by program and operand signature.
// kapy_elementwise looks a verified program up in that table before it falls back to the machines.
//
// Two skeletons.  A program without a reduce: two vectors of 8 elements per lane, every load issued before any
// arithmetic.  A program with reduces along the rows (the row machine's business otherwise): a workgroup keeps a
// whole row in registers, CH vectors per lane, walks rows blockIdx.x, +gridDim.x, ... with the next row's loads in
// flight, and evaluates the program with row values (CH x 8 registers) and per-row values (one register).
#include <dlfcn.h>
#include <hip/hiprtc.h>
#include <stdlib.h>
#include <string.h>
#include <unistd.h>

#include <algorithm>
#include <atomic>
#include <map>
#include <mutex>
#include <string>
#include <vector>

#include "common.hpp"

namespace kapy {
namespace {

// what the generated kernel takes; the same text is part of every generated source
constexpr int kJitInputs = 8;
struct JitArgs {
  const char *in[kJitInputs];
  int64_t stride0[kJitInputs];
  char *out;
  int64_t out_stride0;
  int32_t rows, vec_per_row;
  int32_t width;  // elements per row (vec_per_row * 8, or less when the last vector of a row is partial)
};
const char *kArgsText = R"(
struct JitArgs {
  const char *in[8];
  int64_t stride0[8];
  char *out;
  int64_t out_stride0;
  int32_t rows, vec_per_row;
  int32_t width;
};
// The ragged end of a row: only the first `valid` (1..7) elements of vector jv exist; a whole-vector access would reach
// past the view (and possibly past its allocation), so they move one by one.
__device__ __forceinline__ Raw8 fetch8_partial(const StackIn &g, int32_t i, int32_t jv, int valid) {
  const int eb = dtype_elem_bytes(g.dtype);
  const char *ptr = g.base + ((g.kind == kInRow ? 0 : i * g.stride0) + (int64_t)jv * 8) * eb;
  Raw8 r;
  r.lo = r.hi = u32x4{0, 0, 0, 0};
  if (eb == 2) r.lo = load16_partial(ptr, valid);
  else if (eb == 4) {
#pragma unroll
    for (int e = 0; e < 8; ++e)
      if (e < valid) {
        const uint32_t w = ((const uint32_t *)ptr)[e];
        if (e < 4) r.lo[e & 3] = w;
        else r.hi[e & 3] = w;
      }
  } else {
#pragma unroll
    for (int e = 0; e < 8; ++e)
      if (e < valid) r.lo[e >> 2] |= (uint32_t)((const uint8_t *)ptr)[e] << (8 * (e & 3));
  }
  return r;
}
template <bool RAGGED>
__device__ __forceinline__ Raw8 fetch8_row(const StackIn &g, int32_t i, int32_t jv, int32_t width, bool streaming) {
  if (RAGGED && (jv + 1) * 8 > width) return fetch8_partial(g, i, jv, width - jv * 8);
  return fetch8(g, i, jv, streaming);
}
template <bool NARROW, bool RAGGED>
__device__ __forceinline__ void store8_row(char *out, int dtype, int64_t row_start, int32_t jv, int32_t width, const float (&f)[8]) {
  if (RAGGED && (jv + 1) * 8 > width) {
#pragma unroll
    for (int e = 0; e < 8; ++e)
      if (jv * 8 + e < width) store_from_f32(out, dtype, row_start + jv * 8 + e, f[e]);
    return;
  }
  store8<NARROW>(out, dtype, row_start + (int64_t)jv * 8, f);
}
// Elements (il, 8*jl .. 8*jl+7) of a tile (64 columns wide) staged as it lies in a column-major operand's memory (stage[column][row], PITCH
// bytes per column), as the 8-element memory image a row-major operand would have given.
template <int EB, int PITCH>
__device__ __forceinline__ Raw8 gather8(const char *stage, int il, int jl) {
  Raw8 r;
  r.lo = r.hi = u32x4{0, 0, 0, 0};
#pragma unroll
  for (int e = 0; e < 8; ++e) {
    const char *at = stage + (jl * 8 + e) * PITCH + il * EB;
    if (EB == 2) r.lo[e >> 1] |= (uint32_t)(*(const uint16_t *)at) << (16 * (e & 1));
    else if (EB == 4) {
      const uint32_t w = *(const uint32_t *)at;
      if (e < 4) r.lo[e & 3] = w;
      else r.hi[e & 3] = w;
    } else r.lo[e >> 2] |= (uint32_t)(*(const uint8_t *)at) << (8 * (e & 3));
  }
  return r;
}
__device__ __forceinline__ void fill8(float (&x)[8], float v) {
#pragma unroll
  for (int e = 0; e < 8; ++e) x[e] = v;
}
__device__ __forceinline__ void copy8(float (&x)[8], const float (&y)[8]) {
#pragma unroll
  for (int e = 0; e < 8; ++e) x[e] = y[e];
}
// Sum or maximum of one row value over its row (the row machine's reduce step): each lane folds its active chunks, a
// butterfly folds the wave, the waves meet in `red` (one barrier).  A NaN anywhere makes the maximum NaN.
template <int CH, int THREADS, bool SUM, bool RAGGED>
__device__ __forceinline__ float row_reduce(const float (&v)[CH][8], int32_t vec_per_row, int32_t width, float *red) {
  const int tid = threadIdx.x;
  float acc = SUM ? -0.f : -__builtin_inff();
#pragma unroll
  for (int c = 0; c < CH; ++c) {
    const int32_t jv = c * THREADS + tid;
    if (RAGGED && jv < vec_per_row && (jv + 1) * 8 > width) {  // the row's last, partial vector: its first elements only
#pragma unroll
      for (int e = 0; e < 8; ++e)
        if (jv * 8 + e < width) acc = SUM ? acc + v[c][e] : max_nan(acc, v[c][e]);
    } else if (jv < vec_per_row) {
      float part;
      if (SUM) part = ((v[c][0] + v[c][1]) + (v[c][2] + v[c][3])) + ((v[c][4] + v[c][5]) + (v[c][6] + v[c][7]));
      else {
        part = fmaxf(fmaxf(fmaxf(v[c][0], v[c][1]), fmaxf(v[c][2], v[c][3])), fmaxf(fmaxf(v[c][4], v[c][5]), fmaxf(v[c][6], v[c][7])));
        bool any_nan = false;
#pragma unroll
        for (int e = 0; e < 8; ++e) any_nan |= v[c][e] != v[c][e];
        if (any_nan) part = __builtin_nanf("");
      }
      acc = SUM ? acc + part : max_nan(acc, part);
    }
  }
#pragma unroll
  for (int off = 32; off >= 1; off >>= 1) {
    const float other = __shfl_xor(acc, off, 64);
    acc = SUM ? acc + other : max_nan(acc, other);
  }
  if (THREADS > 64) {
    constexpr int WAVES = THREADS / 64;
    if ((tid & 63) == 0) red[tid >> 6] = acc;
    __syncthreads();
    acc = red[0];
#pragma unroll
    for (int w = 1; w < WAVES; ++w) acc = SUM ? acc + red[w] : max_nan(acc, red[w]);
  }
  return acc;
}
// The lane's CH vectors of one row of an operand (vector c*THREADS + lane; nothing is read past the row's end).
template <int CH, int THREADS, bool RAGGED>
__device__ __forceinline__ void row_fetch8(const StackIn &g, int32_t i, int32_t vec_per_row, int32_t width, bool streaming, Raw8 (&raw)[CH]) {
#pragma unroll
  for (int c = 0; c < CH; ++c) {
    const int32_t jv = c * THREADS + (int32_t)threadIdx.x;
    raw[c].lo = raw[c].hi = u32x4{0, 0, 0, 0};
    if (jv < vec_per_row) raw[c] = fetch8_row<RAGGED>(g, i, jv, width, streaming);
  }
}
)";

const char *kPrelude =
    "typedef signed char int8_t; typedef unsigned char uint8_t; typedef short int16_t; typedef unsigned short uint16_t;\n"
    "typedef int int32_t; typedef unsigned int uint32_t; typedef long int64_t; typedef unsigned long uint64_t;\n"
    "typedef unsigned long uintptr_t;\n"
#include "jit_headers.inc"
    ;

constexpr int kTileRows = 64;  // rows of a tile of the tiled skeleton (64 columns wide): 32 per vector a lane handles
enum Kind { kFull = 0, kRow = 1, kCol = 2, kScalar = 3, kColMajor = 4 /* full extent, contiguous along axis 0 */ };

struct Signature {
  int n_ins = 0;
  int in_dtype[kJitInputs], in_kind[kJitInputs];
  int out_dtype = 0;
  bool narrow = true;
  bool ragged = false;       // the width is not a multiple of 8: the last vector of every row moves element by element
  bool tiled = false;        // an operand is column-major: 64 x 64 tiles, such operands staged through LDS
  bool rowwise = false;      // the program reduces along rows: the row skeleton, compiled for one (threads, chunks) shape
  int threads = 256, chunks = 1;
};

// An operand as the kernels see it.  When the result is column-major (contiguous along axis 0) the whole problem is
// looked at transposed: extents and strides of every operand swap, the result becomes row-major and row-major operands
// column-major - a store with swapped strides is a load with swapped strides of the transposed problem.
struct View {
  const char *base;
  int64_t e0, e1, s0, s1;
  int dtype;
};
void canonical_views(const kapy_global *const *ins, int n_ins, const kapy_global *out, View *vi, View *vo) {
  const bool swap = out->stride1 != 1 && out->stride0 == 1;
  auto view = [&](const kapy_global *g) {
    View v{view_base(g), extent0(g), extent1(g), g->stride0, g->stride1, g->dtype};
    if (swap) {
      std::swap(v.e0, v.e1);
      std::swap(v.s0, v.s1);
    }
    return v;
  };
  *vo = view(out);
  for (int k = 0; k < n_ins; ++k) vi[k] = view(ins[k]);
}

// Which programs a specialised kernel serves and how each operand is read: the result contiguous along rows (after the
// transposition above) with rows that start aligned to 8 elements; operands full (row- or column-major, 16-byte
// aligned along their contiguous axis), one row, one column or a scalar; no padding pattern other than zero, one store,
// reduces only along rows.
bool classify(const kapy_ew_inst *prog, int n_inst, const int *result_dtype, const kapy_global *const *ins, int n_ins, const kapy_global *out,
              Signature *sig, View *vi, View *vo) {
  if (n_ins > kJitInputs) return false;
  int stores = 0;
  for (int k = 0; k < n_inst; ++k) {
    const int op = prog[k].op;
    if (op == KAPY_EW_REDUCE_SUM || op == KAPY_EW_REDUCE_MAX) {
      if (prog[k].b != 1) return false;  // along columns: not resident per workgroup
      sig->rowwise = true;
    }
    if (op == KAPY_EW_LD_GLOBAL && prog[k].c != KAPY_PAD_ZERO) return false;
    if (op == KAPY_EW_ARANGE && out->stride1 != 1) return false;  // (an arange names its axis: no transposed view of it)
    stores += op == KAPY_EW_ST_GLOBAL;
  }
  if (stores != 1) return false;
  canonical_views(ins, n_ins, out, vi, vo);
  if (sig->rowwise && out->stride1 != 1) return false;  // (a reduce names its axis: no transposed view of it)
  const int64_t o0 = vo->e0, o1 = vo->e1;
  const int ob = dtype_bytes(out->dtype);
  if (!(is_float(out->dtype) || is_int(out->dtype)) || vo->s1 != 1) return false;
  if (((uintptr_t)vo->base % (8 * ob)) || (vo->s0 * ob) % (8 * ob)) return false;
  if (o0 * ((o1 + 7) / 8) >= (int64_t(1) << 31) - 1024) return false;
  sig->ragged = o1 % 8 != 0;
  if (sig->rowwise) {
    const int64_t vpr = (o1 + 7) / 8;
    if (vpr > 4096) return false;  // a row of more than 32768 elements does not stay in one workgroup's registers
    sig->threads = vpr <= 256 ? 64 : vpr <= 1024 ? 256 : 1024;
    sig->chunks = (int)((vpr + sig->threads - 1) / sig->threads);
  }
  sig->n_ins = n_ins;
  sig->out_dtype = out->dtype;
  sig->narrow = out->dtype == KAPY_F16 || out->dtype == KAPY_BF16;
  for (int k = 0; k < n_inst; ++k) sig->narrow = sig->narrow && !is_f8(result_dtype[k]) && !is_int(result_dtype[k]);
  int staged_bytes = 0;
  for (int k = 0; k < n_ins; ++k) {
    const View &g = vi[k];
    if (!is_float(g.dtype) && !is_int(g.dtype)) return false;
    sig->narrow = sig->narrow && (g.dtype == KAPY_F16 || g.dtype == KAPY_BF16);
    const int eb = dtype_bytes(g.dtype);
    const bool vec_ok = g.s1 == 1 && ((uintptr_t)g.base % (8 * eb)) == 0 && (g.e0 == 1 || (g.s0 * eb) % (8 * eb) == 0);  // (one row: no pitch to align)
    // column-major: 16-byte pieces along axis 0, whole ones only
    const bool col_major_ok = g.s0 == 1 && ((uintptr_t)g.base % 16) == 0 && (g.s1 * eb) % 16 == 0 && (g.e0 * eb) % 16 == 0 && g.s1 >= 0 &&
                              !sig->rowwise && !sig->ragged;
    sig->in_dtype[k] = g.dtype;
    if (g.e0 == o0 && g.e1 == o1 && vec_ok) sig->in_kind[k] = kFull;
    else if (g.e0 == 1 && g.e1 == o1 && vec_ok) sig->in_kind[k] = kRow;
    else if (g.e1 == 1 && g.e0 == o0) sig->in_kind[k] = kCol;
    else if (g.e0 == 1 && g.e1 == 1) sig->in_kind[k] = kScalar;
    else if (g.e0 == o0 && g.e1 == o1 && col_major_ok) {
      sig->in_kind[k] = kColMajor;
      sig->tiled = true;
      staged_bytes += 64 * (kTileRows * eb + 16);
    } else return false;
  }
  return staged_bytes <= 60 * 1024;
}

std::string make_key(const kapy_ew_inst *prog, int n_inst, const Signature &sig) {
  std::string key;
  key.reserve(n_inst * sizeof(kapy_ew_inst) + 64);
  for (int k = 0; k < n_inst; ++k) {
    kapy_ew_inst I = prog[k];  // fields an op does not read must not tell two equal programs apart
    const int op = I.op;
    const bool int_binary_op = (op >= KAPY_EW_ADDI && op <= KAPY_EW_MINUI) || op == KAPY_EW_CMPI || op == KAPY_EW_CMPF;
    const bool int_cast = op >= KAPY_EW_TRUNCI && op <= KAPY_EW_BITCAST;
    const bool unary_or_cast = !(op == KAPY_EW_LD_GLOBAL || op == KAPY_EW_SPLAT || op == KAPY_EW_FMA || op == KAPY_EW_ADDF || op == KAPY_EW_SUBF ||
                                 op == KAPY_EW_MULF || op == KAPY_EW_DIVF || op == KAPY_EW_MAXIMUMF || op == KAPY_EW_MINIMUMF || op == KAPY_EW_MAXNUMF ||
                                 op == KAPY_EW_MINNUMF || op == KAPY_EW_REMF || int_binary_op || op == KAPY_EW_SELECT || op == KAPY_EW_ARANGE);
    if (op == KAPY_EW_SPLAT) {
      I.b = I.c = 0;
      if (is_int(I.dtype)) I.imm = 0.f;   // an integer splat's value is field a
      else I.a = 0;
    } else I.imm = 0.f;
    if (op == KAPY_EW_LD_GLOBAL) I.b = 0;
    if (unary_or_cast) I.b = I.c = 0;
    if (op != KAPY_EW_FMA && op != KAPY_EW_SELECT && op != KAPY_EW_CMPI && op != KAPY_EW_CMPF && !unary_or_cast && op != KAPY_EW_LD_GLOBAL) I.c = 0;
    if (op != KAPY_EW_FPTOFP) I.rmode = 0;
    if (op != KAPY_EW_FPTOFP && op != KAPY_EW_SPLAT && !int_cast) I.dtype = 0;
    if (op == KAPY_EW_ST_GLOBAL) I.dst = 0;
    key.append((const char *)&I, sizeof I);
  }
  for (int k = 0; k < sig.n_ins; ++k) {
    key.push_back((char)sig.in_dtype[k]);
    key.push_back((char)sig.in_kind[k]);
  }
  key.push_back((char)sig.out_dtype);
  key.push_back((char)sig.ragged);
  key.push_back((char)sig.tiled);
  if (sig.rowwise) {
    key.push_back((char)(sig.threads / 64));
    key.push_back((char)sig.chunks);
  }
  return key;
}

void appendf(std::string &s, const char *fmt, ...) __attribute__((format(printf, 2, 3)));
void appendf(std::string &s, const char *fmt, ...) {
  char buf[1024];
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(buf, sizeof buf, fmt, ap);
  va_end(ap);
  s += buf;
}

struct Node {
  int op, a = -1, b = -1, c = -1, dtype = -1, rmode = KAPY_RN, input = -1;
  float imm = 0.f;
  int ia = 0, ib = 0, ic = 0;  // the instruction's integer fields as given (an integer splat's value, arange's start and axis, a predicate)
  bool used = false;
  std::string name;  // the array, register or constant holding the value
  bool is_const = false;
  bool uniform = false;  // row skeleton: one value per row (a reduce's result, a column or scalar operand, a splat, and what follows from those)
};

// The program's values in program order (the store is not one of them: its operand's index goes to *stored), with
// `used` set on those the store depends on.
std::vector<Node> build_nodes(const kapy_ew_inst *prog, int n_inst, const int *result_dtype, int *stored, std::vector<char> *input_used) {
  std::vector<Node> nodes;
  int reg[64];
  for (int &r : reg) r = -1;
  *stored = -1;
  for (int k = 0; k < n_inst; ++k) {
    const kapy_ew_inst &I = prog[k];
    Node n;
    n.op = I.op;
    n.dtype = result_dtype[k];
    n.rmode = I.rmode;
    n.imm = I.imm;
    n.ia = I.a;
    n.ib = I.b;
    n.ic = I.c;
    switch (I.op) {
    case KAPY_EW_LD_GLOBAL: n.input = I.a; break;
    case KAPY_EW_SPLAT: case KAPY_EW_ARANGE: break;
    case KAPY_EW_ST_GLOBAL: *stored = reg[I.a]; continue;
    case KAPY_EW_FMA: case KAPY_EW_SELECT: n.a = reg[I.a]; n.b = reg[I.b]; n.c = reg[I.c]; break;
    KAPY_EW_BINARY_CASES:
      n.a = reg[I.a]; n.b = reg[I.b]; break;
    default: n.a = reg[I.a];
    }
    nodes.push_back(n);
    reg[I.dst] = (int)nodes.size() - 1;
  }
  std::vector<int> todo{*stored};
  while (!todo.empty()) {
    const int id = todo.back();
    todo.pop_back();
    if (id < 0 || nodes[id].used) continue;
    nodes[id].used = true;
    todo.push_back(nodes[id].a);
    todo.push_back(nodes[id].b);
    todo.push_back(nodes[id].c);
  }
  input_used->assign(kJitInputs, 0);
  for (const Node &n : nodes)
    if (n.used && n.op == KAPY_EW_LD_GLOBAL) (*input_used)[n.input] = 1;
  return nodes;
}

std::string source_head() {
  std::string s = kPrelude;
  s += "namespace kapy { namespace {\n";
  s += kArgsText;
  s += "} }\nusing namespace kapy;\n";
  return s;
}

// splats: one rounding to the splat's type, as the machines do when they push an immediate
void emit_splats(std::string &s, std::vector<Node> &nodes) {
  for (size_t id = 0; id < nodes.size(); ++id) {
    Node &n = nodes[id];
    if (!n.used || n.op != KAPY_EW_SPLAT) continue;
    uint32_t bits;
    memcpy(&bits, &n.imm, 4);
    n.name = "c" + std::to_string(id);
    n.is_const = n.uniform = true;
    if (is_int(n.dtype)) appendf(s, "  const float %s = int_reg(int_canon((int32_t)0x%08xu, %d));\n", n.name.c_str(), (uint32_t)n.ia, n.dtype);
    else appendf(s, "  const float %s = round_to_dtype(bits_f32(0x%08xu), %d, true);\n", n.name.c_str(), bits, n.dtype);
  }
}

// The per-element expression of an op on integer registers, or one that makes or consumes them (compare, select, the
// integer casts, arange), over the operands' expressions A, B, C; idx0 / idx1: the element's position along the two axes.
// Empty for every other op.
std::string int_op_expr(const Node &n, const std::vector<Node> &nodes, const std::string &A, const std::string &B, const std::string &C,
                        const std::string &idx0, const std::string &idx1) {
  const std::string op = std::to_string(n.op), dt = std::to_string(n.dtype);
  if (n.op == KAPY_EW_ARANGE) return "int_reg(" + std::to_string(n.ia) + " + " + (n.ib ? idx1 : idx0) + ")";
  if (n.op == KAPY_EW_SELECT) return "((reg_int(" + A + ") & 1) ? " + B + " : " + C + ")";
  if (n.op == KAPY_EW_CMPI) return "int_reg(int_compare(" + std::to_string(n.ic) + ", reg_int(" + A + "), reg_int(" + B + "), " + std::to_string(nodes[n.a].dtype) + "))";
  if (n.op == KAPY_EW_CMPF) return "int_reg(float_compare(" + std::to_string(n.ic) + ", " + A + ", " + B + "))";
  if (n.op == KAPY_EW_ABSI || (n.op >= KAPY_EW_TRUNCI && n.op <= KAPY_EW_BITCAST)) return "convert_reg(" + op + ", " + A + ", " + std::to_string(nodes[n.a].dtype) + ", " + dt + ")";
  if (n.op >= KAPY_EW_ADDI && n.op <= KAPY_EW_MINUI) return "int_reg(int_binary(" + op + ", reg_int(" + A + "), reg_int(" + B + "), " + dt + "))";
  return "";
}

// A program without a reduce as straight-line code: every value that the store depends on becomes one array of 8 fp32
// (the exact image of the typed value, rounded to the op's result type after every op, as the machines do), a splat one
// constant.
std::string generate_flat(const kapy_ew_inst *prog, int n_inst, const int *result_dtype, const Signature &sig, const std::string &name) {
  int stored = -1;
  std::vector<char> input_used;
  std::vector<Node> nodes = build_nodes(prog, n_inst, result_dtype, &stored, &input_used);
  std::string s = source_head();
  appendf(s, "extern \"C\" __global__ __launch_bounds__(256) void %s(JitArgs p) {\n", name.c_str());
  appendf(s, "  constexpr bool NARROW = %s, RAGGED = %s;\n", sig.narrow ? "true" : "false", sig.ragged ? "true" : "false");
  if (sig.tiled) {
    // 64 x 64 tiles, walked diagonally (tile row + tile column mod the number of tile rows) so that the tiles in flight
    // spread over the memory channels along both axes.  A column-major operand's tile is copied to LDS as it lies in
    // memory, 16 bytes per lane along its contiguous axis, and read from there along the other.
    appendf(s, "  const uint32_t tiles_j = (uint32_t)(p.vec_per_row + 7) / 8u, tiles_i = (uint32_t)(p.rows + %d) / %du;\n"
               "  const uint32_t tile_j = blockIdx.x %% tiles_j, tile_i = (blockIdx.x / tiles_j + tile_j) %% tiles_i;\n"
               "  const int32_t i0 = (int32_t)tile_i * %d, j0 = (int32_t)tile_j * 64;\n", kTileRows - 1, kTileRows, kTileRows);
    for (int k = 0; k < sig.n_ins; ++k) {
      if (!input_used[k] || sig.in_kind[k] != kColMajor) continue;
      const int eb = dtype_bytes(sig.in_dtype[k]), pitch = kTileRows * eb + 16, vec = 16 / eb, per_col = kTileRows / vec;
      appendf(s, "  __shared__ __attribute__((aligned(16))) char stage%d[64 * %d];\n", k, pitch);
      appendf(s, "  for (int v = threadIdx.x; v < 64 * %d; v += 256) {\n    const int jc = v / %d, iv = v %% %d;\n"
                 "    const int32_t j = j0 + jc, i = i0 + iv * %d;\n    u32x4 w = {0, 0, 0, 0};\n"
                 "    if (j < p.width && i < p.rows) w = __builtin_nontemporal_load((const u32x4 *)(p.in[%d] + ((int64_t)j * p.stride0[%d] + i) * %d));\n"
                 "    *(u32x4 *)(stage%d + jc * %d + iv * 16) = w;\n  }\n",
              per_col, per_col, per_col, vec, k, k, eb, k, pitch);
    }
    s += "  __syncthreads();\n";
  } else {
    s += "  const uint32_t total = (uint32_t)p.rows * (uint32_t)p.vec_per_row;\n"
         "  const uint32_t first = blockIdx.x * 512u + threadIdx.x;\n";
  }
  const int U = sig.tiled ? kTileRows / 32 : 2;  // vectors of 8 per lane
  appendf(s, "  constexpr int U = %d;\n  int32_t row[U], jv[U];\n", U);
  for (int k = 0; k < sig.n_ins; ++k) {
    if (!input_used[k]) continue;
    if (sig.in_kind[k] == kFull || sig.in_kind[k] == kRow || sig.in_kind[k] == kColMajor) appendf(s, "  Raw8 raw%d[U];\n", k);
    else appendf(s, "  float raw%d[U];\n", k);
  }
  emit_splats(s, nodes);
  if (sig.tiled)
    s += "#pragma unroll\n  for (int u = 0; u < U; ++u) {\n"
         "    const int il = (int)(u * 256 + threadIdx.x) >> 3, jl = (int)threadIdx.x & 7;\n"
         "    row[u] = -1;\n"
         "    if (i0 + il < p.rows && (int32_t)tile_j * 8 + jl < p.vec_per_row) {\n"
         "      row[u] = i0 + il;\n"
         "      jv[u] = (int32_t)tile_j * 8 + jl;\n";
  else
    s += "#pragma unroll\n  for (int u = 0; u < U; ++u) {\n"
         "    const uint32_t slot = first + u * 256u;\n"
         "    row[u] = -1;\n"
         "    if (slot < total) {\n"
         "      row[u] = (int32_t)(slot / (uint32_t)p.vec_per_row);\n"
         "      jv[u] = (int32_t)(slot - (uint32_t)row[u] * (uint32_t)p.vec_per_row);\n";
  for (int k = 0; k < sig.n_ins; ++k) {
    if (!input_used[k]) continue;
    const int kind = sig.in_kind[k], dt = sig.in_dtype[k];
    if (kind == kColMajor)
      appendf(s, "      raw%d[u] = gather8<%d, %d>(stage%d, il, jl);\n", k, dtype_bytes(dt), kTileRows * dtype_bytes(dt) + 16, k);
    else if (kind == kFull || kind == kRow)
      appendf(s, "      { const StackIn g{p.in[%d], p.stride0[%d], %d, %d}; raw%d[u] = fetch8_row<RAGGED>(g, row[u], jv[u], p.width, %s); }\n", k, k, dt,
              kind == kFull ? 0 : 1, k, kind == kFull ? "true" : "false");
    else
      appendf(s, "      raw%d[u] = load_as_f32(p.in[%d], %d, %s);\n", k, k, dt, kind == kCol ? ("row[u] * p.stride0[" + std::to_string(k) + "]").c_str() : "0");
  }
  s += "    }\n  }\n#pragma unroll\n  for (int u = 0; u < U; ++u) {\n    if (row[u] < 0) continue;\n";
  auto elem = [&](int id) { return nodes[id].is_const ? nodes[id].name : nodes[id].name + "[e]"; };
  // an operand as an array of 8 (div8 and the store take arrays)
  int n_filled = 0;
  auto as_array = [&](int id) {
    if (!nodes[id].is_const) return nodes[id].name;
    const std::string a = "a" + std::to_string(n_filled++) + nodes[id].name;
    appendf(s, "    float %s[8]; fill8(%s, %s);\n", a.c_str(), a.c_str(), nodes[id].name.c_str());
    return a;
  };
  for (size_t id = 0; id < nodes.size(); ++id) {
    Node &n = nodes[id];
    if (!n.used || n.op == KAPY_EW_SPLAT) continue;
    const std::string v = "v" + std::to_string(id);
    const char *vn = v.c_str();
    auto round_result = [&]() {
      if (n.dtype != KAPY_F32) appendf(s, "    round8<NARROW>(%s, %d, true);\n", vn, n.dtype);
    };
    auto per_element = [&](const std::string &expr) {
      appendf(s, "    float %s[8];\n#pragma unroll\n    for (int e = 0; e < 8; ++e) %s[e] = %s;\n", vn, vn, expr.c_str());
    };
    n.name = v;
    {
      const std::string ie = int_op_expr(n, nodes, n.a >= 0 ? elem(n.a) : "", n.b >= 0 ? elem(n.b) : "", n.c >= 0 ? elem(n.c) : "", "row[u]", "(jv[u] * 8 + e)");
      if (!ie.empty()) {
        per_element(ie);
        continue;
      }
    }
    switch (n.op) {
    case KAPY_EW_LD_GLOBAL: {
      const int k = n.input, kind = sig.in_kind[k];
      if (kind == kFull || kind == kRow || kind == kColMajor) appendf(s, "    float %s[8]; widen8(raw%d[u], %d, %s);\n", vn, k, sig.in_dtype[k], vn);
      else appendf(s, "    float %s[8]; fill8(%s, raw%d[u]);\n", vn, vn, k);
      break;
    }
    case KAPY_EW_FPTOFP: {
      // values are fp32 images of typed values: widening to f32 changes nothing, and the store rounds to nearest itself
      const bool free_cast = n.dtype == KAPY_F32 || ((int)id == stored && n.dtype == sig.out_dtype && n.rmode != KAPY_RZ);
      if (free_cast) {
        n.name = nodes[n.a].name;
        n.is_const = nodes[n.a].is_const;
      } else {
        per_element(elem(n.a));
        appendf(s, "    round8<NARROW>(%s, %d, %s);\n", vn, n.dtype, n.rmode != KAPY_RZ ? "true" : "false");
      }
      break;
    }
    case KAPY_EW_ADDF: per_element("__fadd_rn(" + elem(n.a) + ", " + elem(n.b) + ")"); round_result(); break;
    case KAPY_EW_SUBF: per_element("__fsub_rn(" + elem(n.a) + ", " + elem(n.b) + ")"); round_result(); break;
    case KAPY_EW_MULF: per_element("__fmul_rn(" + elem(n.a) + ", " + elem(n.b) + ")"); round_result(); break;
    case KAPY_EW_MAXIMUMF: per_element("max_nan(" + elem(n.a) + ", " + elem(n.b) + ")"); round_result(); break;
    case KAPY_EW_MINIMUMF: per_element("min_nan(" + elem(n.a) + ", " + elem(n.b) + ")"); round_result(); break;
    case KAPY_EW_MAXNUMF: per_element("max_num(" + elem(n.a) + ", " + elem(n.b) + ")"); round_result(); break;
    case KAPY_EW_MINNUMF: per_element("min_num(" + elem(n.a) + ", " + elem(n.b) + ")"); round_result(); break;
    case KAPY_EW_REMF: per_element("rem_f(" + elem(n.a) + ", " + elem(n.b) + ")"); round_result(); break;
    case KAPY_EW_FMA: per_element("fma_typed(" + elem(n.a) + ", " + elem(n.b) + ", " + elem(n.c) + ", " + std::to_string(n.dtype) + ")"); round_result(); break;
    case KAPY_EW_DIVF: {
      const std::string a = as_array(n.a), b = as_array(n.b);
      appendf(s, "    float %s[8]; div8(%s, %s, %s);\n", vn, a.c_str(), b.c_str(), vn);
      round_result();
      break;
    }
    default:  // the unary ops
      per_element(elem(n.a));
      appendf(s, "    unary8<NARROW>(%d, %d, %s);\n", n.op, n.dtype, vn);
      round_result();
    }
  }
  const std::string result = as_array(stored);
  appendf(s, "    store8_row<NARROW, RAGGED>(p.out, %d, (int64_t)row[u] * p.out_stride0, jv[u], p.width, %s);\n  }\n}\n", sig.out_dtype, result.c_str());
  return s;
}

// A program with reduces along the rows.  Row values are arrays [CH][8], per-row values single registers; operands that
// are one row for all rows ([1 x n]: a norm's gamma and beta) are read once per workgroup and parked, as they lie in
// memory, in each lane's own corner of the dynamic LDS (*lds_bytes; read at their use from L2 instead when that corner
// would exceed 48 KiB).  Two exchange areas serve the reduces in turn, counted across rows: a wave can write one again
// only after the barrier of the other, which every wave reaches after it has read the first.
std::string generate_rows(const kapy_ew_inst *prog, int n_inst, const int *result_dtype, const Signature &sig, const std::string &name, int *lds_bytes) {
  int stored = -1;
  std::vector<char> input_used;
  std::vector<Node> nodes = build_nodes(prog, n_inst, result_dtype, &stored, &input_used);
  const int CH = sig.chunks, TH = sig.threads;
  // parked row operands: 16 bytes per lane and chunk, twice that for f32
  int park_slot[kJitInputs], n_park = 0;
  for (int k = 0; k < sig.n_ins; ++k) {
    park_slot[k] = -1;
    if (input_used[k] && sig.in_kind[k] == kRow) {
      park_slot[k] = n_park;
      n_park += sig.in_dtype[k] == KAPY_F32 ? 2 : 1;
    }
  }
  const bool park = n_park > 0 && n_park * CH * TH * 16 <= 48 * 1024;
  *lds_bytes = park ? n_park * CH * TH * 16 : 0;

  std::string s = source_head();
  appendf(s, "extern \"C\" __global__ __launch_bounds__(%d) void %s(JitArgs p) {\n", TH, name.c_str());
  appendf(s, "  constexpr bool NARROW = %s, RAGGED = %s;\n  constexpr int CH = %d, THREADS = %d;\n", sig.narrow ? "true" : "false", sig.ragged ? "true" : "false", CH, TH);
  s += "  __shared__ float red[2][16];\n  extern __shared__ u32x4 parked[];\n  int phase = 0;\n  const int32_t vpr = p.vec_per_row;\n";
  emit_splats(s, nodes);
  for (int k = 0; k < sig.n_ins; ++k) {
    if (!input_used[k]) continue;
    const int kind = sig.in_kind[k], dt = sig.in_dtype[k];
    appendf(s, "  const StackIn g%d{p.in[%d], p.stride0[%d], %d, %d};\n", k, k, k, dt, kind == kRow ? 1 : 0);
    if (kind == kFull) appendf(s, "  Raw8 raw%d[CH];\n  row_fetch8<CH, THREADS, RAGGED>(g%d, blockIdx.x, vpr, p.width, true, raw%d);\n", k, k, k);
    else if (kind == kRow && park) {
      appendf(s, "  {\n    Raw8 t[CH];\n    row_fetch8<CH, THREADS, RAGGED>(g%d, 0, vpr, p.width, false, t);\n#pragma unroll\n    for (int c = 0; c < CH; ++c) {\n"
                 "      parked[(%d * CH + c) * THREADS + threadIdx.x] = t[c].lo;\n", k, park_slot[k]);
      if (dt == KAPY_F32) appendf(s, "      parked[(%d * CH + c) * THREADS + threadIdx.x] = t[c].hi;\n", park_slot[k] + 1);
      s += "    }\n  }\n";
    } else if (kind == kScalar) appendf(s, "  const float s%d = load_as_f32(p.in[%d], %d, 0);\n", k, k, dt);
  }
  s += "  for (int32_t i = blockIdx.x; i < p.rows; i += gridDim.x) {\n";
  // the row operands first: their registers are asked for again (the next row) right after
  std::string full_name[kJitInputs];
  for (int k = 0; k < sig.n_ins; ++k) {
    if (!input_used[k] || sig.in_kind[k] != kFull) continue;
    full_name[k] = "x" + std::to_string(k);
    appendf(s, "    float x%d[CH][8];\n#pragma unroll\n    for (int c = 0; c < CH; ++c) widen8(raw%d[c], %d, x%d[c]);\n", k, k, sig.in_dtype[k], k);
  }
  for (int k = 0; k < sig.n_ins; ++k)
    if (input_used[k] && sig.in_kind[k] == kFull)
      appendf(s, "    if (i + (int32_t)gridDim.x < p.rows) row_fetch8<CH, THREADS, RAGGED>(g%d, i + gridDim.x, vpr, p.width, true, raw%d);\n", k, k);

  auto elem = [&](int id) { return nodes[id].uniform ? nodes[id].name : nodes[id].name + "[c][e]"; };
  int n_filled = 0;
  // a per-row value as an array of 8 (div8 and the store take arrays)
  auto filled = [&](int id) {
    const std::string a = "f" + std::to_string(n_filled++);
    appendf(s, "    float %s[8]; fill8(%s, %s);\n", a.c_str(), a.c_str(), nodes[id].name.c_str());
    return a;
  };
  const char *kChunks = "#pragma unroll\n    for (int c = 0; c < CH; ++c)";
  for (size_t id = 0; id < nodes.size(); ++id) {
    Node &n = nodes[id];
    if (!n.used || n.op == KAPY_EW_SPLAT) continue;
    const bool reduce = n.op == KAPY_EW_REDUCE_SUM || n.op == KAPY_EW_REDUCE_MAX;
    n.uniform = reduce || ((n.a < 0 || nodes[n.a].uniform) && (n.b < 0 || nodes[n.b].uniform) && (n.c < 0 || nodes[n.c].uniform) && n.op != KAPY_EW_LD_GLOBAL);
    if (n.op == KAPY_EW_LD_GLOBAL) n.uniform = sig.in_kind[n.input] == kCol || sig.in_kind[n.input] == kScalar;
    if (n.op == KAPY_EW_ARANGE) n.uniform = n.ib == 0;  // along axis 0: the row's index, one value per row
    n.name = (n.uniform ? "u" : "v") + std::to_string(id);
    const char *vn = n.name.c_str();
    const std::string dt = std::to_string(n.dtype);
    auto round_result = [&]() {
      if (n.dtype == KAPY_F32) return;
      if (n.uniform) appendf(s, "    %s = round_to_dtype(%s, %d, true);\n", vn, vn, n.dtype);
      else appendf(s, "    %s round8<NARROW>(%s[c], %d, true);\n", kChunks, vn, n.dtype);
    };
    auto assign = [&](const std::string &expr) {
      if (n.uniform) appendf(s, "    float %s = %s;\n", vn, expr.c_str());
      else appendf(s, "    float %s[CH][8];\n    %s\n#pragma unroll\n      for (int e = 0; e < 8; ++e) %s[c][e] = %s;\n", vn, kChunks, vn, expr.c_str());
    };
    {
      const std::string ie = int_op_expr(n, nodes, n.a >= 0 ? elem(n.a) : "", n.b >= 0 ? elem(n.b) : "", n.c >= 0 ? elem(n.c) : "", "i",
                                         "((c * THREADS + (int32_t)threadIdx.x) * 8 + e)");
      if (!ie.empty()) {
        assign(ie);
        continue;
      }
    }
    switch (n.op) {
    case KAPY_EW_LD_GLOBAL: {
      const int k = n.input, kind = sig.in_kind[k];
      if (kind == kFull) n.name = full_name[k];
      else if (kind == kCol) appendf(s, "    const float %s = load_as_f32(p.in[%d], %d, (int64_t)i * p.stride0[%d]);\n", vn, k, sig.in_dtype[k], k);
      else if (kind == kScalar) n.name = "s" + std::to_string(k);
      else {
        appendf(s, "    float %s[CH][8];\n    %s {\n      Raw8 t;\n      t.lo = t.hi = u32x4{0, 0, 0, 0};\n", vn, kChunks);
        if (park) {
          appendf(s, "      t.lo = parked[(%d * CH + c) * THREADS + threadIdx.x];\n", park_slot[k]);
          if (sig.in_dtype[k] == KAPY_F32) appendf(s, "      t.hi = parked[(%d * CH + c) * THREADS + threadIdx.x];\n", park_slot[k] + 1);
        } else appendf(s, "      if (c * THREADS + (int32_t)threadIdx.x < vpr) t = fetch8_row<RAGGED>(g%d, 0, c * THREADS + (int32_t)threadIdx.x, p.width, false);\n", k);
        appendf(s, "      widen8(t, %d, %s[c]);\n    }\n", sig.in_dtype[k], vn);
      }
      break;
    }
    case KAPY_EW_REDUCE_SUM: case KAPY_EW_REDUCE_MAX:
      if (nodes[n.a].uniform) {  // the same value n times
        if (n.op == KAPY_EW_REDUCE_SUM) appendf(s, "    float %s = __fmul_rn(%s, (float)p.width);\n", vn, nodes[n.a].name.c_str());
        else appendf(s, "    float %s = %s;\n", vn, nodes[n.a].name.c_str());
      } else {
        appendf(s, "    float %s = row_reduce<CH, THREADS, %s, RAGGED>(%s, vpr, p.width, red[phase & 1]);\n    ++phase;\n", vn, n.op == KAPY_EW_REDUCE_SUM ? "true" : "false",
                nodes[n.a].name.c_str());
      }
      round_result();
      break;
    case KAPY_EW_FPTOFP: {
      const bool free_cast = n.dtype == KAPY_F32 || ((int)id == stored && n.dtype == sig.out_dtype && n.rmode != KAPY_RZ);
      if (free_cast) n.name = nodes[n.a].name;
      else if (n.uniform) appendf(s, "    float %s = round_to_dtype(%s, %d, %s);\n", vn, nodes[n.a].name.c_str(), n.dtype, n.rmode != KAPY_RZ ? "true" : "false");
      else {
        assign(elem(n.a));
        appendf(s, "    %s round8<NARROW>(%s[c], %d, %s);\n", kChunks, vn, n.dtype, n.rmode != KAPY_RZ ? "true" : "false");
      }
      break;
    }
    case KAPY_EW_ADDF: assign("__fadd_rn(" + elem(n.a) + ", " + elem(n.b) + ")"); round_result(); break;
    case KAPY_EW_SUBF: assign("__fsub_rn(" + elem(n.a) + ", " + elem(n.b) + ")"); round_result(); break;
    case KAPY_EW_MULF: assign("__fmul_rn(" + elem(n.a) + ", " + elem(n.b) + ")"); round_result(); break;
    case KAPY_EW_MAXIMUMF: assign("max_nan(" + elem(n.a) + ", " + elem(n.b) + ")"); round_result(); break;
    case KAPY_EW_MINIMUMF: assign("min_nan(" + elem(n.a) + ", " + elem(n.b) + ")"); round_result(); break;
    case KAPY_EW_MAXNUMF: assign("max_num(" + elem(n.a) + ", " + elem(n.b) + ")"); round_result(); break;
    case KAPY_EW_MINNUMF: assign("min_num(" + elem(n.a) + ", " + elem(n.b) + ")"); round_result(); break;
    case KAPY_EW_REMF: assign("rem_f(" + elem(n.a) + ", " + elem(n.b) + ")"); round_result(); break;
    case KAPY_EW_FMA: assign("fma_typed(" + elem(n.a) + ", " + elem(n.b) + ", " + elem(n.c) + ", " + dt + ")"); round_result(); break;
    case KAPY_EW_DIVF:
      if (n.uniform) assign("__fdiv_rn(" + elem(n.a) + ", " + elem(n.b) + ")");
      else {
        const std::string a = nodes[n.a].uniform ? filled(n.a) : nodes[n.a].name + "[c]";
        const std::string b = nodes[n.b].uniform ? filled(n.b) : nodes[n.b].name + "[c]";
        appendf(s, "    float %s[CH][8];\n    %s div8(%s, %s, %s[c]);\n", vn, kChunks, a.c_str(), b.c_str(), vn);
      }
      round_result();
      break;
    default:  // the unary ops
      if (n.uniform) assign("apply_unary(" + std::to_string(n.op) + ", " + elem(n.a) + ")");
      else {
        assign(elem(n.a));
        appendf(s, "    %s unary8<NARROW>(%d, %d, %s[c]);\n", kChunks, n.op, n.dtype, vn);
      }
      round_result();
    }
  }
  if (nodes[stored].uniform) {
    const std::string a = filled(stored);
    appendf(s, "    %s {\n      const int32_t jv = c * THREADS + (int32_t)threadIdx.x;\n      if (jv < vpr) store8_row<NARROW, RAGGED>(p.out, %d, (int64_t)i * p.out_stride0, jv, p.width, %s);\n    }\n",
            kChunks, sig.out_dtype, a.c_str());
  } else {
    appendf(s, "    %s {\n      const int32_t jv = c * THREADS + (int32_t)threadIdx.x;\n      if (jv < vpr) store8_row<NARROW, RAGGED>(p.out, %d, (int64_t)i * p.out_stride0, jv, p.width, %s[c]);\n    }\n",
            kChunks, sig.out_dtype, nodes[stored].name.c_str());
  }
  s += "  }\n}\n";
  return s;
}

// The kernel's name carries its skeleton and a hash of the table key, so that a profile tells the compiled programs apart.
std::string kernel_name(const Signature &sig, const std::string &key) {
  uint32_t h = 2166136261u;
  for (unsigned char ch : key) h = (h ^ ch) * 16777619u;
  char buf[48];
  snprintf(buf, sizeof buf, "kapy_ew_%s_%08x", sig.rowwise ? "rows" : "flat", h);
  return buf;
}

std::string generate(const kapy_ew_inst *prog, int n_inst, const int *result_dtype, const Signature &sig, const std::string &name, int *lds_bytes) {
  *lds_bytes = 0;
  return sig.rowwise ? generate_rows(prog, n_inst, result_dtype, sig, name, lds_bytes) : generate_flat(prog, n_inst, result_dtype, sig, name);
}

// ---- the runtime compiler, opened on first use --------------------------------------------------------------------
struct Rtc {
  void *handle = nullptr;
  decltype(&hiprtcCreateProgram) create = nullptr;
  decltype(&hiprtcCompileProgram) compile = nullptr;
  decltype(&hiprtcGetProgramLogSize) log_size = nullptr;
  decltype(&hiprtcGetProgramLog) log = nullptr;
  decltype(&hiprtcGetCodeSize) code_size = nullptr;
  decltype(&hiprtcGetCode) code = nullptr;
  decltype(&hiprtcDestroyProgram) destroy = nullptr;
  bool ok = false;
};
const Rtc &rtc() {
  static Rtc r = [] {
    Rtc t;
    for (const char *name : {"libhiprtc.so.7", "libhiprtc.so"}) {
      t.handle = dlopen(name, RTLD_NOW | RTLD_LOCAL);
      if (t.handle) break;
    }
    if (!t.handle) return t;
#define KAPY_RTC_SYM(field, symbol) t.field = (decltype(t.field))dlsym(t.handle, #symbol)
    KAPY_RTC_SYM(create, hiprtcCreateProgram);
    KAPY_RTC_SYM(compile, hiprtcCompileProgram);
    KAPY_RTC_SYM(log_size, hiprtcGetProgramLogSize);
    KAPY_RTC_SYM(log, hiprtcGetProgramLog);
    KAPY_RTC_SYM(code_size, hiprtcGetCodeSize);
    KAPY_RTC_SYM(code, hiprtcGetCode);
    KAPY_RTC_SYM(destroy, hiprtcDestroyProgram);
#undef KAPY_RTC_SYM
    t.ok = t.create && t.compile && t.log_size && t.log && t.code_size && t.code && t.destroy;
    return t;
  }();
  return r;
}

// KAPY_EW_CACHE_DIR names a directory in which compiled code objects are kept from one process to the next, under the hash of
// the generated text (which embeds the device helpers, so a new build of the library never finds a stale kernel) and of the
// compiler's options.  A file is written under a temporary name and renamed, so a reader never sees half of one.
std::string cache_path(const std::string &source, const char *const *opts, int n_opts) {
  const char *dir = getenv("KAPY_EW_CACHE_DIR");
  if (!dir || !dir[0]) return std::string();
  uint64_t h = 1469598103934665603ull;
  auto mix = [&](const char *data, size_t n) {
    for (size_t i = 0; i < n; ++i) h = (h ^ (unsigned char)data[i]) * 1099511628211ull;
  };
  mix(source.data(), source.size());
  for (int k = 0; k < n_opts; ++k) mix(opts[k], strlen(opts[k]) + 1);
  char name[64];
  snprintf(name, sizeof name, "/kapy_ew_%016llx_%zu.co", (unsigned long long)h, source.size());
  return std::string(dir) + name;
}
bool read_file(const std::string &path, std::vector<char> *data) {
  FILE *f = fopen(path.c_str(), "rb");
  if (!f) return false;
  bool ok = fseek(f, 0, SEEK_END) == 0;
  const long n = ok ? ftell(f) : -1;
  ok = ok && n > 0 && fseek(f, 0, SEEK_SET) == 0;
  if (ok) {
    data->resize((size_t)n);
    ok = fread(data->data(), 1, (size_t)n, f) == (size_t)n;
  }
  fclose(f);
  return ok;
}
void write_file_atomically(const std::string &path, const std::vector<char> &data) {
  const std::string tmp = path + ".tmp" + std::to_string((long)getpid());
  FILE *f = fopen(tmp.c_str(), "wb");
  if (!f) return;  // an unusable cache directory only costs the compile next time
  const bool ok = fwrite(data.data(), 1, data.size(), f) == data.size();
  if (fclose(f) != 0 || !ok || rename(tmp.c_str(), path.c_str()) != 0) remove(tmp.c_str());
}

// from_cache (out): the code object was read from KAPY_EW_CACHE_DIR rather than compiled; use_cache = false compiles in any
// case and overwrites what the cache holds (the caller found the cached object unusable).
int compile_source(const std::string &source, std::vector<char> *code, bool *from_cache, bool use_cache = true) {
  // Packed fp32 VALU forms stay off, as for every device compile of this library.  Contraction only inside one
  // expression: in the generated text every op of the program is a statement of its own and must keep its own rounding
  // (with everything in one basic block the default, cross-statement mode would fuse a mulf and the addf after it).
  const char *opts[] = {"--offload-arch=gfx950", "-O3", "-std=c++17", "-ffp-contract=on", "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"};
  constexpr int kOpts = (int)(sizeof opts / sizeof opts[0]);
  const std::string cached = cache_path(source, opts, kOpts);
  *from_cache = false;
  if (use_cache && !cached.empty() && read_file(cached, code)) {
    *from_cache = true;
    return KAPY_OK;
  }
  if (!use_cache && !cached.empty()) remove(cached.c_str());
  const Rtc &r = rtc();
  if (!r.ok) return fail(KAPY_ERR_UNSUPPORTED, "elementwise_specialize: the runtime compiler (libhiprtc) is not available");
  hiprtcProgram prog = nullptr;
  if (r.create(&prog, source.c_str(), "kapy_ew_specialised.hip", 0, nullptr, nullptr) != HIPRTC_SUCCESS)
    return fail(KAPY_ERR_HIP, "elementwise_specialize: hiprtcCreateProgram failed");
  const hiprtcResult rc = r.compile(prog, kOpts, opts);
  if (rc != HIPRTC_SUCCESS) {
    size_t n = 0;
    r.log_size(prog, &n);
    std::string log(n, '\0');
    if (n) r.log(prog, &log[0]);
    r.destroy(&prog);
    return fail(KAPY_ERR_HIP, "elementwise_specialize: compile failed (%d): %.400s", (int)rc, log.c_str());
  }
  size_t n = 0;
  r.code_size(prog, &n);
  code->resize(n);
  const hiprtcResult got = r.code(prog, code->data());
  r.destroy(&prog);
  if (got != HIPRTC_SUCCESS || n == 0) return fail(KAPY_ERR_HIP, "elementwise_specialize: no code object");
  if (!cached.empty()) write_file_atomically(cached, *code);
  return KAPY_OK;
}

struct Loaded {
  hipModule_t module = nullptr;
  hipFunction_t fn = nullptr;
  int lds_bytes = 0;   // row skeleton: the parked row operands
  int resident = 0;    // row skeleton: workgroups the device holds at once (each walks its share of the rows)
};
std::mutex g_mutex;
std::map<std::pair<int, std::string>, Loaded> g_table;  // (device, key) -> kernel
std::atomic<int> g_count{0};
std::atomic<int64_t> g_launches{0};

}  // namespace

int specialize_program(const kapy_ew_inst *prog, int n_inst, const int *result_dtype, const kapy_global *const *ins, int n_ins, const kapy_global *out) {
  Signature sig;
  View vi[kJitInputs], vo;
  if (!classify(prog, n_inst, result_dtype, ins, n_ins, out, &sig, vi, &vo))
    return fail(KAPY_ERR_UNSUPPORTED,
                "elementwise_specialize: needs one store, reduces only along rows of at most 32768 elements, zero padding, a result contiguous along "
                "one axis with lines that start aligned to 8 elements, and operands that are full (row- or column-major, 16-byte aligned), row, "
                "column or scalar views");
  int device = 0;
  KAPY_HIP_CHECK(hipGetDevice(&device));
  const std::string key = make_key(prog, n_inst, sig);
  {
    std::lock_guard<std::mutex> lock(g_mutex);
    if (g_table.count({device, key})) return KAPY_OK;
  }
  std::vector<char> code;
  Loaded k;
  const std::string name = kernel_name(sig, key);
  const std::string source = generate(prog, n_inst, result_dtype, sig, name, &k.lds_bytes);
  bool from_cache = false;
  int rc = compile_source(source, &code, &from_cache);
  if (rc) return rc;
  // A cached object is keyed by a hash only and may be damaged, foreign or built for another compiler: one that does not load, or
  // does not hold the kernel, is thrown away and the source compiled again.
  auto load = [&]() {
    hipError_t e = hipModuleLoadData(&k.module, code.data());
    if (e != hipSuccess) { k.module = nullptr; return e; }
    e = hipModuleGetFunction(&k.fn, k.module, name.c_str());
    if (e != hipSuccess) { (void)hipModuleUnload(k.module); k.module = nullptr; }
    return e;
  };
  hipError_t e = load();
  if (e != hipSuccess && from_cache) {
    (void)hipGetLastError();
    rc = compile_source(source, &code, &from_cache, false);
    if (rc) return rc;
    e = load();
  }
  if (e != hipSuccess) return fail(KAPY_ERR_HIP, "elementwise_specialize: the code object does not load: %s", hipGetErrorString(e));
  if (sig.rowwise) {
    int per_cu = 1;
    e = hipModuleOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, k.fn, sig.threads, (size_t)k.lds_bytes);
    if (e != hipSuccess) {
      (void)hipModuleUnload(k.module);
      return fail(KAPY_ERR_HIP, "elementwise_specialize: occupancy query failed: %s", hipGetErrorString(e));
    }
    k.resident = device_cus() * (per_cu > 0 ? per_cu : 1);
  }
  std::lock_guard<std::mutex> lock(g_mutex);
  if (!g_table.emplace(std::make_pair(device, key), k).second) (void)hipModuleUnload(k.module);  // another thread was first
  else g_count.fetch_add(1);
  return KAPY_OK;
}

int launch_specialized(const kapy_ew_inst *prog, int n_inst, const int *result_dtype, const kapy_global *const *ins, int n_ins, const kapy_global *out,
                       hipStream_t stream) {
  if (g_count.load(std::memory_order_acquire) == 0) return 0;
  Signature sig;
  View vi[kJitInputs], vo;
  if (!classify(prog, n_inst, result_dtype, ins, n_ins, out, &sig, vi, &vo)) return 0;
  int device = 0;
  KAPY_HIP_CHECK(hipGetDevice(&device));
  Loaded k;
  {
    std::lock_guard<std::mutex> lock(g_mutex);
    auto it = g_table.find({device, make_key(prog, n_inst, sig)});
    if (it == g_table.end()) return 0;
    k = it->second;
  }
  JitArgs args;
  memset(&args, 0, sizeof args);
  for (int i = 0; i < n_ins; ++i) {
    args.in[i] = vi[i].base;
    args.stride0[i] = sig.in_kind[i] == kColMajor ? vi[i].s1 : vi[i].s0;  // the pitch between rows, or between columns
  }
  args.out = (char *)vo.base;
  args.out_stride0 = vo.s0;
  args.rows = (int32_t)vo.e0;
  args.vec_per_row = (int32_t)((vo.e1 + 7) / 8);
  args.width = (int32_t)vo.e1;
  size_t size = sizeof args;
  void *extra[] = {HIP_LAUNCH_PARAM_BUFFER_POINTER, &args, HIP_LAUNCH_PARAM_BUFFER_SIZE, &size, HIP_LAUNCH_PARAM_END};
  if (sig.rowwise) {
    const unsigned grid = (unsigned)std::min<int64_t>(args.rows, k.resident);
    KAPY_HIP_CHECK(hipModuleLaunchKernel(k.fn, grid, 1, 1, (unsigned)sig.threads, 1, 1, (unsigned)k.lds_bytes, stream, nullptr, extra));
  } else if (sig.tiled) {
    const int64_t tiles = (int64_t)((args.rows + kTileRows - 1) / kTileRows) * ((args.vec_per_row + 7) / 8);
    KAPY_HIP_CHECK(hipModuleLaunchKernel(k.fn, (unsigned)tiles, 1, 1, 256, 1, 1, 0, stream, nullptr, extra));
  } else {
    const int64_t slots = (int64_t)args.rows * args.vec_per_row;
    KAPY_HIP_CHECK(hipModuleLaunchKernel(k.fn, (unsigned)((slots + 511) / 512), 1, 1, 256, 1, 1, 0, stream, nullptr, extra));
  }
  g_launches.fetch_add(1, std::memory_order_relaxed);
  return 1;
}

// How often an unmatched program of this signature has been called on this device, and whether compiling it has failed before:
// kapy_elementwise compiles a program that keeps coming back (from its second call by default) and never tries a failed one again.
namespace {
struct Seen {
  int calls = 0;
  bool failed = false;
};
std::map<std::pair<int, std::string>, Seen> g_seen;
}  // namespace
bool unmatched_call_wants_compile(const kapy_ew_inst *prog, int n_inst, const int *result_dtype, const kapy_global *const *ins, int n_ins, const kapy_global *out,
                                  int from_call) {
  Signature sig;
  View vi[kJitInputs], vo;
  if (!classify(prog, n_inst, result_dtype, ins, n_ins, out, &sig, vi, &vo)) return false;
  int device = 0;
  if (hipGetDevice(&device) != hipSuccess) return false;
  std::lock_guard<std::mutex> lock(g_mutex);
  Seen &seen = g_seen[{device, make_key(prog, n_inst, sig)}];
  if (seen.calls < from_call) ++seen.calls;
  return !seen.failed && seen.calls >= from_call;
}
void unmatched_compile_failed(const kapy_ew_inst *prog, int n_inst, const int *result_dtype, const kapy_global *const *ins, int n_ins, const kapy_global *out) {
  Signature sig;
  View vi[kJitInputs], vo;
  if (!classify(prog, n_inst, result_dtype, ins, n_ins, out, &sig, vi, &vo)) return;
  int device = 0;
  if (hipGetDevice(&device) != hipSuccess) return;
  std::lock_guard<std::mutex> lock(g_mutex);
  g_seen[{device, make_key(prog, n_inst, sig)}].failed = true;
}

void specialized_stats(int64_t *loaded, int64_t *launches) {
  if (loaded) *loaded = g_count.load();
  if (launches) *launches = g_launches.load();
}

int specialized_source(const kapy_ew_inst *prog, int n_inst, const int *result_dtype, const kapy_global *const *ins, int n_ins, const kapy_global *out,
                       char *source, int64_t capacity, int64_t *source_bytes, int64_t *code_bytes) {
  Signature sig;
  View vi[kJitInputs], vo;
  if (!classify(prog, n_inst, result_dtype, ins, n_ins, out, &sig, vi, &vo))
    return fail(KAPY_ERR_UNSUPPORTED, "elementwise_source: the program or its operands do not fit a specialised kernel");
  int lds_bytes = 0;
  const std::string text = generate(prog, n_inst, result_dtype, sig, kernel_name(sig, make_key(prog, n_inst, sig)), &lds_bytes);
  if (source && capacity > 0) {
    const size_t n = std::min<size_t>(text.size(), (size_t)capacity - 1);
    memcpy(source, text.data(), n);
    source[n] = '\0';
  }
  if (source_bytes) *source_bytes = (int64_t)text.size();
  if (code_bytes) {
    std::vector<char> code;
    bool from_cache = false;
    int rc = compile_source(text, &code, &from_cache);
    if (rc) return rc;
    *code_bytes = (int64_t)code.size();
  }
  return KAPY_OK;
}

}  // namespace kapy
