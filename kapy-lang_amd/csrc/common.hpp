// common.hpp — shared host-side helpers of the library: error reporting, descriptor arithmetic,
// HIP call checking.  No device code here.
#pragma once
#include <hip/hip_runtime.h>
#include <stdarg.h>
#include <stdint.h>
#include <stdio.h>

#include "../../include/kapy_hip.h"

// the case labels of every op with two register operands
#define KAPY_EW_BINARY_CASES                                                                                                          \
  case KAPY_EW_ADDF: case KAPY_EW_SUBF: case KAPY_EW_MULF: case KAPY_EW_DIVF: case KAPY_EW_MAXIMUMF: case KAPY_EW_MINIMUMF: case KAPY_EW_MAXNUMF:  \
  case KAPY_EW_MINNUMF: case KAPY_EW_REMF: case KAPY_EW_ADDI: case KAPY_EW_SUBI: case KAPY_EW_MULI: case KAPY_EW_DIVSI: case KAPY_EW_DIVUI:                 \
  case KAPY_EW_FLOORDIVSI: case KAPY_EW_CEILDIVSI: case KAPY_EW_CEILDIVUI: case KAPY_EW_REMSI: case KAPY_EW_REMUI: case KAPY_EW_ANDI: case KAPY_EW_ORI:      \
  case KAPY_EW_XORI: case KAPY_EW_SHLI: case KAPY_EW_SHRSI: case KAPY_EW_SHRUI: case KAPY_EW_MAXSI: case KAPY_EW_MAXUI: case KAPY_EW_MINSI:               \
  case KAPY_EW_MINUI: case KAPY_EW_CMPI: case KAPY_EW_CMPF

namespace kapy {

// Thread-local text of the last failure; the counterpart of the reference's emitOpError
// diagnostics (e.g. lib/Dialect/Kapy/IR/Kapy.cpp:272-287).
char *last_error_buffer();
int fail(int status, const char *fmt, ...) __attribute__((format(printf, 2, 3)));

#define KAPY_HIP_CHECK(expr)                                                                   \
  do {                                                                                         \
    hipError_t e_ = (expr);                                                                    \
    if (e_ != hipSuccess) return ::kapy::fail(KAPY_ERR_HIP, "%s: %s", #expr, hipGetErrorString(e_)); \
  } while (0)

inline int dtype_bytes(int32_t dtype) {
  switch (dtype) {
  case KAPY_F16: case KAPY_BF16: case KAPY_I16: return 2;
  case KAPY_F32: case KAPY_I32: return 4;
  case KAPY_F8E4M3: case KAPY_F8E5M2: case KAPY_I8: case KAPY_I1: return 1;
  }
  return 0;
}
inline bool is_float(int32_t d) { return d == KAPY_F16 || d == KAPY_BF16 || d == KAPY_F32 || d == KAPY_F8E4M3 || d == KAPY_F8E5M2; }
inline bool is_f8(int32_t d) { return d == KAPY_F8E4M3 || d == KAPY_F8E5M2; }
inline bool is_int(int32_t d) { return d == KAPY_I8 || d == KAPY_I16 || d == KAPY_I32 || d == KAPY_I1; }
inline const char *dtype_name(int32_t d) {
  static const char *names[] = {"f16", "bf16", "f32", "f8E4M3", "f8E5M2", "i8", "i16", "i32", "i1"};
  return d >= 0 && d < 9 ? names[d] : "?";
}

inline int64_t extent0(const kapy_global *g) { return int64_t(g->end0) - g->start0; }
inline int64_t extent1(const kapy_global *g) { return int64_t(g->end1) - g->start1; }
// Address (in elements, relative to g->ptr) of view element (0,0).
inline int64_t origin(const kapy_global *g) { return int64_t(g->start0) * g->stride0 + int64_t(g->start1) * g->stride1; }
inline const char *view_base(const kapy_global *g) { return (const char *)g->ptr + origin(g) * dtype_bytes(g->dtype); }

// Largest power-of-two byte count (<= 16) that divides the address of every row/column start of
// the view: what a vector access along the contiguous axis may assume.
inline int vector_bytes(const kapy_global *g, int contiguous_axis) {
  int b = dtype_bytes(g->dtype);
  uint64_t bits = (uint64_t)(uintptr_t)view_base(g);
  int64_t pitch = (contiguous_axis == 1 ? int64_t(g->stride0) : int64_t(g->stride1)) * b;
  int64_t rows = contiguous_axis == 1 ? extent0(g) : extent1(g);
  if (rows > 1) bits |= (uint64_t)(pitch < 0 ? -pitch : pitch);
  int v = 16;
  while (v > b && (bits & (uint64_t)(v - 1))) v >>= 1;
  return v;
}

// Compiles a verified program that contains a reduce for the row machine and launches it (elementwise_row.hip).
// result_dtype[k] is the element type of instruction k's result.
int run_row_program(const kapy_ew_inst *prog, int n_inst, const int *result_dtype, const kapy_global *const *ins, int n_ins, const kapy_global *out,
                    hipStream_t stream);

// Specialised kernels for verified elementwise programs (elementwise_jit.cpp).  specialize_program compiles and loads one
// for the current device; launch_specialized returns 1 when it launched one, 0 when none is loaded for this program and
// operand signature, a negative status on failure; specialized_source writes the generated text and, if asked, compiles it.
int specialize_program(const kapy_ew_inst *prog, int n_inst, const int *result_dtype, const kapy_global *const *ins, int n_ins, const kapy_global *out);
int launch_specialized(const kapy_ew_inst *prog, int n_inst, const int *result_dtype, const kapy_global *const *ins, int n_ins, const kapy_global *out,
                       hipStream_t stream);
void specialized_stats(int64_t *loaded, int64_t *launches);
// Counts a call of a program that no hand-written kernel matches; true when it should be compiled now (its from_call-th call of
// this signature on this device or a later one, and compiling it has not failed before).
bool unmatched_call_wants_compile(const kapy_ew_inst *prog, int n_inst, const int *result_dtype, const kapy_global *const *ins, int n_ins, const kapy_global *out,
                                  int from_call);
void unmatched_compile_failed(const kapy_ew_inst *prog, int n_inst, const int *result_dtype, const kapy_global *const *ins, int n_ins, const kapy_global *out);
int specialized_source(const kapy_ew_inst *prog, int n_inst, const int *result_dtype, const kapy_global *const *ins, int n_ins, const kapy_global *out,
                       char *source, int64_t capacity, int64_t *source_bytes, int64_t *code_bytes);

int check_global(const kapy_global *g, const char *what);
// The partial-line part (bytes: its size) of the array in the library's device image that serves reductions without a
// caller's workspace (wave_ops.hip), or nullptr; calls that use it must not overlap in time on one GPU.
float *reduce_scratch_lines(size_t *bytes, uint32_t **counters = nullptr);   // counters: the array's arrival counters (4096 words, zero between calls)
// softmax of every column of a 16-bit row-major matrix in two launches (elementwise_col.hip): 1 = launched, 0 = the shapes
// are not the kernels', a negative status on failure.
// kapy_copy / kapy_copy_batched (copy.hip); grid may be null.
int copy_impl(const kapy_global *src, const kapy_global *dst, const kapy_copy_cfg *cfg, const kapy_grid2 *grid, void *stream);
int run_matmul_f16acc(const kapy_global *lhs, const kapy_global *rhs, const kapy_global *acc, const kapy_global *result, int k_step, hipStream_t s);
int run_column_softmax(const kapy_global *x, const kapy_global *out, hipStream_t stream);
// Many copies / matrix products of one shape as one launch over a table of base addresses in device memory (batched.hip):
// n rows of (source, target) or (lhs, rhs, accumulator input or 0, result), the addresses of element (0, 0) of each view.
struct CopyTableShape {
  int32_t d0, d1, elem_bytes;
  int64_t ss0, ss1, ds0, ds1;  // element strides of source and target
};
struct MatmulTableShape {
  int32_t M, N, K, ab_dtype, acc_dtype, d_dtype;
  int64_t a_sm, b_sk, acc_sm, acc_sn, d_sm, d_sn;  // lhs rows and rhs k-rows contiguous
};
int copy_table_launch(const uint64_t *device_table, int32_t n, const CopyTableShape &shape, bool vec16, hipStream_t s);
int matmul_table_launch(const uint64_t *device_table, int32_t n, const MatmulTableShape &shape, hipStream_t s);
int ensure_device();
int device_cus();

}  // namespace kapy
