// kapy_hip.hpp — the host side of the hot path in C++, above the C ABI of kapy_hip.h.
//
// kapy::OpBuilder mirrors the part of the reference's KapyOpBuilder that the hot path uses
// (python/src/ir.cc:730-1181: create_mk_global, create_sv_global, create_ld_global, create_st_global,
// create_constant_* scalars, create_splat, create_broadcast, create_transpose, create_arange, create_fptofp / extf / truncf / bitcast / sitofp /
// fptosi / intcast, the float and integer arith builders, the create_cmpi_* / create_cmpf_* families, create_select,
// the math builders, create_elementwise_extern_lib, create_reduce, create_matmul: 97 of its 112 create_* names - the rest build
// modules, blocks, control flow and the ids of a program, which a recorded dataflow graph has none of), with the same names and
// argument meaning.  Where the reference
// appends an op to a function that is compiled later, this builder records the op in a dataflow graph;
// create_st_global - the op with the side effect - lowers the graph under its source to ONE library call:
//   a load (optionally transposed) stored back            -> kapy_copy
//   a matmul, optionally followed on its result by a scale, a broadcast bias row, an activation and the cast
//                                                          -> kapy_matmul / kapy_matmul_fused
//   anything else made of elementwise ops and row reduces  -> kapy_elementwise (one fused kernel)
// Failures throw kapy::Error carrying the kapy_status and the verifier's text (the reference's builders throw
// std::invalid_argument / emit op errors).  Header only; link against libkapy_hip.so.
#ifndef KAPY_HIP_HPP
#define KAPY_HIP_HPP

#include <stdexcept>
#include <utility>
#include <string>
#include <vector>

#include "kapy_hip.h"

namespace kapy {

struct Error : std::runtime_error {
  int status;
  Error(int status_, const std::string &what) : std::runtime_error(what), status(status_) {}
};

// An SSA value of the builder: a global-memory tensor (descriptor) or a register tensor (graph node).
class Value {
 public:
  Value() = default;
  bool valid() const { return id_ >= 0; }

 private:
  friend class OpBuilder;
  explicit Value(int id) : id_(id) {}
  int id_ = -1;
};

class OpBuilder {
 public:
  // stream: the hipStream_t every lowered call is issued on (nullptr = the default stream)
  explicit OpBuilder(void *stream = nullptr) : stream_(stream) {}

  // ---- memory descriptors (python/src/ir.cc:1013-1034) ------------------------------------------------
  Value create_mk_global(void *global_address, int32_t dynamic_offset, int32_t size0, int32_t size1, int32_t stride0, int32_t stride1,
                         kapy_dtype element_type, int32_t alignment = 16) {
    Node n;
    n.kind = Node::kGlobal;
    check(kapy_mk_global(&n.global, global_address, dynamic_offset, size0, size1, stride0, stride1, element_type, alignment));
    n.dtype = element_type;
    return push(n);
  }
  Value create_sv_global(Value source, int32_t start0, int32_t end0, int32_t start1, int32_t end1) {
    Node n;
    n.kind = Node::kGlobal;
    check(kapy_sv_global(&n.global, &global_of(source, "sv_global"), start0, end0, start1, end1));
    n.dtype = node(source).dtype;
    return push(n);
  }

  // ---- shared-memory descriptors (ir.cc:1050-1070): plain data, as the lowering's structs are ----------------------
  // byte_offset: where the planner (kapy_smem_plan) put the buffer; (bank_param, line_param): its swizzling, (0, 0) = none
  kapy_shared create_mk_shared(const std::vector<int64_t> &shape, kapy_dtype element_type, bool row_major, int64_t byte_offset = 0,
                               int32_t bank_param = 0, int32_t line_param = 0) {
    if (shape.size() != 2) throw Error(KAPY_ERR_VERIFY, "mk_shared: tensors have rank 2");
    kapy_shared t;
    check(kapy_mk_shared(&t, byte_offset, (int32_t)shape[0], (int32_t)shape[1], element_type, row_major ? 1 : 0, bank_param, line_param));
    return t;
  }
  kapy_shared create_sv_shared(const kapy_shared &source, int32_t start0, int32_t end0, int32_t start1, int32_t end1) {
    kapy_shared t;
    check(kapy_sv_shared(&t, &source, start0, end0, start1, end1));
    return t;
  }

  // ---- loads and stores (ir.cc:1035-1049) ---------------------------------------------------------------
  // (argument order as in the reference: source, paddingOption, cacheModifier, evictPriority, isVolatile)
  Value create_ld_global(Value source, kapy_padding_option padding_option = KAPY_PAD_ZERO, kapy_cache_modifier cache_modifier = KAPY_CACHE_NONE,
                         kapy_evict_priority evict_priority = KAPY_EVICT_NORMAL, bool is_volatile = false) {
    Node n;
    n.kind = Node::kLoad;
    n.global = global_of(source, "ld_global");
    n.dtype = node(source).dtype;
    n.padding = padding_option;
    n.cache = cache_modifier;
    n.evict = evict_priority;
    n.is_volatile = is_volatile;
    return push(n);
  }
  // Lowers everything `source` depends on and stores it: the one call that launches work.
  // (the hints of a store apply to the move it launches; a load's hints stand in where the store gives none)
  void create_st_global(Value source, Value target, kapy_cache_modifier cache_modifier = KAPY_CACHE_NONE,
                        kapy_evict_priority evict_priority = KAPY_EVICT_NORMAL, bool is_volatile = false) {
    const kapy_global &out = global_of(target, "st_global");
    const Node &s = node(source);
    if (s.kind == Node::kGlobal) throw Error(KAPY_ERR_VERIFY, "st_global: source must be a register tensor");
    if (s.kind == Node::kLoad) {  // a layout move: bits travel untouched
      kapy_copy_cfg cfg = {s.transposed ? 1 : 0, s.padding, cache_modifier != KAPY_CACHE_NONE ? cache_modifier : s.cache,
                           evict_priority != KAPY_EVICT_NORMAL ? evict_priority : s.evict, (is_volatile || s.is_volatile) ? 1 : 0, 0};
      check(kapy_copy(&s.global, &out, &cfg, stream_));
      return;
    }
    if (depends_on_matmul(source.id_)) {
      lower_matmul(source.id_, out);
      return;
    }
    std::vector<kapy_ew_inst> prog;
    std::vector<const kapy_global *> ins;
    emit_program(source.id_, &prog, &ins);
    check(kapy_elementwise(prog.data(), (int32_t)prog.size(), ins.data(), (int32_t)ins.size(), &out, stream_));
  }
  // The elementwise program create_st_global(source, ...) would run (for inspection and for kapy_elementwise_specialize).
  std::vector<kapy_ew_inst> program_of(Value source, std::vector<kapy_global> *inputs = nullptr) {
    std::vector<kapy_ew_inst> prog;
    std::vector<const kapy_global *> ins;
    emit_program(source.id_, &prog, &ins);
    if (inputs) {
      inputs->clear();
      for (const kapy_global *g : ins) inputs->push_back(*g);
    }
    return prog;
  }

  // ---- shape ops (ir.cc:1071-1090) ------------------------------------------------------------------------
  // the reference splats a scalar Value to a tensor shape; a program's shape is its result's, so the scalar and its type suffice
  Value create_splat(float source, kapy_dtype element_type) {
    Node n;
    n.kind = Node::kOp;
    n.op = KAPY_EW_SPLAT;
    n.dtype = element_type;
    n.imm = source;
    return push(n);
  }
  // an integer splat (the reference splats a create_constant_int* scalar): the value wraps to the type's width
  Value create_splat(int32_t source, kapy_dtype element_type) {
    if (element_type <= KAPY_F8E5M2) return create_splat((float)source, element_type);
    Node n;
    n.kind = Node::kOp;
    n.op = KAPY_EW_SPLAT;
    n.dtype = element_type;
    n.ival = source;
    return push(n);
  }
  // ---- scalar constants (ir.cc:480-560: create_constant_int1 ... create_constant_float64, create_constant_zero,
  // create_constant_all_ones).  A scalar here exists to be splat: create_splat(scalar) makes the tensor of the scalar's type
  // (f64 and i64 scalars have no tensor type in this library and can only be splat to a named narrower type).
  Value create_constant_int1(bool v) { return scalar_int(v ? 1 : 0, KAPY_I1); }
  Value create_constant_int8(int8_t v) { return scalar_int(v, KAPY_I8); }
  Value create_constant_int16(int16_t v) { return scalar_int(v, KAPY_I16); }
  Value create_constant_int32(int32_t v) { return scalar_int(v, KAPY_I32); }
  Value create_constant_int64(int64_t v) { return scalar_int(v, -64); }
  Value create_constant_float8e4m3(float v) { return scalar_float(v, KAPY_F8E4M3); }
  Value create_constant_float8e5m2(float v) { return scalar_float(v, KAPY_F8E5M2); }
  Value create_constant_float16(float v) { return scalar_float(v, KAPY_F16); }
  Value create_constant_bfloat16(float v) { return scalar_float(v, KAPY_BF16); }
  Value create_constant_float32(float v) { return scalar_float(v, KAPY_F32); }
  Value create_constant_float64(double v) { return scalar_float(v, -64); }
  Value create_constant_zero(kapy_dtype type) { return type <= KAPY_F8E5M2 ? scalar_float(0.0, type) : scalar_int(0, type); }
  Value create_constant_all_ones(kapy_dtype type) {
    if (type <= KAPY_F8E5M2) throw Error(KAPY_ERR_UNSUPPORTED, "constant_all_ones: integer types only");
    return scalar_int(-1, type);
  }
  // the reference's form of splat: a scalar Value in, a tensor of its type out (element_type: a narrower type for an f64 / i64 scalar)
  Value create_splat(Value scalar, int element_type = -1) {
    const Node &sc = node(scalar);
    if (sc.kind != Node::kScalar) throw Error(KAPY_ERR_VERIFY, "splat: operand must be a scalar constant");
    const int dt = element_type >= 0 ? element_type : sc.dtype;
    if (dt < 0) throw Error(KAPY_ERR_UNSUPPORTED, "splat: a 64-bit scalar needs the tensor's element type");
    const bool to_float = dt <= KAPY_F8E5M2;
    if (to_float != sc.scalar_is_float) throw Error(KAPY_ERR_VERIFY, "splat: scalar and tensor must both be float or both integer");
    if (to_float) return create_splat((float)sc.scalar_f, (kapy_dtype)dt);
    return create_splat((int32_t)sc.scalar_i, (kapy_dtype)dt);
  }

  // kapy.arange (ir.cc:730-743): i32 values start, start + 1, ... along `axis`, shape [end - start, 1] or [1, end - start];
  // inside a program it is the element's index along that axis plus start, broadcast over the other axis
  Value create_arange(unsigned axis, int32_t start, int32_t end) {
    if (axis > 1) throw Error(KAPY_ERR_INVALID, "program axis must be 0, 1");
    if (end <= start) throw Error(KAPY_ERR_VERIFY, "arange: end must be greater than start");
    Node n;
    n.kind = Node::kOp;
    n.op = KAPY_EW_ARANGE;
    n.dtype = KAPY_I32;
    n.ival = start;
    n.axis = (int)axis;
    return push(n);
  }
  // kapy.broadcast: extents of 1 stretch to the result's.  A load of a [1 x n] or [m x 1] view already is one; the
  // requested shape is checked when the program is verified against its result.
  Value create_broadcast(Value source, const std::vector<int64_t> & /*shape*/) {
    if (node(source).kind == Node::kGlobal) throw Error(KAPY_ERR_VERIFY, "broadcast: source must be a tensor");
    return source;
  }
  // kapy.transpose of a loaded tensor is the load with swapped strides; of a computed tensor: store it through a
  // descriptor with swapped strides instead
  Value create_transpose(Value source) {
    Node n = node(source);
    if (n.kind != Node::kLoad) throw Error(KAPY_ERR_UNSUPPORTED, "transpose: only of a loaded tensor (store a computed one through swapped strides)");
    n.transposed = !n.transposed;
    return push(n);
  }

  // ---- casts (ir.cc:744-790) ---------------------------------------------------------------------------
  Value create_fptofp(Value source, kapy_dtype element_type, kapy_rounding_mode rounding_mode = KAPY_RN) {
    return unary(KAPY_EW_FPTOFP, source, element_type, rounding_mode);
  }
  Value create_extf(Value source, kapy_dtype element_type) { return create_fptofp(source, element_type, KAPY_RN); }
  Value create_truncf(Value source, kapy_dtype element_type) { return create_fptofp(source, element_type, KAPY_RN); }

  // (ir.cc:755-790) arith.bitcast, sitofp, fptosi; create_intcast picks bitcast / trunci / extsi / extui from the widths
  Value create_bitcast(Value source, kapy_dtype element_type) { return unary(KAPY_EW_BITCAST, source, element_type); }
  Value create_sitofp(Value source, kapy_dtype element_type) { return unary(KAPY_EW_SITOFP, source, element_type); }
  Value create_fptosi(Value source, kapy_dtype element_type) { return unary(KAPY_EW_FPTOSI, source, element_type); }
  Value create_intcast(Value source, kapy_dtype element_type, bool is_signed) {
    const int from = bits_of(node(source).dtype), to = bits_of(element_type);
    if (from == to) return create_bitcast(source, element_type);
    if (from > to) return unary(KAPY_EW_TRUNCI, source, element_type);
    return unary(is_signed ? KAPY_EW_EXTSI : KAPY_EW_EXTUI, source, element_type);
  }

  // ---- arith / math (ir.cc:791-1157) ---------------------------------------------------------------------
  Value create_muli(Value lhs, Value rhs) { return binary(KAPY_EW_MULI, lhs, rhs); }
  Value create_divsi(Value lhs, Value rhs) { return binary(KAPY_EW_DIVSI, lhs, rhs); }
  Value create_divui(Value lhs, Value rhs) { return binary(KAPY_EW_DIVUI, lhs, rhs); }
  Value create_remsi(Value lhs, Value rhs) { return binary(KAPY_EW_REMSI, lhs, rhs); }
  Value create_remui(Value lhs, Value rhs) { return binary(KAPY_EW_REMUI, lhs, rhs); }
  Value create_addi(Value lhs, Value rhs) { return binary(KAPY_EW_ADDI, lhs, rhs); }
  Value create_subi(Value lhs, Value rhs) { return binary(KAPY_EW_SUBI, lhs, rhs); }
  Value create_shli(Value lhs, Value rhs) { return binary(KAPY_EW_SHLI, lhs, rhs); }
  Value create_shrui(Value lhs, Value rhs) { return binary(KAPY_EW_SHRUI, lhs, rhs); }
  Value create_shrsi(Value lhs, Value rhs) { return binary(KAPY_EW_SHRSI, lhs, rhs); }
  Value create_minsi(Value lhs, Value rhs) { return binary(KAPY_EW_MINSI, lhs, rhs); }
  Value create_minui(Value lhs, Value rhs) { return binary(KAPY_EW_MINUI, lhs, rhs); }
  Value create_maxsi(Value lhs, Value rhs) { return binary(KAPY_EW_MAXSI, lhs, rhs); }
  Value create_maxui(Value lhs, Value rhs) { return binary(KAPY_EW_MAXUI, lhs, rhs); }
  Value create_andi(Value lhs, Value rhs) { return binary(KAPY_EW_ANDI, lhs, rhs); }
  Value create_ori(Value lhs, Value rhs) { return binary(KAPY_EW_ORI, lhs, rhs); }
  Value create_xori(Value lhs, Value rhs) { return binary(KAPY_EW_XORI, lhs, rhs); }
  Value create_absi(Value source) { return unary(KAPY_EW_ABSI, source); }
  // arith.cmpi / arith.cmpf (ir.cc:891-1000): an i1 tensor
  Value create_cmpi_sle(Value lhs, Value rhs) { return compare(KAPY_EW_CMPI, KAPY_CMPI_SLE, lhs, rhs); }
  Value create_cmpi_slt(Value lhs, Value rhs) { return compare(KAPY_EW_CMPI, KAPY_CMPI_SLT, lhs, rhs); }
  Value create_cmpi_sge(Value lhs, Value rhs) { return compare(KAPY_EW_CMPI, KAPY_CMPI_SGE, lhs, rhs); }
  Value create_cmpi_sgt(Value lhs, Value rhs) { return compare(KAPY_EW_CMPI, KAPY_CMPI_SGT, lhs, rhs); }
  Value create_cmpi_ule(Value lhs, Value rhs) { return compare(KAPY_EW_CMPI, KAPY_CMPI_ULE, lhs, rhs); }
  Value create_cmpi_ult(Value lhs, Value rhs) { return compare(KAPY_EW_CMPI, KAPY_CMPI_ULT, lhs, rhs); }
  Value create_cmpi_uge(Value lhs, Value rhs) { return compare(KAPY_EW_CMPI, KAPY_CMPI_UGE, lhs, rhs); }
  Value create_cmpi_ugt(Value lhs, Value rhs) { return compare(KAPY_EW_CMPI, KAPY_CMPI_UGT, lhs, rhs); }
  Value create_cmpi_eq(Value lhs, Value rhs) { return compare(KAPY_EW_CMPI, KAPY_CMPI_EQ, lhs, rhs); }
  Value create_cmpi_ne(Value lhs, Value rhs) { return compare(KAPY_EW_CMPI, KAPY_CMPI_NE, lhs, rhs); }
  Value create_cmpf_olt(Value lhs, Value rhs) { return compare(KAPY_EW_CMPF, KAPY_CMPF_OLT, lhs, rhs); }
  Value create_cmpf_ogt(Value lhs, Value rhs) { return compare(KAPY_EW_CMPF, KAPY_CMPF_OGT, lhs, rhs); }
  Value create_cmpf_ole(Value lhs, Value rhs) { return compare(KAPY_EW_CMPF, KAPY_CMPF_OLE, lhs, rhs); }
  Value create_cmpf_oge(Value lhs, Value rhs) { return compare(KAPY_EW_CMPF, KAPY_CMPF_OGE, lhs, rhs); }
  Value create_cmpf_oeq(Value lhs, Value rhs) { return compare(KAPY_EW_CMPF, KAPY_CMPF_OEQ, lhs, rhs); }
  Value create_cmpf_one(Value lhs, Value rhs) { return compare(KAPY_EW_CMPF, KAPY_CMPF_ONE, lhs, rhs); }
  Value create_cmpf_ult(Value lhs, Value rhs) { return compare(KAPY_EW_CMPF, KAPY_CMPF_ULT, lhs, rhs); }
  Value create_cmpf_ugt(Value lhs, Value rhs) { return compare(KAPY_EW_CMPF, KAPY_CMPF_UGT, lhs, rhs); }
  Value create_cmpf_ule(Value lhs, Value rhs) { return compare(KAPY_EW_CMPF, KAPY_CMPF_ULE, lhs, rhs); }
  Value create_cmpf_uge(Value lhs, Value rhs) { return compare(KAPY_EW_CMPF, KAPY_CMPF_UGE, lhs, rhs); }
  Value create_cmpf_ueq(Value lhs, Value rhs) { return compare(KAPY_EW_CMPF, KAPY_CMPF_UEQ, lhs, rhs); }
  Value create_cmpf_une(Value lhs, Value rhs) { return compare(KAPY_EW_CMPF, KAPY_CMPF_UNE, lhs, rhs); }
  // arith.select on tensors (ir.cc:1162-1167; SelectOpToLLVM.cpp:21-98): condition an i1 tensor
  Value create_select(Value condition, Value true_value, Value false_value) {
    Node n;
    n.kind = Node::kOp;
    n.op = KAPY_EW_SELECT;
    n.a = tensor(condition, "select");
    n.b = tensor(true_value, "select");
    n.c = tensor(false_value, "select");
    n.dtype = node(true_value).dtype;
    return push(n);
  }
  Value create_addf(Value lhs, Value rhs) { return binary(KAPY_EW_ADDF, lhs, rhs); }
  Value create_subf(Value lhs, Value rhs) { return binary(KAPY_EW_SUBF, lhs, rhs); }
  Value create_mulf(Value lhs, Value rhs) { return binary(KAPY_EW_MULF, lhs, rhs); }
  Value create_divf(Value lhs, Value rhs) { return binary(KAPY_EW_DIVF, lhs, rhs); }
  Value create_maximumf(Value lhs, Value rhs) { return binary(KAPY_EW_MAXIMUMF, lhs, rhs); }
  Value create_minimumf(Value lhs, Value rhs) { return binary(KAPY_EW_MINIMUMF, lhs, rhs); }
  Value create_maxnumf(Value lhs, Value rhs) { return binary(KAPY_EW_MAXNUMF, lhs, rhs); }
  Value create_minnumf(Value lhs, Value rhs) { return binary(KAPY_EW_MINNUMF, lhs, rhs); }
  Value create_remf(Value lhs, Value rhs) { return binary(KAPY_EW_REMF, lhs, rhs); }
  // kapy.clampf(source, low, high, propagateNan) (ir.cc:886-890; ClampFOpConversion, ElementwiseOpToLLVM.cpp:699-728):
  // min(max(source, low), high) with maximumf / minimumf when NaNs propagate, maxnumf / minnumf when they do not
  Value create_clampf(Value source, Value low, Value high, bool propagate_nan = true) {
    if (!propagate_nan) return create_minnumf(create_maxnumf(source, low), high);
    return create_minimumf(create_maximumf(source, low), high);
  }
  Value create_fma(Value a, Value b, Value c) {
    Node n;
    n.kind = Node::kOp;
    n.op = KAPY_EW_FMA;
    n.a = tensor(a, "fma");
    n.b = tensor(b, "fma");
    n.c = tensor(c, "fma");
    n.dtype = node(a).dtype;
    return push(n);
  }
  Value create_negf(Value source) { return unary(KAPY_EW_NEGF, source); }
  Value create_absf(Value source) { return unary(KAPY_EW_ABSF, source); }
  Value create_exp(Value source) { return unary(KAPY_EW_EXP, source); }
  Value create_exp2(Value source) { return unary(KAPY_EW_EXP2, source); }
  Value create_log(Value source) { return unary(KAPY_EW_LOG, source); }
  Value create_log2(Value source) { return unary(KAPY_EW_LOG2, source); }
  Value create_sqrt(Value source) { return unary(KAPY_EW_SQRT, source); }
  Value create_rsqrt(Value source) { return unary(KAPY_EW_RSQRT, source); }
  Value create_erf(Value source) { return unary(KAPY_EW_ERF, source); }
  Value create_floor(Value source) { return unary(KAPY_EW_FLOOR, source); }
  Value create_ceil(Value source) { return unary(KAPY_EW_CEIL, source); }
  Value create_sin(Value source) { return unary(KAPY_EW_SIN, source); }
  Value create_cos(Value source) { return unary(KAPY_EW_COS, source); }
  // create_elementwise_extern_lib (ir.cc:1168-1174): the library functions the path uses, by name
  Value create_elementwise_extern_lib(const std::string &name, Value source) {
    // (also under the names of the device library the reference links, symName of ir.cc:1168-1174)
    static const struct { const char *name; int op; } known[] = {
        {"tanh", KAPY_EW_TANH}, {"__nv_tanhf", KAPY_EW_TANH}, {"gelu", KAPY_EW_GELU_TANH}, {"gelu_tanh", KAPY_EW_GELU_TANH},
        {"__nv_expf", KAPY_EW_EXP}, {"__nv_exp2f", KAPY_EW_EXP2}, {"__nv_logf", KAPY_EW_LOG}, {"__nv_log2f", KAPY_EW_LOG2}, {"__nv_sqrtf", KAPY_EW_SQRT},
        {"__nv_rsqrtf", KAPY_EW_RSQRT}, {"__nv_erff", KAPY_EW_ERF}, {"__nv_sinf", KAPY_EW_SIN}, {"__nv_cosf", KAPY_EW_COS}, {"__nv_floorf", KAPY_EW_FLOOR},
        {"__nv_ceilf", KAPY_EW_CEIL}, {"__nv_fabsf", KAPY_EW_ABSF}};
    for (const auto &k : known)
      if (name == k.name) return unary(k.op, source);
    throw Error(KAPY_ERR_UNSUPPORTED, "elementwise_extern_lib: unknown function " + name);
  }

  // ---- reduce and matmul (ir.cc:1101-1105, 1175-1181) ---------------------------------------------------------
  // kapy.reduce with an addf (is_max = false) or maximumf combiner along `axis`, its result broadcast back over the axis
  Value create_reduce(Value source, int32_t axis, bool is_max = false) {
    Node n;
    n.kind = Node::kOp;
    n.op = is_max ? KAPY_EW_REDUCE_MAX : KAPY_EW_REDUCE_SUM;
    n.a = tensor(source, "reduce");
    n.axis = axis;
    n.dtype = node(source).dtype;
    return push(n);
  }
  // acc may be an invalid Value (no accumulator input); the result has the accumulator type f32
  Value create_matmul(Value lhs, Value rhs, Value acc = Value(), kapy_matmul_impl_way impl_way = KAPY_MATMUL_AUTO) {
    if (node(lhs).kind != Node::kLoad || node(rhs).kind != Node::kLoad || (acc.valid() && node(acc).kind != Node::kLoad))
      throw Error(KAPY_ERR_UNSUPPORTED, "matmul: operands must be loaded tensors");
    Node n;
    n.kind = Node::kMatmul;
    n.a = lhs.id_;
    n.b = rhs.id_;
    n.c = acc.id_;
    n.impl_way = impl_way;
    n.dtype = KAPY_F32;
    return push(n);
  }

 private:
  struct Node {
    enum Kind { kGlobal, kLoad, kOp, kMatmul, kScalar } kind = kOp;
    kapy_global global{};
    int op = -1, a = -1, b = -1, c = -1, dtype = KAPY_F32, rmode = KAPY_RN, axis = 1;
    int padding = KAPY_PAD_ZERO, cache = KAPY_CACHE_NONE, evict = KAPY_EVICT_NORMAL, impl_way = KAPY_MATMUL_AUTO;
    bool transposed = false, is_volatile = false;
    float imm = 0.f;
    int ival = 0, pred = 0;  // an integer splat's value or arange's start; a compare's predicate
    bool scalar_is_float = false;  // kScalar: a constant that create_splat turns into a tensor
    double scalar_f = 0.0;
    int64_t scalar_i = 0;
  };
  std::vector<Node> nodes_;
  void *stream_;

  static void check(int rc) {
    if (rc < 0) throw Error(rc, kapy_last_error());
  }
  Value push(const Node &n) {
    nodes_.push_back(n);
    return Value((int)nodes_.size() - 1);
  }
  const Node &node(Value v) const {
    if (v.id_ < 0 || v.id_ >= (int)nodes_.size()) throw Error(KAPY_ERR_INVALID, "use of an undefined value");
    return nodes_[v.id_];
  }
  const kapy_global &global_of(Value v, const char *what) const {
    if (node(v).kind != Node::kGlobal) throw Error(KAPY_ERR_VERIFY, std::string(what) + ": operand must be a global-memory tensor");
    return node(v).global;
  }
  Value scalar_float(double v, int dtype) {
    Node n;
    n.kind = Node::kScalar;
    n.dtype = dtype;
    n.scalar_is_float = true;
    n.scalar_f = v;
    return push(n);
  }
  Value scalar_int(int64_t v, int dtype) {
    Node n;
    n.kind = Node::kScalar;
    n.dtype = dtype;
    n.scalar_i = v;
    return push(n);
  }
  int tensor(Value v, const char *what) const {
    if (node(v).kind == Node::kScalar) throw Error(KAPY_ERR_VERIFY, std::string(what) + ": operand must be a tensor (splat the scalar first)");
    if (node(v).kind == Node::kGlobal) throw Error(KAPY_ERR_VERIFY, std::string(what) + ": operand must be a register tensor (ld_global it first)");
    return v.id_;
  }
  Value unary(int op, Value source, int dtype = -1, int rmode = KAPY_RN) {
    Node n;
    n.kind = Node::kOp;
    n.op = op;
    n.a = tensor(source, "elementwise");
    n.dtype = dtype >= 0 ? dtype : node(source).dtype;
    n.rmode = rmode;
    return push(n);
  }
  static int bits_of(int dtype) {
    switch (dtype) {
    case KAPY_I1: return 1;
    case KAPY_F8E4M3: case KAPY_F8E5M2: case KAPY_I8: return 8;
    case KAPY_F16: case KAPY_BF16: case KAPY_I16: return 16;
    default: return 32;
    }
  }
  Value compare(int op, int predicate, Value lhs, Value rhs) {
    Node n;
    n.kind = Node::kOp;
    n.op = op;
    n.a = tensor(lhs, "compare");
    n.b = tensor(rhs, "compare");
    n.pred = predicate;
    n.dtype = KAPY_I1;
    return push(n);
  }
  Value binary(int op, Value lhs, Value rhs) {
    Node n;
    n.kind = Node::kOp;
    n.op = op;
    n.a = tensor(lhs, "elementwise");
    n.b = tensor(rhs, "elementwise");
    n.dtype = node(lhs).dtype;
    return push(n);
  }
  // the view a load reads: strides and extents swapped when it went through create_transpose
  static kapy_global view_of(const Node &ld) {
    kapy_global g = ld.global;
    if (ld.transposed) {
      std::swap(g.start0, g.start1);
      std::swap(g.end0, g.end1);
      std::swap(g.stride0, g.stride1);
    }
    return g;
  }
  bool depends_on_matmul(int id) const {
    if (id < 0) return false;
    const Node &n = nodes_[id];
    if (n.kind == Node::kMatmul) return true;
    if (n.kind != Node::kOp) return false;
    return depends_on_matmul(n.a) || depends_on_matmul(n.b) || depends_on_matmul(n.c);
  }

  // Post-order walk of the graph under `root` into a straight-line program.  A register is freed after the last use of
  // its value, so graphs far larger than the 16 registers of a program fit as long as 16 values are never live at once.
  std::vector<kapy_global> views_;  // storage for the descriptors the emitted program points at
  void emit_program(int root, std::vector<kapy_ew_inst> *prog, std::vector<const kapy_global *> *ins) {
    if (root < 0 || root >= (int)nodes_.size()) throw Error(KAPY_ERR_INVALID, "use of an undefined value");
    std::vector<int> order, uses(nodes_.size(), 0), reg(nodes_.size(), -1);
    std::vector<char> seen(nodes_.size(), 0);
    struct Walk {
      const std::vector<Node> &nodes;
      std::vector<int> &order, &uses;
      std::vector<char> &seen;
      void visit(int id) {
        ++uses[id];
        if (seen[id]) return;
        seen[id] = 1;
        const Node &n = nodes[id];
        if (n.kind == Node::kMatmul || n.kind == Node::kGlobal) throw Error(KAPY_ERR_UNSUPPORTED, "elementwise: operand is not a register tensor of this program");
        if (n.kind == Node::kOp)
          for (int o : {n.a, n.b, n.c})
            if (o >= 0) visit(o);
        order.push_back(id);
      }
    } walk{nodes_, order, uses, seen};
    walk.visit(root);
    views_.clear();
    views_.reserve(order.size());
    std::vector<int> free_regs;
    for (int r = 15; r >= 0; --r) free_regs.push_back(r);
    auto release = [&](int id) {
      if (id >= 0 && --uses[id] == 0) free_regs.push_back(reg[id]);
    };
    for (int id : order) {
      const Node &n = nodes_[id];
      kapy_ew_inst I = {n.op, 0, 0, 0, 0, n.dtype, n.rmode, n.imm};
      if (n.kind == Node::kLoad) {
        views_.push_back(view_of(n));
        ins->push_back(&views_.back());
        I.op = KAPY_EW_LD_GLOBAL;
        I.a = (int32_t)ins->size() - 1;
        I.c = n.padding;
      } else {
        I.a = n.a >= 0 ? reg[n.a] : 0;
        I.b = n.b >= 0 ? reg[n.b] : 0;
        I.c = n.c >= 0 ? reg[n.c] : 0;
        if (n.op == KAPY_EW_REDUCE_SUM || n.op == KAPY_EW_REDUCE_MAX) I.b = n.axis;
        if (n.op == KAPY_EW_CMPI || n.op == KAPY_EW_CMPF) I.c = n.pred;
        if (n.op == KAPY_EW_ARANGE) { I.a = n.ival; I.b = n.axis; }
        if (n.op == KAPY_EW_SPLAT && n.dtype >= KAPY_I8) I.a = n.ival;
        release(n.a);
        release(n.b);
        release(n.c);
      }
      if (free_regs.empty()) throw Error(KAPY_ERR_UNSUPPORTED, "elementwise: more than 16 values live at once");
      reg[id] = free_regs.back();
      free_regs.pop_back();
      I.dst = reg[id];
      prog->push_back(I);
    }
    --uses[root];
    prog->push_back({KAPY_EW_ST_GLOBAL, 0, reg[root], 0, 0, 0, KAPY_RN, 0.f});
  }

  // matmul [-> mulf splat] [-> addf broadcast(extf? ld bias)] [-> activation] [-> fptofp]: the tail goes into the epilogue
  void lower_matmul(int root, const kapy_global &out) {
    int cur = root;
    kapy_matmul_epilogue epi = {nullptr, 1.0f, -1, 0.f};
    bool tail = false;
    auto is_op = [&](int id, int op) { return id >= 0 && nodes_[id].kind == Node::kOp && nodes_[id].op == op; };
    auto splat_of = [&](int id, float *v) {
      if (!is_op(id, KAPY_EW_SPLAT)) return false;
      *v = nodes_[id].imm;
      return true;
    };
    // The value stored must have the element type of the view it is stored into (st_global: SameOperandsElementType,
    // Ops.td:163-170).  A final fptofp is the kernel's own cast: its type must be the view's and its rounding mode is
    // the kernel's; without one the f32 accumulator chain can only be stored into an f32 view.
    int rmode = KAPY_RN;
    if (is_op(cur, KAPY_EW_FPTOFP)) {
      if (nodes_[cur].dtype != out.dtype) throw Error(KAPY_ERR_VERIFY, "st_global: source and target must have same element type");
      rmode = nodes_[cur].rmode;
      cur = nodes_[cur].a;
      if (cur >= 0 && nodes_[cur].dtype != KAPY_F32) throw Error(KAPY_ERR_UNSUPPORTED, "matmul: the cast of the result must be applied to the f32 accumulator chain");
    } else if (nodes_[cur].dtype != out.dtype) {
      throw Error(KAPY_ERR_VERIFY, "st_global: source and target must have same element type");
    }
    // the activation
    float operand = 0.f;
    if (is_op(cur, KAPY_EW_MAXIMUMF) || is_op(cur, KAPY_EW_MINIMUMF)) {
      const Node &n = nodes_[cur];
      if (splat_of(n.b, &operand)) { epi.act = n.op; epi.act_operand = operand; cur = n.a; tail = true; }
      else if (splat_of(n.a, &operand)) { epi.act = n.op; epi.act_operand = operand; cur = n.b; tail = true; }
    } else if (cur >= 0 && nodes_[cur].kind == Node::kOp && nodes_[cur].op >= KAPY_EW_NEGF && nodes_[cur].op <= KAPY_EW_GELU_TANH) {
      epi.act = nodes_[cur].op;
      cur = nodes_[cur].a;
      tail = true;
    }
    // the bias: a loaded [1 x N] row, possibly widened
    kapy_global bias;
    if (is_op(cur, KAPY_EW_ADDF)) {
      // (the addend joins an f32 value: arith ops need equal element types, so a 16-bit row must have been widened)
      auto as_bias = [&](int id) {
        if (is_op(id, KAPY_EW_FPTOFP) && nodes_[id].dtype == KAPY_F32) id = nodes_[id].a;
        else if (id >= 0 && nodes_[id].kind == Node::kLoad && nodes_[id].dtype != KAPY_F32)
          throw Error(KAPY_ERR_VERIFY, "addf: operands must have same element type");
        return id >= 0 && nodes_[id].kind == Node::kLoad ? id : -1;
      };
      const Node &n = nodes_[cur];
      int b = as_bias(n.b), other = n.a;
      if (b < 0) { b = as_bias(n.a); other = n.b; }
      if (b < 0) throw Error(KAPY_ERR_UNSUPPORTED, "matmul: only a loaded bias row can be added in the epilogue");
      bias = view_of(nodes_[b]);
      epi.bias = &bias;
      cur = other;
      tail = true;
    }
    // the scale
    if (is_op(cur, KAPY_EW_MULF)) {
      const Node &n = nodes_[cur];
      float s;
      if (splat_of(n.b, &s)) { epi.alpha = s; cur = n.a; tail = true; }
      else if (splat_of(n.a, &s)) { epi.alpha = s; cur = n.b; tail = true; }
    }
    if (cur < 0 || nodes_[cur].kind != Node::kMatmul)
      throw Error(KAPY_ERR_UNSUPPORTED, "matmul: the ops on its result must be [mulf splat] [addf bias row] [activation] [fptofp]");
    const Node &mm = nodes_[cur];
    const kapy_global lhs = view_of(nodes_[mm.a]), rhs = view_of(nodes_[mm.b]);
    kapy_matmul_cfg cfg = {mm.impl_way, 0, 0, 0, rmode, 0, 0, 0, nullptr, 0};
    if (tail) {
      if (mm.c >= 0) throw Error(KAPY_ERR_UNSUPPORTED, "matmul: an accumulator input and a fused tail do not combine");
      check(kapy_matmul_fused(&lhs, &rhs, &out, &epi, &cfg, stream_));
    } else {
      kapy_global acc;
      if (mm.c >= 0) acc = view_of(nodes_[mm.c]);
      check(kapy_matmul(&lhs, &rhs, mm.c >= 0 ? &acc : nullptr, &out, &cfg, stream_));
    }
  }
};

}  // namespace kapy

#endif  // KAPY_HIP_HPP
