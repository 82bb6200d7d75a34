"""ctypes binding of libkapy_hip.so for the test and benchmark harness.

The product is the C ABI in include/kapy_hip.h; this module only loads it, declares argument
types and offers a few conveniences around torch tensors (device memory and streams).  It never
computes anything itself and has no fallback: a missing library is an ImportError, a failing call
raises KapyError with the library's own message.
"""
import ctypes as C
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(os.path.dirname(_HERE), "lib", "libkapy_hip.so")

F16, BF16, F32, F8E4M3, F8E5M2, I8, I16, I32, I1 = range(9)
RZ, RN = 0, 1
PAD_ZERO, PAD_QNAN, PAD_PINF, PAD_NINF = range(4)
CACHE_NONE, CACHE_CA, CACHE_CG, CACHE_CS = 0, 1, 2, 3
EVICT_NORMAL, EVICT_FIRST, EVICT_LAST, EVICT_UNCHANGED, NO_ALLOCATE = range(5)
OK, ERR_INVALID, ERR_VERIFY, ERR_UNSUPPORTED, ERR_HIP = 0, -1, -2, -3, -4
MATMUL_AUTO, MMA_M16N8K8_F16, MMA_M16N8K16_F16, MMA_M16N8K8_TF32, MMA_M16N8K16_F8 = 0, 1, 2, 3, 4
MFMA_32X32X16_16B, MFMA_16X16X32_16B, MFMA_16X16X128_F8, MFMA_32X32X64_F8 = 16, 17, 18, 19
DTYPE_BYTES = {F16: 2, BF16: 2, F32: 4, F8E4M3: 1, F8E5M2: 1, I8: 1, I16: 2, I32: 4, I1: 1}

(EW_LD_GLOBAL, EW_SPLAT, EW_FPTOFP, EW_ADDF, EW_SUBF, EW_MULF, EW_DIVF, EW_FMA, EW_MAXIMUMF, EW_MINIMUMF,
 EW_NEGF, EW_ABSF, EW_EXP, EW_EXP2, EW_LOG, EW_LOG2, EW_SQRT, EW_RSQRT, EW_TANH, EW_ERF, EW_GELU_TANH,
 EW_ST_GLOBAL, EW_REDUCE_SUM, EW_REDUCE_MAX, EW_FLOOR, EW_CEIL, EW_SIN, EW_COS, EW_MAXNUMF, EW_MINNUMF, EW_REMF) = range(31)
(EW_ADDI, EW_SUBI, EW_MULI, EW_DIVSI, EW_DIVUI, EW_FLOORDIVSI, EW_CEILDIVSI, EW_CEILDIVUI, EW_REMSI, EW_REMUI, EW_ANDI, EW_ORI, EW_XORI,
 EW_SHLI, EW_SHRSI, EW_SHRUI, EW_MAXSI, EW_MAXUI, EW_MINSI, EW_MINUI, EW_ABSI, EW_CMPI, EW_CMPF, EW_SELECT, EW_TRUNCI, EW_EXTSI, EW_EXTUI,
 EW_SITOFP, EW_FPTOSI, EW_BITCAST, EW_ARANGE) = range(31, 62)
(CMPI_EQ, CMPI_NE, CMPI_SLT, CMPI_SLE, CMPI_SGT, CMPI_SGE, CMPI_ULT, CMPI_ULE, CMPI_UGT, CMPI_UGE) = range(10)
(CMPF_FALSE, CMPF_OEQ, CMPF_OGT, CMPF_OGE, CMPF_OLT, CMPF_OLE, CMPF_ONE, CMPF_ORD, CMPF_UEQ, CMPF_UGT, CMPF_UGE, CMPF_ULT, CMPF_ULE, CMPF_UNE,
 CMPF_UNO, CMPF_TRUE) = range(16)

EXPORTS = [
    "kapy_version", "kapy_last_error", "kapy_device_info", "kapy_mk_global", "kapy_sv_global",
    "kapy_fragments_loops", "kapy_fragments_map", "kapy_fragments_transpose", "kapy_fragments_exchange_axes",
    "kapy_fragments_default", "kapy_layout_string", "kapy_access_simd_size", "kapy_change_source", "kapy_change_num_shuffles",
    "kapy_swizzle_offset", "kapy_swizzle_search", "kapy_swizzle_search_gfx950", "kapy_matmul_layouts", "kapy_matmul_lds_layout",
    "kapy_copy", "kapy_copy_batched", "kapy_elementwise", "kapy_fptofp", "kapy_matmul", "kapy_matmul_scaled_f8",
    "kapy_change", "kapy_reduce", "kapy_reduce_ex", "kapy_reduce_workspace_bytes", "kapy_run_mlir", "kapy_run_mlir_stats", "kapy_run_mlir_plan_stats", "kapy_parse_mlir",
    "kapy_smem_plan", "kapy_smem_barriers", "kapy_analyze_mlir",
    "kapy_elementwise_specialize", "kapy_elementwise_source", "kapy_elementwise_specialize_stats", "kapy_matmul_fused",
    "kapy_matmul_workspace_bytes", "kapy_matmul_turn_workspace_bytes", "kapy_matmul_static_workspace",
    "kapy_mk_shared", "kapy_sv_shared", "kapy_shared_address",
]


class KapyError(RuntimeError):
    def __init__(self, status, message):
        super().__init__("kapy status %d: %s" % (status, message))
        self.status = status
        self.message = message


class Global(C.Structure):
    _fields_ = [("ptr", C.c_void_p), ("start0", C.c_int32), ("start1", C.c_int32), ("end0", C.c_int32),
                ("end1", C.c_int32), ("stride0", C.c_int32), ("stride1", C.c_int32), ("dtype", C.c_int32),
                ("alignment", C.c_int32)]


class Fragments(C.Structure):
    _fields_ = [("lane_array", C.c_int32 * 2), ("lane_loops", C.c_int32 * 2), ("minor_axis", C.c_int32),
                ("major_axis", C.c_int32)]

    @classmethod
    def make(cls, lane_array, lane_loops, minor, major):
        f = cls()
        f.lane_array[:] = lane_array
        f.lane_loops[:] = lane_loops
        f.minor_axis, f.major_axis = minor, major
        return f

    def astuple(self):
        return (list(self.lane_array), list(self.lane_loops), self.minor_axis, self.major_axis)


class Swizzling(C.Structure):
    _fields_ = [("stride0", C.c_int32), ("stride1", C.c_int32), ("bank_param", C.c_int32), ("line_param", C.c_int32), ("rotate", C.c_int32)]


class CopyCfg(C.Structure):
    _fields_ = [("transpose", C.c_int32), ("padding_option", C.c_int32), ("cache_modifier", C.c_int32),
                ("evict_priority", C.c_int32), ("is_volatile", C.c_int32), ("reserved", C.c_int32)]


class Shared(C.Structure):
    _fields_ = [("offset", C.c_int64), ("start0", C.c_int32), ("start1", C.c_int32), ("end0", C.c_int32), ("end1", C.c_int32),
                ("dtype", C.c_int32), ("layout", Swizzling)]


class Grid2(C.Structure):
    _fields_ = [("n0", C.c_int32), ("n1", C.c_int32), ("src_off0", C.c_int64), ("src_off1", C.c_int64),
                ("dst_off0", C.c_int64), ("dst_off1", C.c_int64)]


class EwInst(C.Structure):
    _fields_ = [("op", C.c_int32), ("dst", C.c_int32), ("a", C.c_int32), ("b", C.c_int32), ("c", C.c_int32),
                ("dtype", C.c_int32), ("rmode", C.c_int32), ("imm", C.c_float)]


class MatmulCfg(C.Structure):
    _fields_ = [("impl_way", C.c_int32), ("tile_m", C.c_int32), ("tile_n", C.c_int32), ("tile_k", C.c_int32),
                ("rmode", C.c_int32), ("stages", C.c_int32), ("waves", C.c_int32), ("split_k", C.c_int32),
                ("workspace", C.c_void_p), ("workspace_bytes", C.c_int64), ("accumulate", C.c_int32), ("reserved", C.c_int32)]


ACCUMULATE_F32, ACCUMULATE_ELEMENT = 0, 1


class ReduceCfg(C.Structure):
    _fields_ = [("combiner", C.c_int32), ("arithmetic", C.c_int32), ("layout", C.POINTER(Fragments)), ("workspace", C.c_void_p),
                ("workspace_bytes", C.c_int64)]


(REDUCE_ADDF, REDUCE_MAXIMUMF, REDUCE_MINIMUMF, REDUCE_MULF, REDUCE_MAXNUMF, REDUCE_MINNUMF, REDUCE_ADDI, REDUCE_MULI, REDUCE_MAXSI, REDUCE_MINSI,
 REDUCE_MAXUI, REDUCE_MINUI, REDUCE_ANDI, REDUCE_ORI, REDUCE_XORI) = range(15)
REDUCE_WIDE, REDUCE_REFERENCE = 0, 1


class MatmulEpilogue(C.Structure):
    _fields_ = [("bias", C.POINTER(Global)), ("alpha", C.c_float), ("act", C.c_int32), ("act_operand", C.c_float)]


class SmemBuffer(C.Structure):
    _fields_ = [("size", C.c_int64), ("live_start", C.c_int64), ("live_end", C.c_int64), ("offset", C.c_int64)]


class SmemOp(C.Structure):
    _fields_ = [("block", C.c_int32), ("kind", C.c_int32), ("first_access", C.c_int32), ("n_accesses", C.c_int32)]


class SmemAccess(C.Structure):
    _fields_ = [("begin", C.c_int64), ("end", C.c_int64), ("is_write", C.c_int32), ("reserved", C.c_int32)]


class MlirArg(C.Structure):
    _fields_ = [("ptr", C.c_void_p), ("bytes", C.c_int64), ("i32", C.c_int32), ("reserved", C.c_int32)]


_lib = None


def lib():
    """The loaded library.  Raises ImportError when it has not been built."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise ImportError("%s is missing: build it with `make -C kapy-lang_amd` (there is no fallback path)" % LIB_PATH)
    L = C.CDLL(LIB_PATH)
    i64, i32, vp = C.c_int64, C.c_int32, C.c_void_p
    P = C.POINTER
    A2 = i64 * 2
    L.kapy_version.restype = C.c_int
    L.kapy_last_error.restype = C.c_char_p
    L.kapy_device_info.argtypes = [P(i32), P(i32), P(i32), C.c_char_p, i32]
    L.kapy_mk_global.argtypes = [P(Global), vp, i32, i32, i32, i32, i32, i32, i32]
    L.kapy_sv_global.argtypes = [P(Global), P(Global), i32, i32, i32, i32]
    L.kapy_mk_shared.argtypes = [P(Shared), i64, i32, i32, i32, i32, i32, i32]
    L.kapy_sv_shared.argtypes = [P(Shared), P(Shared), i32, i32, i32, i32]
    L.kapy_shared_address.restype = i64
    L.kapy_shared_address.argtypes = [P(Shared), i64, i64]
    L.kapy_fragments_loops.argtypes = [P(Fragments), A2, A2, A2]
    L.kapy_fragments_map.argtypes = [P(Fragments), A2, i32, A2, A2]
    L.kapy_fragments_transpose.argtypes = [P(Fragments), P(Fragments)]
    L.kapy_fragments_exchange_axes.argtypes = [P(Fragments), P(Fragments)]
    L.kapy_fragments_default.argtypes = [A2, A2, i32, P(Fragments)]
    L.kapy_layout_string.restype = i64
    L.kapy_layout_string.argtypes = [P(Fragments), A2, C.c_char_p, i64]
    L.kapy_access_simd_size.restype = i64
    L.kapy_access_simd_size.argtypes = [i64, i64, i64]
    L.kapy_change_source.argtypes = [P(Fragments), P(Fragments), A2, i64, i64, P(i64), P(i64)]
    L.kapy_change_num_shuffles.restype = i64
    L.kapy_change_num_shuffles.argtypes = [P(Fragments), P(Fragments), A2]
    L.kapy_swizzle_offset.restype = i64
    L.kapy_swizzle_offset.argtypes = [P(Swizzling), i64, i64, i64]
    L.kapy_swizzle_search.argtypes = [P(Fragments), A2, i64, i64, i64, i64, P(i32), i32]
    L.kapy_swizzle_search_gfx950.argtypes = [P(Fragments), A2, i64, i64, i64, i64, P(i32), i32]
    L.kapy_matmul_layouts.argtypes = [i32, i32, P(Fragments), P(i32)]
    L.kapy_matmul_lds_layout.argtypes = [i32, i32, P(Swizzling)]
    L.kapy_copy.argtypes = [P(Global), P(Global), P(CopyCfg), vp]
    L.kapy_copy_batched.argtypes = [P(Global), P(Global), P(CopyCfg), P(Grid2), vp]
    L.kapy_elementwise.argtypes = [P(EwInst), i32, P(P(Global)), i32, P(Global), vp]
    L.kapy_elementwise_specialize.argtypes = [P(EwInst), i32, P(P(Global)), i32, P(Global)]
    L.kapy_elementwise_specialize_stats.argtypes = [P(i64), P(i64)]
    L.kapy_elementwise_source.argtypes = [P(EwInst), i32, P(P(Global)), i32, P(Global), C.c_char_p, i64, P(i64), P(i64)]
    L.kapy_fptofp.argtypes = [P(Global), P(Global), i32, vp]
    L.kapy_matmul.argtypes = [P(Global), P(Global), P(Global), P(Global), P(MatmulCfg), vp]
    L.kapy_matmul_turn_workspace_bytes.restype = i64
    L.kapy_matmul_turn_workspace_bytes.argtypes = [P(Global), P(Global)]
    L.kapy_matmul_static_workspace.argtypes = [P(Global), P(Global), P(Global), P(Global), P(MatmulCfg), vp]
    L.kapy_matmul_workspace_bytes.restype = i64
    L.kapy_matmul_workspace_bytes.argtypes = [i64, i64]
    L.kapy_matmul_fused.argtypes = [P(Global), P(Global), P(Global), P(MatmulEpilogue), P(MatmulCfg), vp]
    L.kapy_matmul_scaled_f8.argtypes = [P(Global), P(Global), vp, vp, P(Global), P(MatmulCfg), vp]
    L.kapy_change.argtypes = [vp, P(Fragments), P(Fragments), A2, vp, vp]
    L.kapy_reduce.argtypes = [P(Global), P(Global), i32, i32, vp]
    L.kapy_reduce_ex.argtypes = [P(Global), P(Global), i32, P(ReduceCfg), vp]
    L.kapy_reduce_workspace_bytes.restype = C.c_int64
    L.kapy_reduce_workspace_bytes.argtypes = []
    L.kapy_smem_plan.restype = i64
    L.kapy_smem_plan.argtypes = [P(SmemBuffer), i32, i64]
    L.kapy_smem_barriers.argtypes = [P(SmemOp), i32, P(SmemAccess), i32, P(i32), P(i32), i32, P(i32)]
    L.kapy_analyze_mlir.argtypes = [C.c_char_p, C.c_char_p, P(i64), P(i32), P(i64), i32, P(i32), P(i32), i32]
    L.kapy_run_mlir.argtypes = [C.c_char_p, C.c_char_p, P(MlirArg), i32, i32 * 3, vp]
    L.kapy_run_mlir_stats.argtypes = [P(i64)]
    L.kapy_run_mlir_plan_stats.argtypes = [P(i64), P(i64), P(i64)]
    L.kapy_parse_mlir.argtypes = [C.c_char_p, C.c_char_p, P(i32), P(i32), P(i32)]
    for name in EXPORTS:
        f = getattr(L, name)
        if name not in ("kapy_last_error", "kapy_smem_plan", "kapy_layout_string", "kapy_access_simd_size", "kapy_change_num_shuffles", "kapy_swizzle_offset",
                        "kapy_matmul_workspace_bytes", "kapy_matmul_turn_workspace_bytes", "kapy_reduce_workspace_bytes", "kapy_shared_address"):
            f.restype = C.c_int
    _lib = L
    return L


def layout_string(frag, shape):
    n = lib().kapy_layout_string(C.byref(frag), A2(*shape), None, 0)
    if n < 0:
        raise KapyError(n, last_error())
    buf = C.create_string_buffer(n + 1)
    lib().kapy_layout_string(C.byref(frag), A2(*shape), buf, n + 1)
    return buf.value.decode()


def last_error():
    return lib().kapy_last_error().decode()


def check(status):
    if status < 0:
        raise KapyError(status, last_error())
    return status


def A2(a, b):
    return (C.c_int64 * 2)(a, b)


# ---------------------------------------------------------------- descriptors
def mk_global(ptr, size0, size1, stride0, stride1, dtype, dynamic_offset=0, alignment=16):
    g = Global()
    check(lib().kapy_mk_global(C.byref(g), C.c_void_p(ptr), dynamic_offset, size0, size1, stride0, stride1, dtype, alignment))
    return g


def sv_global(g, start0, end0, start1, end1):
    r = Global()
    check(lib().kapy_sv_global(C.byref(r), C.byref(g), start0, end0, start1, end1))
    return r


def tensor_global(t, dtype, size0=None, size1=None, stride0=None, stride1=None, dynamic_offset=0, alignment=16):
    """Descriptor over a 2-D torch tensor's storage (any torch dtype of the right width)."""
    if size0 is None:
        size0, size1 = t.shape
        stride0, stride1 = t.stride()
    return mk_global(t.data_ptr(), size0, size1, stride0, stride1, dtype, dynamic_offset, alignment)


def current_stream():
    import torch
    return C.c_void_p(torch.cuda.current_stream().cuda_stream)


# ---------------------------------------------------------------- ops
def copy(src, dst, transpose=False, padding=PAD_ZERO, cache=CACHE_NONE, evict=EVICT_NORMAL, volatile=False, stream=None):
    cfg = CopyCfg(int(transpose), padding, cache, evict, int(volatile), 0)
    check(lib().kapy_copy(C.byref(src), C.byref(dst), C.byref(cfg), stream if stream is not None else current_stream()))


def copy_batched(src, dst, grid, transpose=False, padding=PAD_ZERO, cache=CACHE_NONE, evict=EVICT_NORMAL, volatile=False, stream=None):
    cfg = CopyCfg(int(transpose), padding, cache, evict, int(volatile), 0)
    g = Grid2(*grid)
    check(lib().kapy_copy_batched(C.byref(src), C.byref(dst), C.byref(cfg), C.byref(g),
                                  stream if stream is not None else current_stream()))


def program(insts):
    arr = (EwInst * len(insts))()
    for k, d in enumerate(insts):
        arr[k] = EwInst(d["op"], d.get("dst", 0), d.get("a", 0), d.get("b", 0), d.get("c", 0), d.get("dtype", 0),
                        d.get("rmode", RN), d.get("imm", 0.0))
    return arr


def gelu_program(out_dtype=F16, scale=0.5):
    """y = GELU_tanh(x*scale + bias): ld x, ld bias, extf both, mulf by splat, addf, gelu, fptofp rn, st."""
    return program([
        dict(op=EW_LD_GLOBAL, dst=0, a=0),
        dict(op=EW_LD_GLOBAL, dst=1, a=1),
        dict(op=EW_FPTOFP, dst=2, a=0, dtype=F32),
        dict(op=EW_FPTOFP, dst=3, a=1, dtype=F32),
        dict(op=EW_SPLAT, dst=4, dtype=F32, imm=scale),
        dict(op=EW_MULF, dst=2, a=2, b=4),
        dict(op=EW_ADDF, dst=2, a=2, b=3),
        dict(op=EW_GELU_TANH, dst=2, a=2),
        dict(op=EW_FPTOFP, dst=5, a=2, dtype=out_dtype, rmode=RN),
        dict(op=EW_ST_GLOBAL, a=5),
    ])


def softmax_insts(dtype=F16):
    """Row softmax in fp32: y = exp(x - max_row(x)) / sum_row(exp(x - max_row(x))), one rounding to `dtype`."""
    return [
        dict(op=EW_LD_GLOBAL, dst=0, a=0),
        dict(op=EW_FPTOFP, dst=1, a=0, dtype=F32),
        dict(op=EW_REDUCE_MAX, dst=2, a=1, b=1),
        dict(op=EW_SUBF, dst=1, a=1, b=2),
        dict(op=EW_EXP, dst=1, a=1),
        dict(op=EW_REDUCE_SUM, dst=2, a=1, b=1),
        dict(op=EW_DIVF, dst=1, a=1, b=2),
        dict(op=EW_FPTOFP, dst=3, a=1, dtype=dtype, rmode=RN),
        dict(op=EW_ST_GLOBAL, a=3),
    ]


def layernorm_insts(n, dtype=F16, eps=1e-5, affine=True):
    """Row layer norm in fp32 over rows of n elements: ((x - mean) * rsqrt(var + eps)) * gamma + beta with
    gamma = ins[1], beta = ins[2] as [1 x n] rows when `affine`."""
    prog = [
        dict(op=EW_LD_GLOBAL, dst=0, a=0),
        dict(op=EW_FPTOFP, dst=1, a=0, dtype=F32),
        dict(op=EW_SPLAT, dst=2, dtype=F32, imm=1.0 / n),
        dict(op=EW_REDUCE_SUM, dst=3, a=1, b=1),
        dict(op=EW_MULF, dst=3, a=3, b=2),            # mean
        dict(op=EW_SUBF, dst=1, a=1, b=3),            # centred
        dict(op=EW_MULF, dst=4, a=1, b=1),
        dict(op=EW_REDUCE_SUM, dst=4, a=4, b=1),
        dict(op=EW_MULF, dst=4, a=4, b=2),            # variance
        dict(op=EW_SPLAT, dst=5, dtype=F32, imm=eps),
        dict(op=EW_ADDF, dst=4, a=4, b=5),
        dict(op=EW_RSQRT, dst=4, a=4),
        dict(op=EW_MULF, dst=1, a=1, b=4),
    ]
    if affine:
        prog += [
            dict(op=EW_LD_GLOBAL, dst=6, a=1), dict(op=EW_FPTOFP, dst=6, a=6, dtype=F32),
            dict(op=EW_LD_GLOBAL, dst=7, a=2), dict(op=EW_FPTOFP, dst=7, a=7, dtype=F32),
            dict(op=EW_MULF, dst=1, a=1, b=6), dict(op=EW_ADDF, dst=1, a=1, b=7),
        ]
    return prog + [dict(op=EW_FPTOFP, dst=8, a=1, dtype=dtype, rmode=RN), dict(op=EW_ST_GLOBAL, a=8)]


def rmsnorm_insts(n, dtype=F16, eps=1e-6):
    """Row RMS norm in fp32: x * rsqrt(mean(x^2) + eps) * gamma, gamma = ins[1] as a [1 x n] row."""
    return [
        dict(op=EW_LD_GLOBAL, dst=0, a=0),
        dict(op=EW_FPTOFP, dst=1, a=0, dtype=F32),
        dict(op=EW_MULF, dst=2, a=1, b=1),
        dict(op=EW_REDUCE_SUM, dst=2, a=2, b=1),
        dict(op=EW_SPLAT, dst=3, dtype=F32, imm=1.0 / n),
        dict(op=EW_MULF, dst=2, a=2, b=3),
        dict(op=EW_SPLAT, dst=3, dtype=F32, imm=eps),
        dict(op=EW_ADDF, dst=2, a=2, b=3),
        dict(op=EW_RSQRT, dst=2, a=2),
        dict(op=EW_MULF, dst=1, a=1, b=2),
        dict(op=EW_LD_GLOBAL, dst=4, a=1), dict(op=EW_FPTOFP, dst=4, a=4, dtype=F32),
        dict(op=EW_MULF, dst=1, a=1, b=4),
        dict(op=EW_FPTOFP, dst=5, a=1, dtype=dtype, rmode=RN),
        dict(op=EW_ST_GLOBAL, a=5),
    ]


def elementwise(prog, ins, out, stream=None):
    arr = (C.POINTER(Global) * max(len(ins), 1))(*[C.pointer(g) for g in ins])
    check(lib().kapy_elementwise(prog, len(prog), arr, len(ins), C.byref(out),
                                 stream if stream is not None else current_stream()))


def elementwise_specialize(prog, ins, out):
    """Compile the program to a kernel of its own for the current device; later elementwise() calls with the same
    program and operand signature run it."""
    arr = (C.POINTER(Global) * max(len(ins), 1))(*[C.pointer(g) for g in ins])
    check(lib().kapy_elementwise_specialize(prog, len(prog), arr, len(ins), C.byref(out)))


def elementwise_specialize_stats():
    """(specialised kernels loaded, elementwise() calls that ran one) in this process."""
    a, b = C.c_int64(0), C.c_int64(0)
    check(lib().kapy_elementwise_specialize_stats(C.byref(a), C.byref(b)))
    return a.value, b.value


def elementwise_source(prog, ins, out, compile=False):
    """(text of the specialised kernel, size of its gfx950 code object or None); needs no GPU."""
    arr = (C.POINTER(Global) * max(len(ins), 1))(*[C.pointer(g) for g in ins])
    n, code = C.c_int64(0), C.c_int64(0)
    check(lib().kapy_elementwise_source(prog, len(prog), arr, len(ins), C.byref(out), None, 0, C.byref(n), None))
    buf = C.create_string_buffer(n.value + 1)
    check(lib().kapy_elementwise_source(prog, len(prog), arr, len(ins), C.byref(out), buf, n.value + 1, None,
                                        C.byref(code) if compile else None))
    return buf.value.decode(), (code.value if compile else None)


def fptofp(src, dst, rmode=RN, stream=None):
    check(lib().kapy_fptofp(C.byref(src), C.byref(dst), rmode, stream if stream is not None else current_stream()))


def _workspace(workspace):
    """(pointer, bytes) of a workspace given as None, a (pointer, bytes) pair or a torch tensor."""
    if workspace is None:
        return None, 0
    if isinstance(workspace, tuple):
        return workspace
    return workspace.data_ptr(), workspace.numel() * workspace.element_size()


def matmul(lhs, rhs, result, acc=None, impl_way=MATMUL_AUTO, tile=(0, 0, 0), rmode=RN, stages=0, waves=0, split_k=0, workspace=None,
           static_workspace=False, accumulate=ACCUMULATE_F32, stream=None):
    """workspace: zero-initialised device memory (a torch tensor or a (pointer, bytes) pair) that lets the library split K;
    static_workspace: call kapy_matmul_static_workspace instead (the library's own array); accumulate: ACCUMULATE_ELEMENT keeps
    f16 accumulators rounded once per instruction of impl_way, the reference's arithmetic for f16 results."""
    ws, ws_bytes = _workspace(workspace)
    cfg = MatmulCfg(impl_way, tile[0], tile[1], tile[2], rmode, stages, waves, split_k, ws, ws_bytes, accumulate, 0)
    fn = lib().kapy_matmul_static_workspace if static_workspace else lib().kapy_matmul
    check(fn(C.byref(lhs), C.byref(rhs), C.byref(acc) if acc is not None else None, C.byref(result),
             C.byref(cfg), stream if stream is not None else current_stream()))


def matmul_fused(lhs, rhs, result, bias=None, alpha=1.0, act=-1, act_operand=0.0, tile=(0, 0, 0), stages=0, stream=None):
    """result = cast(act(lhs @ rhs * alpha + bias)): the elementwise tail runs in the GEMM's epilogue."""
    epi = MatmulEpilogue(C.pointer(bias) if bias is not None else None, alpha, act, act_operand)
    cfg = MatmulCfg(MATMUL_AUTO, tile[0], tile[1], tile[2], RN, stages, 0, 0, None, 0)
    check(lib().kapy_matmul_fused(C.byref(lhs), C.byref(rhs), C.byref(result), C.byref(epi), C.byref(cfg),
                                  stream if stream is not None else current_stream()))


def matmul_scaled_f8(a8, w8, row_scale_ptr, col_scale_ptr, result, split_k=0, workspace=None, tile=(0, 0, 0), stream=None):
    ws, ws_bytes = _workspace(workspace)
    cfg = MatmulCfg(MATMUL_AUTO, tile[0], tile[1], tile[2], RN, 0, 0, split_k, ws, ws_bytes)
    check(lib().kapy_matmul_scaled_f8(C.byref(a8), C.byref(w8), C.c_void_p(row_scale_ptr), C.c_void_p(col_scale_ptr),
                                      C.byref(result), C.byref(cfg), stream if stream is not None else current_stream()))


def reduce(src, dst, axis, kind=0, stream=None):
    check(lib().kapy_reduce(C.byref(src), C.byref(dst), axis, kind, stream if stream is not None else current_stream()))


def reduce_ex(src, dst, axis, combiner=0, arithmetic=REDUCE_WIDE, layout=None, workspace=None, stream=None):
    """workspace: None, a (pointer, bytes) pair or a torch tensor."""
    ptr, nbytes = _workspace(workspace)
    cfg = ReduceCfg(combiner, arithmetic, C.pointer(layout) if layout is not None else None, ptr, nbytes)
    check(lib().kapy_reduce_ex(C.byref(src), C.byref(dst), axis, C.byref(cfg), stream if stream is not None else current_stream()))


def parse_mlir(text, func_name=None):
    """(n_args, n_ops, num_warps) of a kapy.func in textual form; raises KapyError when it does not parse."""
    n_args, n_ops, warps = C.c_int32(), C.c_int32(), C.c_int32()
    check(lib().kapy_parse_mlir(text.encode(), func_name.encode() if func_name else None, C.byref(n_args), C.byref(n_ops),
                                C.byref(warps)))
    return n_args.value, n_ops.value, warps.value


def analyze_mlir(text, func_name=None):
    """(shared-memory bytes, offsets of the mk_shared buffers, barrier lines: +line before, -line after)."""
    total, nb, nbar = C.c_int64(), C.c_int32(), C.c_int32()
    offsets, lines = (C.c_int64 * 64)(), (C.c_int32 * 256)()
    check(lib().kapy_analyze_mlir(text.encode(), func_name.encode() if func_name else None, C.byref(total), C.byref(nb), offsets, 64,
                                  C.byref(nbar), lines, 256))
    return total.value, list(offsets[:min(nb.value, 64)]), list(lines[:min(nbar.value, 256)])


def run_mlir(text, args, grid, func_name=None, stream=None):
    """Executes a kapy.func given as text.  args: an int for an i32 argument; a (device pointer, bytes) pair or
    anything with data_ptr()/numel()/element_size() for a !kapy.ptr<1> argument.  grid: 1 to 3 extents."""
    arr = (MlirArg * max(len(args), 1))()
    for k, a in enumerate(args):
        if isinstance(a, int):
            arr[k].i32 = a
        elif isinstance(a, tuple):
            arr[k].ptr, arr[k].bytes = a
        else:
            arr[k].ptr, arr[k].bytes = a.data_ptr(), a.numel() * a.element_size()
    g = list(grid) + [1] * (3 - len(grid))
    check(lib().kapy_run_mlir(text.encode(), func_name.encode() if func_name else None, arr, len(args), (C.c_int32 * 3)(*g),
                              stream if stream is not None else current_stream()))


def run_mlir_stats():
    """How many kapy.st_global ops this process has run as one call for all instances in flight."""
    n = C.c_int64(0)
    check(lib().kapy_run_mlir_stats(C.byref(n)))
    return n.value


def run_mlir_plan_stats():
    """(runs whose device calls are kept, calls of run_mlir served from a kept run, launches over a table of operand
    addresses made by those) of this process."""
    plans, replays, tables = C.c_int64(0), C.c_int64(0), C.c_int64(0)
    check(lib().kapy_run_mlir_plan_stats(C.byref(plans), C.byref(replays), C.byref(tables)))
    return plans.value, replays.value, tables.value


def change(in_ptr, src, dst, shape, out_ptr, stream=None):
    check(lib().kapy_change(C.c_void_p(in_ptr), C.byref(src), C.byref(dst), A2(*shape), C.c_void_p(out_ptr),
                            stream if stream is not None else current_stream()))


def matmul_layouts(impl_way, which):
    """(fragments layout, (m, n, k)) of the lhs (0), rhs (1), accumulator (2) or accumulator with the operands exchanged (3)."""
    f, mnk = Fragments(), (C.c_int32 * 3)()
    check(lib().kapy_matmul_layouts(impl_way, which, C.byref(f), mnk))
    return f, tuple(mnk)


