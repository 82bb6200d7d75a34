"""ctypes binding of the CPU checker (oracle/libkapy_oracle.so).  Test infrastructure only.

Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg import this module.
"""
import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libkapy_oracle.so")

F16, BF16, F32, F8E4M3, F8E5M2, I8, I16, I32, I1 = range(9)
RZ, RN = 0, 1
PAD_ZERO, PAD_QNAN, PAD_PINF, PAD_NINF = range(4)
DTYPE_BYTES = {F16: 2, BF16: 2, F32: 4, F8E4M3: 1, F8E5M2: 1, I8: 1, I16: 2, I32: 4, I1: 1}
NP_STORAGE = {F16: np.uint16, BF16: np.uint16, F32: np.float32, F8E4M3: np.uint8, F8E5M2: np.uint8,
              I8: np.int8, I16: np.int16, I32: np.int32, I1: np.uint8}

(EW_LD_GLOBAL, EW_SPLAT, EW_FPTOFP, EW_ADDF, EW_SUBF, EW_MULF, EW_DIVF, EW_FMA, EW_MAXIMUMF, EW_MINIMUMF,
 EW_NEGF, EW_ABSF, EW_EXP, EW_EXP2, EW_LOG, EW_LOG2, EW_SQRT, EW_RSQRT, EW_TANH, EW_ERF, EW_GELU_TANH,
 EW_ST_GLOBAL, EW_REDUCE_SUM, EW_REDUCE_MAX, EW_FLOOR, EW_CEIL, EW_SIN, EW_COS, EW_MAXNUMF, EW_MINNUMF, EW_REMF) = range(31)
(EW_ADDI, EW_SUBI, EW_MULI, EW_DIVSI, EW_DIVUI, EW_FLOORDIVSI, EW_CEILDIVSI, EW_CEILDIVUI, EW_REMSI, EW_REMUI, EW_ANDI, EW_ORI, EW_XORI,
 EW_SHLI, EW_SHRSI, EW_SHRUI, EW_MAXSI, EW_MAXUI, EW_MINSI, EW_MINUI, EW_ABSI, EW_CMPI, EW_CMPF, EW_SELECT, EW_TRUNCI, EW_EXTSI, EW_EXTUI,
 EW_SITOFP, EW_FPTOSI, EW_BITCAST, EW_ARANGE) = range(31, 62)
(CMPI_EQ, CMPI_NE, CMPI_SLT, CMPI_SLE, CMPI_SGT, CMPI_SGE, CMPI_ULT, CMPI_ULE, CMPI_UGT, CMPI_UGE) = range(10)
(CMPF_FALSE, CMPF_OEQ, CMPF_OGT, CMPF_OGE, CMPF_OLT, CMPF_OLE, CMPF_ONE, CMPF_ORD, CMPF_UEQ, CMPF_UGT, CMPF_UGE, CMPF_ULT, CMPF_ULE, CMPF_UNE,
 CMPF_UNO, CMPF_TRUE) = range(16)


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


class EwInst(C.Structure):
    _fields_ = [("op", C.c_int32), ("dst", C.c_int32), ("a", C.c_int32), ("b", C.c_int32), ("c", C.c_int32),
                ("dtype", C.c_int32), ("rmode", C.c_int32), ("imm", C.c_float)]


def build():
    subprocess.check_call(["make", "-C", _HERE, "-s", "-B"])


_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        L = C.CDLL(_LIB_PATH)
        i64, i32, u64, dbl, vp = C.c_int64, C.c_int32, C.c_uint64, C.c_double, C.c_void_p
        P = C.POINTER
        L.ko_f64_to_f16.restype = C.c_uint16; L.ko_f64_to_f16.argtypes = [dbl, C.c_int]
        L.ko_f64_to_bf16.restype = C.c_uint16; L.ko_f64_to_bf16.argtypes = [dbl, C.c_int]
        L.ko_f64_to_e4m3.restype = C.c_uint8; L.ko_f64_to_e4m3.argtypes = [dbl, C.c_int]
        L.ko_f64_to_e5m2.restype = C.c_uint8; L.ko_f64_to_e5m2.argtypes = [dbl, C.c_int]
        L.ko_f64_to_f32.restype = C.c_float; L.ko_f64_to_f32.argtypes = [dbl, C.c_int]
        for n, t in (("f16", C.c_uint16), ("bf16", C.c_uint16), ("e4m3", C.c_uint8), ("e5m2", C.c_uint8)):
            f = getattr(L, "ko_%s_to_f64" % n)
            f.restype = dbl
            f.argtypes = [t]
        L.ko_fptofp.restype = C.c_int
        L.ko_fptofp.argtypes = [vp, C.c_int, vp, C.c_int, C.c_int, i64, C.c_int]
        L.ko_padding_word.restype = C.c_uint32; L.ko_padding_word.argtypes = [C.c_int, C.c_int]
        L.ko_splitmix64.restype = u64; L.ko_splitmix64.argtypes = [u64]
        L.ko_fill_uniform.restype = None; L.ko_fill_uniform.argtypes = [vp, C.c_int, i64, u64, u64, dbl, dbl]
        L.ko_fill_normal.restype = None; L.ko_fill_normal.argtypes = [vp, C.c_int, i64, u64, u64, dbl, dbl]
        L.ko_fill_bits16.restype = None; L.ko_fill_bits16.argtypes = [vp, i64, u64, u64]
        A2 = i64 * 2
        L.ko_fragments_loops.restype = None; L.ko_fragments_loops.argtypes = [P(Fragments), A2, A2, A2]
        L.ko_layout_string.restype = i64; L.ko_layout_string.argtypes = [P(Fragments), A2, C.c_char_p, i64]
        L.ko_fragments_map12.restype = None; L.ko_fragments_map12.argtypes = [P(Fragments), A2, C.c_int, i64, i64, A2]
        L.ko_fragments_map3.restype = None; L.ko_fragments_map3.argtypes = [P(Fragments), A2, i64, i64, P(i64), P(i64)]
        L.ko_fragments_transpose.restype = None; L.ko_fragments_transpose.argtypes = [P(Fragments), P(Fragments)]
        L.ko_fragments_exchange_axes.restype = None; L.ko_fragments_exchange_axes.argtypes = [P(Fragments), P(Fragments)]
        L.ko_fragments_default.restype = None; L.ko_fragments_default.argtypes = [A2, A2, C.c_int, i64, P(Fragments)]
        L.ko_access_simd_size.restype = i64; L.ko_access_simd_size.argtypes = [i64, i64, i64, i64]
        L.ko_change_source.restype = None
        L.ko_change_source.argtypes = [P(Fragments), P(Fragments), A2, i64, i64, P(i64), P(i64)]
        L.ko_change_num_shuffles.restype = i64; L.ko_change_num_shuffles.argtypes = [P(Fragments), P(Fragments), A2, i64]
        L.ko_swizzle_offset.restype = i64; L.ko_swizzle_offset.argtypes = [i64] * 8
        L.ko_no_bank_conflict.restype = C.c_int
        L.ko_no_bank_conflict.argtypes = [P(Fragments), A2] + [i64] * 8
        L.ko_swizzle_search.restype = C.c_int
        L.ko_swizzle_search.argtypes = [P(Fragments), A2, i64, i64, i64, i64, i64, i64, P(i64), C.c_int]
        L.ko_no_bank_conflict_gfx950.restype = C.c_int
        L.ko_no_bank_conflict_gfx950.argtypes = [P(Fragments), A2] + [i64] * 7
        L.ko_swizzle_search_gfx950.restype = C.c_int
        L.ko_swizzle_search_gfx950.argtypes = [P(Fragments), A2, i64, i64, i64, i64, P(i64), C.c_int]
        L.ko_swizzle_offset_rotated.restype = i64; L.ko_swizzle_offset_rotated.argtypes = [i64] * 8
        L.ko_mk_global.restype = C.c_int
        L.ko_mk_global.argtypes = [P(Global), vp, i32, i32, i32, i32, i32, C.c_int, i32]
        L.ko_sv_global.restype = C.c_int; L.ko_sv_global.argtypes = [P(Global), P(Global), i32, i32, i32, i32]
        L.ko_ld_global.restype = None; L.ko_ld_global.argtypes = [P(Global), i64, i64, C.c_int, vp]
        L.ko_st_global.restype = None; L.ko_st_global.argtypes = [vp, i64, i64, P(Global)]
        L.ko_transpose_tile.restype = None; L.ko_transpose_tile.argtypes = [vp, i64, i64, C.c_int, vp]
        L.ko_change_tile.restype = None
        L.ko_change_tile.argtypes = [vp, P(Fragments), P(Fragments), A2, C.c_int, i64, vp]
        L.ko_copy.restype = C.c_int; L.ko_copy.argtypes = [P(Global), P(Global), C.c_int, C.c_int]
        L.ko_copy_batched.restype = C.c_int
        L.ko_copy_batched.argtypes = [P(Global), P(Global), C.c_int, C.c_int, i32, i32, i64, i64, i64, i64]
        L.ko_elementwise.restype = C.c_int
        L.ko_elementwise.argtypes = [P(EwInst), C.c_int, P(P(Global)), C.c_int, P(Global)]
        L.ko_matmul.restype = C.c_int
        L.ko_matmul.argtypes = [P(Global), P(Global), P(Global), P(Global), C.c_int]
        L.ko_matmul_f16acc.restype = C.c_int
        L.ko_matmul_f16acc.argtypes = [P(Global), P(Global), P(Global), P(Global), C.c_int]
        L.ko_matmul_scaled_f8.restype = C.c_int
        L.ko_matmul_scaled_f8.argtypes = [P(Global), P(Global), vp, vp, P(Global)]
        L.ko_quantize_e4m3.restype = None
        L.ko_quantize_e4m3.argtypes = [vp, i64, i64, i64, i64, C.c_int, vp, vp]
        L.ko_reduce.restype = C.c_int; L.ko_reduce.argtypes = [P(Global), P(Global), C.c_int, C.c_int]
        L.ko_reduce_reference.restype = C.c_int; L.ko_reduce_reference.argtypes = [P(Global), P(Global), C.c_int, C.c_int, P(Fragments), i64]
        L.ko_baseline_gemm.restype = C.c_int; L.ko_baseline_gemm.argtypes = [P(Global), P(Global), vp, vp, P(Global), P(dbl)]
        L.ko_baseline_gelu_f16.restype = C.c_int; L.ko_baseline_gelu_f16.argtypes = [vp, vp, C.c_float, vp, i64, i64, i64]
        L.ko_baseline_transpose16.restype = C.c_int; L.ko_baseline_transpose16.argtypes = [vp, vp, i64, i64]
        L.ko_baseline_permute_bhsd_bshd16.restype = C.c_int; L.ko_baseline_permute_bhsd_bshd16.argtypes = [vp, vp, i64, i64, i64, i64]
        L.ko_num_threads.restype = C.c_int
        L.ko_decode.restype = dbl; L.ko_decode.argtypes = [vp, C.c_int, i64]
        _lib = L
    return _lib


# ---------------------------------------------------------------- numpy conveniences
def _ptr(a):
    return a.ctypes.data_as(C.c_void_p)


def mk_global(arr, size0, size1, stride0, stride1, dtype, dynamic_offset=0, alignment=16):
    """Descriptor over a numpy storage array (keeps no reference: caller keeps `arr` alive)."""
    g = Global()
    rc = lib().ko_mk_global(C.byref(g), _ptr(arr), dynamic_offset, size0, size1, stride0, stride1, dtype, alignment)
    assert rc == 0
    return g


def sv_global(g, start0, end0, start1, end1):
    r = Global()
    lib().ko_sv_global(C.byref(r), C.byref(g), start0, end0, start1, end1)
    return r


def fill_uniform(n, dtype, seed, stream=0, lo=-1.0, hi=1.0):
    out = np.empty(n, dtype=NP_STORAGE[dtype])
    lib().ko_fill_uniform(_ptr(out), dtype, n, seed, stream, lo, hi)
    return out


def fill_normal(n, dtype, seed, stream=0, mean=0.0, std=1.0):
    out = np.empty(n, dtype=NP_STORAGE[dtype])
    lib().ko_fill_normal(_ptr(out), dtype, n, seed, stream, mean, std)
    return out


def fill_bits16(n, seed, stream=0):
    out = np.empty(n, dtype=np.uint16)
    lib().ko_fill_bits16(_ptr(out), n, seed, stream)
    return out


def decode(arr, dtype):
    """Storage array -> float64 values."""
    if dtype == F16:
        return arr.view(np.float16).astype(np.float64)
    if dtype == BF16:
        return (arr.astype(np.uint32) << 16).view(np.float32).astype(np.float64)
    if dtype in (F8E4M3, F8E5M2):
        f = lib().ko_e4m3_to_f64 if dtype == F8E4M3 else lib().ko_e5m2_to_f64
        table = np.array([f(i) for i in range(256)])
        return table[arr]
    return arr.astype(np.float64)


def fptofp(src, src_dtype, dst_dtype, rmode=RN, via_f16=0):
    dst = np.empty(src.shape, dtype=NP_STORAGE[dst_dtype])
    rc = lib().ko_fptofp(_ptr(src), src_dtype, _ptr(dst), dst_dtype, rmode, src.size, via_f16)
    if rc:
        raise ValueError("ko_fptofp rejected the cast: %d" % rc)
    return dst


def program(insts):
    """insts: list of dicts(op=, dst=, a=, b=, c=, dtype=, rmode=, imm=)."""
    arr = (EwInst * len(insts))()
    for k, d in enumerate(insts):
        arr[k] = EwInst(d["op"], d.get("dst", 0), d.get("a", 0), d.get("b", 0), d.get("c", 0), d.get("dtype", 0),
                        d.get("rmode", RN), d.get("imm", 0.0))
    return arr


def elementwise(prog, ins, out):
    arr = (C.POINTER(Global) * len(ins))(*[C.pointer(g) for g in ins])
    return lib().ko_elementwise(prog, len(prog), arr, len(ins), C.byref(out))


def gelu_program(in_dtype=F16, out_dtype=F16, scale=0.5):
    """y = GELU_tanh(x*scale + bias): ld x, ld bias (row broadcast), extf, mulf, addf, gelu, fptofp rn, st."""
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
