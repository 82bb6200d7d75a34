"""ctypes binding of libkapy_probe.so (include/kapy_probe.h): measurement kernels beside the product library - what the device
sustains (matrix-instruction loops, copies in every form, L2 reads, issue slots beside matrix instructions) and one matrix
instruction on one wavefront, registers in and out.  The benchmark and the tests use it; nothing of the product does.  Errors
are reported through the product library (KapyError carries its message)."""
import ctypes as C
import os

from kapy_hip import check, current_stream, lib as _product_lib

LIB_PATH = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "lib", "libkapy_probe.so")
EXPORTS = ["kapy_mfma_probe", "kapy_probe_mfma", "kapy_probe_copy", "kapy_probe_copy_tiled", "kapy_probe_copy_runs", "kapy_probe_l2_read", "kapy_probe_issue", "kapy_probe_read"]
_lib = None


def lib():
    """The loaded probe library.  Raises ImportError when it has not been built."""
    global _lib
    if _lib is not None:
        return _lib
    _product_lib()          # (its error state and device query are the ones the probes use)
    if not os.path.exists(LIB_PATH):
        raise ImportError("%s is missing: build it with `make -C kapy-lang_amd`" % LIB_PATH)
    L = C.CDLL(LIB_PATH)
    i64, i32, vp = C.c_int64, C.c_int32, C.c_void_p
    P = C.POINTER
    L.kapy_mfma_probe.argtypes = [i32, i32, i32, i32, vp, vp, vp, vp]
    L.kapy_probe_mfma.argtypes = [i32, i32, vp, i32, vp, vp, P(i32), P(i64), vp]
    L.kapy_probe_copy.argtypes = [vp, vp, i64, i32, i32, i32, i32, vp, P(i32), vp]
    L.kapy_probe_read.argtypes = [vp, i64, i32, i32, i32, vp, P(i32), vp]
    L.kapy_probe_copy_tiled.argtypes = [vp, vp, i64, i64, i32, vp]
    L.kapy_probe_l2_read.argtypes = [vp, i64, i32, i32, i32, vp, P(i32), P(i64), vp]
    L.kapy_probe_copy_runs.argtypes = [vp, vp, i64, i64, i32, vp]
    L.kapy_probe_issue.argtypes = [i32, i32, i32, vp, i32, vp, P(i32), P(i64), vp]
    _lib = L
    return L


def mfma_probe(impl_way, lhs_dtype, rhs_dtype, exchanged, lhs_ptr, rhs_ptr, acc_ptr, stream=None):
    check(lib().kapy_mfma_probe(impl_way, lhs_dtype, rhs_dtype, int(exchanged), C.c_void_p(lhs_ptr), C.c_void_p(rhs_ptr), C.c_void_p(acc_ptr),
                                stream if stream is not None else current_stream()))


def probe_mfma(impl_way, dtype, operands_ptr, iterations, sink_ptr, ticks_ptr=None, stream=None):
    """(workgroups, flops) of one launch of the matrix-instruction loop."""
    wgs, flops = C.c_int32(0), C.c_int64(0)
    check(lib().kapy_probe_mfma(impl_way, dtype, C.c_void_p(operands_ptr), iterations, C.c_void_p(sink_ptr), C.c_void_p(ticks_ptr) if ticks_ptr else None,
                                C.byref(wgs), C.byref(flops), stream if stream is not None else current_stream()))
    return wgs.value, flops.value


def probe_copy(src_ptr, dst_ptr, nbytes, vectors_per_lane=4, nt_load=False, nt_store=False, persistent_per_cu=0, ticks_ptr=None, stream=None):
    wgs = C.c_int32(0)
    check(lib().kapy_probe_copy(C.c_void_p(src_ptr), C.c_void_p(dst_ptr), nbytes, vectors_per_lane, int(nt_load), int(nt_store), persistent_per_cu,
                                C.c_void_p(ticks_ptr) if ticks_ptr else None, C.byref(wgs), stream if stream is not None else current_stream()))
    return wgs.value


def probe_read(src_ptr, nbytes, vectors_per_lane=4, nt_load=False, persistent_per_cu=0, sink_ptr=None, stream=None):
    wgs = C.c_int32(0)
    check(lib().kapy_probe_read(C.c_void_p(src_ptr), nbytes, vectors_per_lane, int(nt_load), persistent_per_cu, C.c_void_p(sink_ptr) if sink_ptr else None,
                                C.byref(wgs), stream if stream is not None else current_stream()))
    return wgs.value


def probe_copy_tiled(src_ptr, dst_ptr, rows, row_bytes, through_lds=False, stream=None):
    check(lib().kapy_probe_copy_tiled(C.c_void_p(src_ptr), C.c_void_p(dst_ptr), rows, row_bytes, int(through_lds),
                                      stream if stream is not None else current_stream()))


def probe_copy_runs(src_ptr, dst_ptr, rows, row_bytes, run_bytes, stream=None):
    check(lib().kapy_probe_copy_runs(C.c_void_p(src_ptr), C.c_void_p(dst_ptr), rows, row_bytes, run_bytes, stream if stream is not None else current_stream()))


def probe_issue(impl_way, filler, count, src_ptr, iterations, sink_ptr, stream=None):
    """(workgroups, flops) of one launch of the issue probe: matrix instructions with fillers in the gaps between them."""
    wgs, flops = C.c_int32(0), C.c_int64(0)
    check(lib().kapy_probe_issue(impl_way, filler, count, C.c_void_p(src_ptr) if src_ptr else None, iterations, C.c_void_p(sink_ptr),
                                 C.byref(wgs), C.byref(flops), stream if stream is not None else current_stream()))
    return wgs.value, flops.value


def probe_l2_read(src_ptr, window_bytes, iterations, workgroups_per_cu=1, to_lds=True, sink_ptr=None, stream=None):
    """(workgroups, bytes read) of one launch of the L2 read loop."""
    wgs, nbytes = C.c_int32(0), C.c_int64(0)
    check(lib().kapy_probe_l2_read(C.c_void_p(src_ptr), window_bytes, iterations, workgroups_per_cu, int(to_lds), C.c_void_p(sink_ptr) if sink_ptr else None,
                                   C.byref(wgs), C.byref(nbytes), stream if stream is not None else current_stream()))
    return wgs.value, nbytes.value
