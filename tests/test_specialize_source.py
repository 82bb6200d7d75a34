"""Host-side checks of the specialised-kernel generator: the text it writes for a program, that the runtime compiler
turns that text into a gfx950 code object (no GPU needed for that), and its refusals."""
import ctypes as C

import pytest

import kapy_hip as kh

L, ADD, MUL, DIV, ST, CAST, SPL = kh.EW_LD_GLOBAL, kh.EW_ADDF, kh.EW_MULF, kh.EW_DIVF, kh.EW_ST_GLOBAL, kh.EW_FPTOFP, kh.EW_SPLAT


def _g(rows, cols, dtype, pitch=None):
    return kh.mk_global(0x100000, rows, cols, pitch or cols, 1, dtype)


def _has_runtime_compiler():
    for name in ("libhiprtc.so.7", "libhiprtc.so"):
        try:
            C.CDLL(name)
            return True
        except OSError:
            pass
    return False


SILU = [dict(op=L, dst=0, a=0), dict(op=CAST, dst=1, a=0, dtype=kh.F32), dict(op=kh.EW_NEGF, dst=2, a=1), dict(op=kh.EW_EXP, dst=2, a=2),
        dict(op=SPL, dst=3, dtype=kh.F32, imm=1.0), dict(op=ADD, dst=2, a=2, b=3), dict(op=DIV, dst=2, a=1, b=2),
        dict(op=CAST, dst=4, a=2, dtype=kh.F16, rmode=kh.RN), dict(op=ST, a=4)]


def test_generated_text_follows_the_program():
    src, _ = kh.elementwise_source(kh.program(SILU), [_g(16, 256, kh.F16)], _g(16, 256, kh.F16))
    kernel = src[src.index('extern "C" __global__'):]
    assert "void kapy_ew_flat_" in kernel and "(JitArgs p)" in kernel
    assert "constexpr bool NARROW = true" in kernel
    assert kernel.count("fetch8_row<RAGGED>(") == 1          # one operand, fetched once per vector
    assert "0x3f800000u" in kernel                           # the splat 1.0 as its bit pattern
    assert "unary8<NARROW>(%d, %d" % (kh.EW_EXP, kh.F32) in kernel and "div8(" in kernel
    assert "round8" not in kernel                            # every op is fp32; the final cast is the store's own rounding
    assert "store8_row<NARROW, RAGGED>(p.out, %d" % kh.F16 in kernel
    # dead code is not emitted: an unused load and an unused product
    prog = [dict(op=L, dst=0, a=0), dict(op=L, dst=1, a=1), dict(op=MUL, dst=2, a=0, b=1), dict(op=ST, a=0)]
    src, _ = kh.elementwise_source(kh.program(prog), [_g(8, 64, kh.BF16), _g(8, 64, kh.BF16)], _g(8, 64, kh.BF16))
    kernel = src[src.index('extern "C" __global__'):]
    assert "raw1" not in kernel and "__fmul_rn" not in kernel
    # fp8 anywhere takes the machines' wide form
    prog = [dict(op=L, dst=0, a=0), dict(op=CAST, dst=1, a=0, dtype=kh.F8E4M3, rmode=kh.RN), dict(op=ST, a=1)]
    src, _ = kh.elementwise_source(kh.program(prog), [_g(8, 64, kh.F16)], _g(8, 64, kh.F8E4M3))
    assert "constexpr bool NARROW = false" in src


@pytest.mark.skipif(not _has_runtime_compiler(), reason="libhiprtc is not installed")
def test_generated_text_compiles_for_gfx950():
    cases = [
        (SILU, [_g(16, 256, kh.F16)], _g(16, 256, kh.F16)),
        ([dict(op=L, dst=0, a=0), dict(op=L, dst=1, a=1), dict(op=L, dst=2, a=2), dict(op=L, dst=3, a=3), dict(op=MUL, dst=4, a=0, b=1),
          dict(op=ADD, dst=4, a=4, b=2), dict(op=DIV, dst=4, a=4, b=3), dict(op=kh.EW_TANH, dst=4, a=4), dict(op=ST, a=4)],
         [_g(32, 64, kh.BF16, 128), _g(1, 64, kh.BF16), _g(32, 1, kh.BF16), _g(1, 1, kh.BF16)], _g(32, 64, kh.BF16)),
        ([dict(op=L, dst=0, a=0), dict(op=SPL, dst=1, dtype=kh.F32, imm=0.25), dict(op=DIV, dst=0, a=1, b=0), dict(op=DIV, dst=0, a=0, b=1),
          dict(op=CAST, dst=2, a=0, dtype=kh.F8E5M2, rmode=kh.RZ), dict(op=ST, a=2)], [_g(8, 64, kh.F32)], _g(8, 64, kh.F8E5M2)),
        ([dict(op=SPL, dst=0, dtype=kh.F16, imm=3.0), dict(op=ST, a=0)], [], _g(8, 64, kh.F16)),
    ]
    for insts, ins, out in cases:
        _, code_bytes = kh.elementwise_source(kh.program(insts), ins, out, compile=True)
        assert code_bytes > 1000


def test_row_programs_and_ragged_widths_get_the_other_skeletons():
    softmax_like = [dict(op=L, dst=0, a=0), dict(op=kh.EW_REDUCE_MAX, dst=1, a=0, b=1), dict(op=kh.EW_SUBF, dst=0, a=0, b=1), dict(op=ST, a=0)]
    src, _ = kh.elementwise_source(kh.program(softmax_like), [_g(8, 8192, kh.F16)], _g(8, 8192, kh.F16))
    kernel = src[src.index('extern "C" __global__'):]
    assert "__launch_bounds__(256)" in kernel and "CH = 4, THREADS = 256" in kernel and "RAGGED = false" in kernel
    assert kernel.count("row_reduce<CH, THREADS, false, RAGGED>") == 1 and "for (int32_t i = blockIdx.x; i < p.rows; i += gridDim.x)" in kernel
    src, _ = kh.elementwise_source(kh.program(softmax_like), [_g(8, 100, kh.F16, 104)], _g(8, 100, kh.F16, 104))   # 100 columns, rows 104 apart
    kernel = src[src.index('extern "C" __global__'):]
    assert "CH = 1, THREADS = 64" in kernel and "RAGGED = true" in kernel
    if _has_runtime_compiler():
        for shape in ((8, 8192, None), (8, 100, 104), (3, 32768, None)):
            _, code_bytes = kh.elementwise_source(kh.program(softmax_like), [_g(shape[0], shape[1], kh.F32, shape[2])], _g(shape[0], shape[1], kh.F32, shape[2]), compile=True)
            assert code_bytes > 1000


def test_refusals():
    add = [dict(op=L, dst=0, a=0), dict(op=L, dst=1, a=1), dict(op=ADD, dst=2, a=0, b=1), dict(op=ST, a=2)]
    def refused(insts, ins, out):
        with pytest.raises(kh.KapyError) as e:
            kh.elementwise_source(kh.program(insts), ins, out)
        return str(e.value)
    assert "status %d" % kh.ERR_UNSUPPORTED in refused(add, [_g(8, 64, kh.F16, 68), _g(8, 64, kh.F16)], _g(8, 64, kh.F16))    # pitch % 8
    assert "status %d" % kh.ERR_UNSUPPORTED in refused(add, [_g(8, 60, kh.F16), _g(8, 60, kh.F16)], _g(8, 60, kh.F16))        # rows start unaligned
    column_reduce = [dict(op=L, dst=0, a=0), dict(op=kh.EW_REDUCE_MAX, dst=1, a=0, b=0), dict(op=kh.EW_SUBF, dst=0, a=0, b=1), dict(op=ST, a=0)]
    assert "status %d" % kh.ERR_UNSUPPORTED in refused(column_reduce, [_g(8, 64, kh.F16)], _g(8, 64, kh.F16))
    long_rows = [dict(op=L, dst=0, a=0), dict(op=kh.EW_REDUCE_MAX, dst=1, a=0, b=1), dict(op=ST, a=1)]
    assert "status %d" % kh.ERR_UNSUPPORTED in refused(long_rows, [_g(2, 32776, kh.F16)], _g(2, 32776, kh.F16))
    padded = [dict(op=L, dst=0, a=0, c=kh.PAD_QNAN), dict(op=ST, a=0)]
    assert "status %d" % kh.ERR_UNSUPPORTED in refused(padded, [_g(8, 64, kh.F16)], _g(8, 64, kh.F16))
    mistyped = [dict(op=L, dst=0, a=0), dict(op=L, dst=1, a=1), dict(op=ADD, dst=2, a=0, b=1), dict(op=ST, a=2)]
    assert "status %d" % kh.ERR_VERIFY in refused(mistyped, [_g(8, 64, kh.F16), _g(8, 64, kh.BF16)], _g(8, 64, kh.F16))   # the verifier comes first


def test_specialise_without_a_gpu_fails_loudly():
    import torch
    if torch.cuda.is_available():
        pytest.skip("a GPU is present")
    with pytest.raises(kh.KapyError) as e:
        kh.elementwise_specialize(kh.program(SILU), [_g(16, 256, kh.F16)], _g(16, 256, kh.F16))
    assert "no CPU fallback" in str(e.value)


@pytest.mark.skipif(not _has_runtime_compiler(), reason="libhiprtc is not installed")
def test_code_objects_are_kept_in_the_cache_directory(tmp_path, monkeypatch):
    import os
    import time
    monkeypatch.setenv("KAPY_EW_CACHE_DIR", str(tmp_path))
    prog = kh.program([dict(op=L, dst=0, a=0), dict(op=kh.EW_ERF, dst=0, a=0), dict(op=kh.EW_ABSF, dst=0, a=0), dict(op=ST, a=0)])
    args = ([_g(24, 72, kh.F32)], _g(24, 72, kh.F32))
    t0 = time.time()
    _, first = kh.elementwise_source(prog, *args, compile=True)
    t1 = time.time()
    files = sorted(os.listdir(tmp_path))
    assert len(files) == 1 and files[0].startswith("kapy_ew_") and files[0].endswith(".co")
    assert os.path.getsize(tmp_path / files[0]) == first
    _, second = kh.elementwise_source(prog, *args, compile=True)      # read back, not compiled again
    t2 = time.time()
    assert second == first and sorted(os.listdir(tmp_path)) == files
    assert t2 - t1 < max(0.05, (t1 - t0) / 3)
    # another program: another file; a broken file is replaced by a fresh compile
    kh.elementwise_source(kh.program([dict(op=L, dst=0, a=0), dict(op=kh.EW_NEGF, dst=0, a=0), dict(op=ST, a=0)]), *args, compile=True)
    assert len(os.listdir(tmp_path)) == 2
    open(tmp_path / files[0], "wb").close()
    _, third = kh.elementwise_source(prog, *args, compile=True)
    assert third == first and os.path.getsize(tmp_path / files[0]) == first


@pytest.mark.skipif(not _has_runtime_compiler(), reason="no libhiprtc on this machine")
def test_integer_compare_select_and_arange_programs_compile():
    """Programs with integer registers: a flat one over i32 operands with an i1 condition, and a causal-masked softmax (arange,
    cmpi, select in front of the row reduces) on the row skeleton; both must compile to a gfx950 code object."""
    flat = [dict(op=L, dst=0, a=0), dict(op=L, dst=1, a=1), dict(op=kh.EW_DIVSI, dst=2, a=0, b=1), dict(op=kh.EW_SHRSI, dst=2, a=2, b=1),
            dict(op=kh.EW_CMPI, dst=3, a=2, b=0, c=kh.CMPI_ULT), dict(op=kh.EW_SPLAT, dst=4, dtype=kh.I32, a=-7), dict(op=kh.EW_SELECT, dst=5, a=3, b=2, c=4),
            dict(op=kh.EW_SITOFP, dst=6, a=5, dtype=kh.BF16), dict(op=ST, a=6)]
    src, code = kh.elementwise_source(kh.program(flat), [_g(16, 256, kh.I32), _g(1, 256, kh.I32)], _g(16, 256, kh.BF16), compile=True)
    kernel = src[src.index('extern "C" __global__'):]
    assert "int_binary(%d" % kh.EW_DIVSI in kernel and "int_compare(%d" % kh.CMPI_ULT in kernel and "convert_reg(%d" % kh.EW_SITOFP in kernel
    assert "constexpr bool NARROW = false" in kernel and code > 0
    rows = [dict(op=L, dst=0, a=0), dict(op=CAST, dst=1, a=0, dtype=kh.F32), dict(op=kh.EW_ARANGE, dst=2, a=0, b=0), dict(op=kh.EW_ARANGE, dst=3, a=0, b=1),
            dict(op=kh.EW_CMPI, dst=4, a=3, b=2, c=kh.CMPI_SLE), dict(op=SPL, dst=5, dtype=kh.F32, imm=float("-inf")), dict(op=kh.EW_SELECT, dst=1, a=4, b=1, c=5),
            dict(op=kh.EW_REDUCE_MAX, dst=6, a=1, b=1), dict(op=kh.EW_SUBF, dst=1, a=1, b=6), dict(op=kh.EW_EXP, dst=1, a=1), dict(op=kh.EW_REDUCE_SUM, dst=6, a=1, b=1),
            dict(op=DIV, dst=1, a=1, b=6), dict(op=CAST, dst=7, a=1, dtype=kh.F16, rmode=kh.RN), dict(op=ST, a=7)]
    src, code = kh.elementwise_source(kh.program(rows), [_g(64, 1024, kh.F16)], _g(64, 1024, kh.F16), compile=True)
    kernel = src[src.index('extern "C" __global__'):]
    assert "void kapy_ew_rows_" in kernel and "int_reg(0 + i)" in kernel and "threadIdx.x) * 8 + e)" in kernel and code > 0
