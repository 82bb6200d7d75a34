"""GPU parity for the integer, compare, select and conversion ops of elementwise programs (arith.addi ... arith.select,
kapy.arange; ElementwiseOpToLLVM.cpp:1178-1215, SelectOpToLLVM.cpp:21-98, ArangeOpToLLVM.cpp:22-50): the register machine and
the kernels compiled at run time against the checker, bit for bit (integer work), and a causal-masked softmax - arange, cmpi and
select in front of the row reduces - to the elementwise bar of 2 ulp."""
import numpy as np
import pytest

import kapy_hip as kh
from gpu_util import dev_zeros, dglobal, sync, to_dev, to_host, ulp_diff_f16

pytestmark = pytest.mark.gpu

NP_OF = {1: np.uint8, 2: np.uint16, 4: np.uint32}
NP_INT = {kh.I8: np.int8, kh.I16: np.int16, kh.I32: np.int32}
BITS = {kh.I8: 8, kh.I16: 16, kh.I32: 32}
L, ST = kh.EW_LD_GLOBAL, kh.EW_ST_GLOBAL
INT_BINARY = [kh.EW_ADDI, kh.EW_SUBI, kh.EW_MULI, kh.EW_DIVSI, kh.EW_DIVUI, kh.EW_FLOORDIVSI, kh.EW_CEILDIVSI, kh.EW_CEILDIVUI, kh.EW_REMSI, kh.EW_REMUI,
              kh.EW_ANDI, kh.EW_ORI, kh.EW_XORI, kh.EW_SHLI, kh.EW_SHRSI, kh.EW_SHRUI, kh.EW_MAXSI, kh.EW_MAXUI, kh.EW_MINSI, kh.EW_MINUI]


def _run(ko, insts, ins_np, in_dtypes, out_dtype, m, n, in_shapes=None, compile_it=False):
    """(device result, checker result) of one program; compile_it: specialise first and require that the compiled kernel ran."""
    outb = kh.DTYPE_BYTES[out_dtype]
    want = np.zeros((m, n), NP_OF[outb])
    in_shapes = in_shapes or [(m, n)] * len(ins_np)
    gos = [ko.mk_global(a, s[0], s[1], s[1], 1, dt) for a, s, dt in zip(ins_np, in_shapes, in_dtypes)]
    assert ko.elementwise(ko.program(insts), gos, ko.mk_global(want, m, n, n, 1, out_dtype)) == 0
    devs = [to_dev(a) for a in ins_np]
    dins = [dglobal(t, s[0], s[1], s[1], 1, dt) for t, s, dt in zip(devs, in_shapes, in_dtypes)]
    dout = dev_zeros(m * n, outb, fill=0x55 if outb == 1 else 0x5555)
    prog = kh.program(insts)
    if compile_it:
        kh.elementwise_specialize(prog, dins, dglobal(dout, m, n, n, 1, out_dtype))
    before = kh.elementwise_specialize_stats()[1]
    kh.elementwise(prog, dins, dglobal(dout, m, n, n, 1, out_dtype))
    sync()
    if compile_it:
        assert kh.elementwise_specialize_stats()[1] - before == 1
    return to_host(dout, NP_OF[outb], (m, n)), want


def _operands(rng, dt, m, n):
    bits = BITS[dt]
    lo, hi = -(1 << (bits - 1)), (1 << (bits - 1)) - 1
    special = np.array([0, 1, -1, 2, -2, lo, hi, lo + 1, 3, 7, bits - 1, bits, bits + 1], np.int64)

    def one():
        a = rng.integers(lo, hi + 1, size=m * n, dtype=np.int64)
        pick = rng.integers(0, 4, size=m * n)
        a = np.where(pick == 0, rng.integers(-9, 10, size=m * n, dtype=np.int64), a)
        a = np.where(pick == 1, special[rng.integers(0, len(special), size=m * n)], a)
        return a.reshape(m, n).astype(NP_INT[dt])
    return one(), one()


@pytest.mark.parametrize("dt", [kh.I8, kh.I16, kh.I32])
def test_every_integer_op_on_the_register_machine(ko, dt):
    rng = np.random.default_rng(10 + dt)
    m, n = 37, 53                                        # ragged: the element-wise machine
    x, y = _operands(rng, dt, m, n)
    ld2 = [dict(op=L, dst=0, a=0), dict(op=L, dst=1, a=1)]
    for op in INT_BINARY:
        got, want = _run(ko, ld2 + [dict(op=op, dst=2, a=0, b=1), dict(op=ST, a=2)], [x, y], [dt, dt], dt, m, n)
        assert np.array_equal(got, want), "op %d" % op
    for pred in range(10):
        got, want = _run(ko, ld2 + [dict(op=kh.EW_CMPI, dst=2, a=0, b=1, c=pred), dict(op=ST, a=2)], [x, y], [dt, dt], kh.I1, m, n)
        assert np.array_equal(got, want), "cmpi %d" % pred
        got, want = _run(ko, ld2 + [dict(op=kh.EW_CMPI, dst=2, a=0, b=1, c=pred), dict(op=kh.EW_SELECT, dst=3, a=2, b=0, c=1), dict(op=ST, a=3)],
                         [x, y], [dt, dt], dt, m, n)
        assert np.array_equal(got, want)
    got, want = _run(ko, [dict(op=L, dst=0, a=0), dict(op=kh.EW_ABSI, dst=1, a=0), dict(op=ST, a=1)], [x], [dt], dt, m, n)
    assert np.array_equal(got, want)
    for od in (kh.I8, kh.I16, kh.I32):
        if od == dt:
            continue
        ops = [kh.EW_TRUNCI] if BITS[od] < BITS[dt] else [kh.EW_EXTSI, kh.EW_EXTUI]
        for op in ops:
            got, want = _run(ko, [dict(op=L, dst=0, a=0), dict(op=op, dst=1, a=0, dtype=od), dict(op=ST, a=1)], [x], [dt], od, m, n)
            assert np.array_equal(got, want), "cast %d -> %d" % (dt, od)
    for fd in (kh.F32, kh.F16, kh.BF16):
        got, want = _run(ko, [dict(op=L, dst=0, a=0), dict(op=kh.EW_SITOFP, dst=1, a=0, dtype=fd), dict(op=ST, a=1)], [x], [dt], fd, m, n)
        assert np.array_equal(got, want), "sitofp -> %d" % fd


@pytest.mark.parametrize("dt", [kh.I8, kh.I16, kh.I32])
@pytest.mark.parametrize("m,n", [(64, 256), (33, 1000)])
def test_integer_chains_compiled_equal_the_checker(ko, dt, m, n):
    """Two chains that between them hold every binary integer op, folded with xori so that every op's result reaches the
    store, through the register machine and through a compiled kernel (whole vectors and a ragged width)."""
    rng = np.random.default_rng(20 + dt + n)
    x, y = _operands(rng, dt, m, n)
    for ops in (INT_BINARY[:10], INT_BINARY[10:]):
        insts = [dict(op=L, dst=0, a=0), dict(op=L, dst=1, a=1), dict(op=kh.EW_SPLAT, dst=2, dtype=dt, a=0)]
        for op in ops:
            insts += [dict(op=op, dst=3, a=0, b=1), dict(op=kh.EW_XORI, dst=2, a=2, b=3), dict(op=kh.EW_ADDI, dst=2, a=2, b=2)]
        insts += [dict(op=ST, a=2)]
        machine, want = _run(ko, insts, [x, y], [dt, dt], dt, m, n)
        assert np.array_equal(machine, want)
        compiled, want = _run(ko, insts, [x, y], [dt, dt], dt, m, n, compile_it=True)
        assert np.array_equal(compiled, want)


def test_cmpf_select_and_conversions_compiled_and_interpreted(ko):
    rng = np.random.default_rng(3)
    m, n = 48, 264
    a = (rng.standard_normal((m, n)) * 10.0 ** rng.integers(-2, 11, size=(m, n))).astype(np.float32)
    b = np.where(rng.integers(0, 3, size=(m, n)) == 0, a, rng.standard_normal((m, n)).astype(np.float32)).astype(np.float32)
    a[0, :8] = [np.nan, np.inf, -np.inf, 2147483648.0, -2147483904.0, -0.75, 0.0, -0.0]
    b[0, :8] = [1.0, np.nan, -np.inf, 0.0, 0.0, 0.0, -0.0, 0.0]
    au, bu = a.view(np.uint32), b.view(np.uint32)
    ld2 = [dict(op=L, dst=0, a=0), dict(op=L, dst=1, a=1)]
    for compile_it in (False, True):
        for pred in range(16):
            # select(a <pred> b, fptosi(a), -7) as i32
            insts = ld2 + [dict(op=kh.EW_CMPF, dst=2, a=0, b=1, c=pred), dict(op=kh.EW_FPTOSI, dst=3, a=0, dtype=kh.I32),
                           dict(op=kh.EW_SPLAT, dst=4, dtype=kh.I32, a=-7), dict(op=kh.EW_SELECT, dst=5, a=2, b=3, c=4), dict(op=ST, a=5)]
            got, want = _run(ko, insts, [au, bu], [kh.F32, kh.F32], kh.I32, m, n, compile_it=compile_it)
            assert np.array_equal(got, want), "cmpf %d compiled=%s" % (pred, compile_it)
        for od in (kh.I16, kh.I8):
            got, want = _run(ko, [dict(op=L, dst=0, a=0), dict(op=kh.EW_FPTOSI, dst=1, a=0, dtype=od), dict(op=ST, a=1)], [au], [kh.F32], od, m, n, compile_it=compile_it)
            assert np.array_equal(got, want)
        # sitofp of large i32 to every float type: one rounding (bf16 from the integer's own bits)
        xi = rng.integers(-(1 << 31), 1 << 31, size=(m, n), dtype=np.int64).astype(np.int32)
        xi[0, :6] = [0x00808000, 0x00818000, 0x00808001, -0x00808000, 0x7FFFFFFF, -(1 << 31)]
        for fd in (kh.F32, kh.BF16, kh.F16):
            got, want = _run(ko, [dict(op=L, dst=0, a=0), dict(op=kh.EW_SITOFP, dst=1, a=0, dtype=fd), dict(op=ST, a=1)], [xi], [kh.I32], fd, m, n, compile_it=compile_it)
            assert np.array_equal(got, want), "sitofp -> %d" % fd
        # bitcast f32 <-> i32 around an integer op: flip the sign bit, take the magnitude ordering as integers
        fin = np.where(np.isfinite(a), a, 1.5).astype(np.float32).view(np.uint32)
        insts = [dict(op=L, dst=0, a=0), dict(op=kh.EW_BITCAST, dst=1, a=0, dtype=kh.I32), dict(op=kh.EW_SPLAT, dst=2, dtype=kh.I32, a=-(1 << 31)),
                 dict(op=kh.EW_XORI, dst=1, a=1, b=2), dict(op=kh.EW_BITCAST, dst=3, a=1, dtype=kh.F32), dict(op=ST, a=3)]
        got, want = _run(ko, insts, [fin], [kh.F32], kh.F32, m, n, compile_it=compile_it)
        assert np.array_equal(got, want) and np.array_equal(got, fin ^ 0x80000000)
        f16 = ko.fill_normal(m * n, kh.F16, 77).reshape(m, n)
        insts = [dict(op=L, dst=0, a=0), dict(op=kh.EW_BITCAST, dst=1, a=0, dtype=kh.I16), dict(op=kh.EW_SPLAT, dst=2, dtype=kh.I16, a=0x7FFF),
                 dict(op=kh.EW_ANDI, dst=1, a=1, b=2), dict(op=kh.EW_BITCAST, dst=3, a=1, dtype=kh.F16), dict(op=ST, a=3)]
        got, want = _run(ko, insts, [f16], [kh.F16], kh.F16, m, n, compile_it=compile_it)
        assert np.array_equal(got, want) and np.array_equal(got, f16 & 0x7FFF)          # |x| by its bits


def test_integer_operands_broadcast_and_i1_results(ko):
    """Row, column and scalar integer operands, an i1 result in memory, an i8 mask read back as the condition of a select."""
    rng = np.random.default_rng(4)
    m, n = 40, 136
    x = rng.integers(-1000, 1000, size=(m, n)).astype(np.int32)
    row = rng.integers(-1000, 1000, size=(1, n)).astype(np.int32)
    col = rng.integers(-1000, 1000, size=(m, 1)).astype(np.int32)
    one = np.array([[17]], np.int32)
    insts = [dict(op=L, dst=0, a=0), dict(op=L, dst=1, a=1), dict(op=L, dst=2, a=2), dict(op=L, dst=3, a=3),
             dict(op=kh.EW_ADDI, dst=4, a=0, b=1), dict(op=kh.EW_MULI, dst=4, a=4, b=2), dict(op=kh.EW_REMSI, dst=4, a=4, b=3),
             dict(op=kh.EW_CMPI, dst=5, a=4, b=1, c=kh.CMPI_SLT), dict(op=ST, a=5)]
    for compile_it in (False, True):
        got, want = _run(ko, insts, [x, row, col, one], [kh.I32] * 4, kh.I1, m, n, in_shapes=[(m, n), (1, n), (m, 1), (1, 1)], compile_it=compile_it)
        assert np.array_equal(got, want) and set(np.unique(got)) <= {0, 1}
        assert np.array_equal(got, ((((x + row) * col) - np.trunc(((x + row) * col) / 17.0).astype(np.int64) * 17) < row).astype(np.uint8))
    mask = rng.integers(0, 2, size=(m, n)).astype(np.uint8)
    f = ko.fill_normal(m * n, kh.F16, 5).reshape(m, n)
    insts = [dict(op=L, dst=0, a=0), dict(op=L, dst=1, a=1), dict(op=kh.EW_NEGF, dst=2, a=1), dict(op=kh.EW_SELECT, dst=3, a=0, b=1, c=2), dict(op=ST, a=3)]
    for compile_it in (False, True):
        got, want = _run(ko, insts, [mask, f], [kh.I1, kh.F16], kh.F16, m, n, compile_it=compile_it)
        assert np.array_equal(got, want) and np.array_equal(got, np.where(mask == 1, f, f ^ 0x8000))


def _causal_softmax_insts(dtype, axis=1):
    """softmax over `axis` of x where column <= row, -inf elsewhere: arange x 2, cmpi, select, then the softmax chain."""
    ninf = float("-inf")
    return [dict(op=L, dst=0, a=0), dict(op=kh.EW_FPTOFP, dst=1, a=0, dtype=kh.F32),
            dict(op=kh.EW_ARANGE, dst=2, a=0, b=0), dict(op=kh.EW_ARANGE, dst=3, a=0, b=1), dict(op=kh.EW_CMPI, dst=4, a=3, b=2, c=kh.CMPI_SLE),
            dict(op=kh.EW_SPLAT, dst=5, dtype=kh.F32, imm=ninf), dict(op=kh.EW_SELECT, dst=1, a=4, b=1, c=5),
            dict(op=kh.EW_REDUCE_MAX, dst=6, a=1, b=axis), dict(op=kh.EW_SUBF, dst=1, a=1, b=6), dict(op=kh.EW_EXP, dst=1, a=1),
            dict(op=kh.EW_REDUCE_SUM, dst=6, a=1, b=axis), dict(op=kh.EW_DIVF, dst=1, a=1, b=6),
            dict(op=kh.EW_FPTOFP, dst=7, a=1, dtype=dtype, rmode=kh.RN), dict(op=ST, a=7)]


@pytest.mark.parametrize("dtype", [kh.F16, kh.BF16])
@pytest.mark.parametrize("m,n", [(64, 64), (300, 1024), (100, 2056)])
def test_causal_masked_softmax_rows(ko, dtype, m, n):
    x = ko.fill_normal(m * n, dtype, 41 + n, std=2.0).reshape(m, n)
    got, want = _run(ko, _causal_softmax_insts(dtype), [x], [dtype], dtype, m, n)     # compiled on its first call: no machine takes integer row programs
    assert ulp_diff_f16(got, want).max() <= 2
    g = ko.decode(got, dtype)
    assert not np.triu(g, 1).any()                                                     # nothing above the diagonal
    assert np.allclose(g.sum(axis=1), 1.0, atol=2e-2)
    xf = ko.decode(x, dtype)
    ref = np.where(np.tril(np.ones((m, n), bool)), xf, -np.inf)
    ref = np.exp(ref - ref.max(axis=1, keepdims=True))
    ref /= ref.sum(axis=1, keepdims=True)
    assert np.abs(g - ref).max() <= 2.0 ** (-9 if dtype == kh.F16 else -6)


def test_masked_column_maximum_on_the_column_machine(ko):
    """Integer ops in a program whose reduce runs along axis 0: max over the rows i >= j of each column j (the column machine
    steps through the same register-machine instructions)."""
    m, n = 90, 70
    x = ko.fill_normal(m * n, kh.F16, 51).reshape(m, n)
    insts = [dict(op=L, dst=0, a=0), dict(op=kh.EW_ARANGE, dst=1, a=0, b=0), dict(op=kh.EW_ARANGE, dst=2, a=0, b=1), dict(op=kh.EW_CMPI, dst=3, a=1, b=2, c=kh.CMPI_SGE),
             dict(op=kh.EW_SPLAT, dst=4, dtype=kh.F16, imm=float("-inf")), dict(op=kh.EW_SELECT, dst=0, a=3, b=0, c=4), dict(op=kh.EW_REDUCE_MAX, dst=5, a=0, b=0),
             dict(op=ST, a=5)]
    got, want = _run(ko, insts, [x], [kh.F16], kh.F16, m, n)
    assert np.array_equal(got, want)
    xf = np.where(np.tril(np.ones((m, n), bool)), x.view(np.float16).astype(np.float64), -np.inf)
    assert np.array_equal(got[0].view(np.float16).astype(np.float64), xf.max(axis=0))


def test_integer_programs_are_verified_like_the_reference_types_them(ko):
    x = to_dev(np.zeros((4, 8), np.int32))
    g = dglobal(x, 4, 8, 8, 1, kh.I32)
    f = dglobal(x, 4, 8, 8, 1, kh.F32)
    out = dglobal(dev_zeros(32, 4), 4, 8, 8, 1, kh.I32)
    ld = [dict(op=L, dst=0, a=0), dict(op=L, dst=1, a=1)]
    cases = [(ld + [dict(op=kh.EW_ADDI, dst=2, a=0, b=1), dict(op=ST, a=2)], "same element type"),
             (ld + [dict(op=kh.EW_ADDF, dst=2, a=0, b=0), dict(op=ST, a=2)], "f16, bf16 or f32"),
             (ld + [dict(op=kh.EW_SELECT, dst=2, a=0, b=0, c=0), dict(op=ST, a=2)], "i1"),
             (ld + [dict(op=kh.EW_EXTSI, dst=2, a=0, dtype=kh.I16), dict(op=ST, a=2)], "wider"),
             (ld + [dict(op=kh.EW_BITCAST, dst=2, a=0, dtype=kh.F16), dict(op=ST, a=2)], "same bit width"),
             (ld + [dict(op=kh.EW_CMPI, dst=2, a=0, b=0, c=10), dict(op=ST, a=2)], "predicate"),
             (ld + [dict(op=kh.EW_REDUCE_SUM, dst=2, a=0, b=1), dict(op=ST, a=2)], "f16, bf16 or f32")]
    for insts, text in cases:
        with pytest.raises(kh.KapyError) as e:
            kh.elementwise(kh.program(insts), [g, f], out)
        assert e.value.status in (kh.ERR_VERIFY, kh.ERR_INVALID) and text in e.value.message, e.value.message
