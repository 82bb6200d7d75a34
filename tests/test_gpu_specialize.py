"""GPU parity for elementwise programs compiled to kernels of their own (kapy_elementwise_specialize): the same
programs the stepwise machines run, against the oracle to the same bar (bit-exact where every op is exactly
rounded, <= 2 ulp of the 16-bit result otherwise), with the launch counter showing that the compiled kernel ran."""
import numpy as np
import pytest

import kapy_hip as kh
from gpu_util import dev_zeros, dglobal, sync, to_dev, to_host, ulp_diff_f16
from test_gpu_elementwise import _check_ulp

pytestmark = pytest.mark.gpu

L, ADD, SUB, MUL, DIV, FMA, MAX, MIN, ST, CAST, SPL = (kh.EW_LD_GLOBAL, kh.EW_ADDF, kh.EW_SUBF, kh.EW_MULF, kh.EW_DIVF, kh.EW_FMA, kh.EW_MAXIMUMF,
                                                        kh.EW_MINIMUMF, kh.EW_ST_GLOBAL, kh.EW_FPTOFP, kh.EW_SPLAT)
NP_OF = {1: np.uint8, 2: np.uint16, 4: np.uint32}


def _both(ko, insts, ins_np, in_dtypes, out_dtype, m, n, in_shapes=None, expect_compiled=True):
    """(result of the machines, result after specialising, oracle); asserts which path served the second call."""
    outb = kh.DTYPE_BYTES[out_dtype]
    want = np.zeros((m, n), dtype=NP_OF[outb])
    in_shapes = in_shapes or [(m, n)] * len(ins_np)
    gos = [ko.mk_global(a, s[0], s[1], s[1], 1, dt) for a, s, dt in zip(ins_np, in_shapes, in_dtypes)]
    assert ko.elementwise(ko.program(insts), gos, ko.mk_global(want, m, n, n, 1, out_dtype)) == 0
    devs = [to_dev(a) for a in ins_np]
    prog = kh.program(insts)
    dins = [dglobal(t, s[0], s[1], s[1], 1, dt) for t, s, dt in zip(devs, in_shapes, in_dtypes)]
    results = []
    for step in range(2):
        dout = dev_zeros(m * n, outb)
        before = kh.elementwise_specialize_stats()[1]
        kh.elementwise(prog, dins, dglobal(dout, m, n, n, 1, out_dtype))
        sync()
        ran_compiled = kh.elementwise_specialize_stats()[1] - before
        results.append(to_host(dout, NP_OF[outb], (m, n)))
        if step == 0:
            if ran_compiled:   # an earlier test specialised the same program: nothing to compare the machines with
                results.append(results[0])
                break
            try:
                kh.elementwise_specialize(prog, dins, dglobal(dout, m, n, n, 1, out_dtype))
            except kh.KapyError as e:
                assert not expect_compiled, str(e)
                assert e.args[0].startswith("kapy status %d" % kh.ERR_UNSUPPORTED)
        else:
            assert ran_compiled == (1 if expect_compiled else 0)
    return results[0], results[1], want


@pytest.mark.parametrize("dtype", [kh.F16, kh.BF16])
@pytest.mark.parametrize("m,n", [(16, 256), (33, 1000), (1, 8), (700, 4104)])
def test_exactly_rounded_arithmetic_is_bit_exact(ko, dtype, m, n):
    a = ko.fill_normal(m * n, dtype, 31, 0).reshape(m, n)
    b = ko.fill_normal(m * n, dtype, 31, 1).reshape(m, n)
    insts = [dict(op=L, dst=0, a=0), dict(op=L, dst=1, a=1), dict(op=MUL, dst=2, a=0, b=1), dict(op=ADD, dst=2, a=2, b=0),
             dict(op=SUB, dst=3, a=2, b=1), dict(op=MAX, dst=3, a=3, b=0), dict(op=FMA, dst=3, a=3, b=1, c=0), dict(op=MIN, dst=3, a=3, b=2),
             dict(op=ST, a=3)]
    machine, compiled, want = _both(ko, insts, [a, b], [dtype, dtype], dtype, m, n)
    assert np.array_equal(compiled, want)
    assert np.array_equal(machine, want)


def test_every_operand_kind_reversed_operands_division_and_a_value_used_three_times(ko):
    m, n = 24, 512
    a = ko.fill_normal(m * n, kh.F16, 21, 0).reshape(m, n)
    b = ko.fill_uniform(m * n, kh.F16, 21, 1, 0.5, 2.0).reshape(m, n)
    row, col, one = ko.fill_normal(n, kh.F16, 21, 2), ko.fill_normal(m, kh.F16, 21, 3), ko.fill_normal(1, kh.F16, 21, 4)
    # ((a - b*row) / ((a + col) max (b - one))) * a + a: `a` feeds four ops, which the stack machine can only re-evaluate
    insts = [dict(op=L, dst=0, a=0), dict(op=L, dst=1, a=1), dict(op=L, dst=2, a=2), dict(op=L, dst=3, a=3), dict(op=L, dst=4, a=4),
             dict(op=MUL, dst=5, a=1, b=2), dict(op=SUB, dst=5, a=0, b=5), dict(op=ADD, dst=6, a=0, b=3), dict(op=SUB, dst=7, a=1, b=4),
             dict(op=MAX, dst=6, a=6, b=7), dict(op=DIV, dst=5, a=5, b=6), dict(op=FMA, dst=5, a=5, b=0, c=0), dict(op=ST, a=5)]
    machine, compiled, want = _both(ko, insts, [a, b, row, col, one], [kh.F16] * 5, kh.F16, m, n, [(m, n), (m, n), (1, n), (m, 1), (1, 1)])
    _check_ulp(compiled, want, kh.F16)
    assert np.array_equal(compiled, machine)   # the same device helpers, the same roundings


def test_f32_and_fp8_operands_and_results(ko):
    m, n = 16, 256
    a = ko.fill_normal(m * n, kh.F16, 21, 0).reshape(m, n)
    b = ko.fill_uniform(m * n, kh.F16, 21, 1, 0.5, 2.0).reshape(m, n)
    insts = [dict(op=L, dst=0, a=0), dict(op=L, dst=1, a=1), dict(op=CAST, dst=2, a=0, dtype=kh.F32), dict(op=CAST, dst=3, a=1, dtype=kh.F32),
             dict(op=MUL, dst=4, a=2, b=3), dict(op=SUB, dst=5, a=3, b=2), dict(op=ADD, dst=6, a=2, b=3), dict(op=FMA, dst=7, a=4, b=5, c=6),
             dict(op=ST, a=7)]
    _, compiled, want = _both(ko, insts, [a, b], [kh.F16] * 2, kh.F32, m, n)
    assert np.array_equal(compiled, want)
    x32 = ko.fill_normal(m * n, kh.F32, 22, 0).reshape(m, n)
    for f8 in (kh.F8E4M3, kh.F8E5M2):
        for rmode in (kh.RN, kh.RZ):
            insts = [dict(op=L, dst=0, a=0), dict(op=SPL, dst=1, dtype=kh.F32, imm=37.5), dict(op=MUL, dst=0, a=0, b=1),
                     dict(op=CAST, dst=2, a=0, dtype=f8, rmode=rmode), dict(op=ST, a=2)]
            _, q, wantq = _both(ko, insts, [x32], [kh.F32], f8, m, n)
            assert np.array_equal(q, wantq)
        insts = [dict(op=L, dst=0, a=0), dict(op=CAST, dst=1, a=0, dtype=kh.BF16), dict(op=ST, a=1)]
        _, back, want = _both(ko, insts, [wantq], [f8], kh.BF16, m, n)
        assert np.array_equal(back, want)
    # f16 -> e4m3 with a per-row scale: the activation quantiser in front of the W8A8 matmul
    scale = ko.fill_uniform(m, kh.F32, 23, 0, 0.5, 4.0)
    insts = [dict(op=L, dst=0, a=0), dict(op=CAST, dst=0, a=0, dtype=kh.F32), dict(op=L, dst=1, a=1), dict(op=MUL, dst=0, a=0, b=1),
             dict(op=CAST, dst=2, a=0, dtype=kh.F8E4M3, rmode=kh.RN), dict(op=ST, a=2)]
    _, q, wantq = _both(ko, insts, [a, scale], [kh.F16, kh.F32], kh.F8E4M3, m, n, [(m, n), (m, 1)])
    assert np.array_equal(q, wantq)


@pytest.mark.parametrize("dtype", [kh.F16, kh.BF16])
def test_silu_and_explicit_gelu_chains(ko, dtype):
    m, n = 32, 1024
    x = ko.fill_normal(m * n, dtype, 9, 0, 0.0, 3.0).reshape(m, n)
    c = lambda r, v: dict(op=SPL, dst=r, dtype=kh.F32, imm=v)
    silu = [dict(op=L, dst=0, a=0), dict(op=CAST, dst=1, a=0, dtype=kh.F32), dict(op=kh.EW_NEGF, dst=2, a=1), dict(op=kh.EW_EXP, dst=2, a=2),
            c(3, 1.0), dict(op=ADD, dst=2, a=2, b=3), dict(op=DIV, dst=2, a=1, b=2), dict(op=CAST, dst=4, a=2, dtype=dtype, rmode=kh.RN),
            dict(op=ST, a=4)]
    machine, compiled, want = _both(ko, silu, [x], [dtype], dtype, m, n)
    _check_ulp(compiled, want, dtype)
    assert np.array_equal(compiled, machine)
    gelu = [dict(op=L, dst=0, a=0), dict(op=CAST, dst=1, a=0, dtype=kh.F32), dict(op=MUL, dst=2, a=1, b=1), dict(op=MUL, dst=2, a=2, b=1),
            c(3, 0.044715), dict(op=FMA, dst=2, a=2, b=3, c=1), c(3, 0.7978845608028654), dict(op=MUL, dst=2, a=2, b=3),
            dict(op=kh.EW_TANH, dst=2, a=2), c(3, 1.0), dict(op=ADD, dst=2, a=2, b=3), c(3, 0.5), dict(op=MUL, dst=4, a=1, b=3),
            dict(op=MUL, dst=2, a=2, b=4), dict(op=CAST, dst=5, a=2, dtype=dtype, rmode=kh.RN), dict(op=ST, a=5)]
    _, compiled, want = _both(ko, gelu, [x], [dtype], dtype, m, n)
    _check_ulp(compiled, want, dtype)


@pytest.mark.parametrize("op", [kh.EW_EXP, kh.EW_EXP2, kh.EW_LOG, kh.EW_LOG2, kh.EW_SQRT, kh.EW_RSQRT, kh.EW_TANH, kh.EW_ERF, kh.EW_ABSF,
                                kh.EW_NEGF])
def test_unary_ops_with_special_values(ko, op):
    m, n = 8, 256
    x = ko.fill_normal(m * n, kh.F16, 40 + op, 0).reshape(m, n)
    sp = np.array([0.0, -0.0, np.inf, -np.inf, np.nan, 60000.0, -60000.0, 1e-7, -8.0, 8.0, 11.0, -11.0], dtype=np.float16).view(np.uint16)
    x.ravel()[:len(sp)] = sp
    insts = [dict(op=L, dst=0, a=0), dict(op=CAST, dst=1, a=0, dtype=kh.F32), dict(op=op, dst=1, a=1),
             dict(op=CAST, dst=2, a=1, dtype=kh.F16, rmode=kh.RN), dict(op=ST, a=2)]
    _, compiled, want = _both(ko, insts, [x], [kh.F16], kh.F16, m, n)
    _check_ulp(compiled, want, kh.F16)


def test_a_kernel_serves_only_the_operand_signature_it_was_compiled_for(ko):
    """Specialised for two full operands; the same program with a row operand goes to the machines (and stays correct)."""
    m, n = 16, 128
    a = ko.fill_normal(m * n, kh.F16, 51, 0).reshape(m, n)
    b = ko.fill_normal(m * n, kh.F16, 51, 1).reshape(m, n)
    insts = [dict(op=L, dst=0, a=0), dict(op=L, dst=1, a=1), dict(op=MUL, dst=2, a=0, b=1), dict(op=SUB, dst=2, a=2, b=1), dict(op=ST, a=2)]
    _, compiled, want = _both(ko, insts, [a, b], [kh.F16] * 2, kh.F16, m, n)
    assert np.array_equal(compiled, want)
    before = kh.elementwise_specialize_stats()
    row = np.ascontiguousarray(b[0])
    want = np.zeros((m, n), np.uint16)
    assert ko.elementwise(ko.program(insts), [ko.mk_global(a, m, n, n, 1, kh.F16), ko.mk_global(row, 1, n, n, 1, kh.F16)],
                          ko.mk_global(want, m, n, n, 1, kh.F16)) == 0
    da, dr, dout = to_dev(a), to_dev(row), dev_zeros(m * n, 2)
    kh.elementwise(kh.program(insts), [dglobal(da, m, n, n, 1, kh.F16), dglobal(dr, 1, n, n, 1, kh.F16)], dglobal(dout, m, n, n, 1, kh.F16))
    sync()
    assert kh.elementwise_specialize_stats() == before
    assert np.array_equal(to_host(dout, np.uint16, (m, n)), want)
    # rows that do not start 8 elements apart cannot be specialised at all
    n2 = 100
    a2, b2 = np.ascontiguousarray(a[:, :n2]), np.ascontiguousarray(b[:, :n2])
    _, second, want = _both(ko, insts, [a2, b2], [kh.F16] * 2, kh.F16, m, n2, expect_compiled=False)
    assert np.array_equal(second, want)


def _windows(ko, arrays, dtypes, out_dtype, m, width, pitch, kinds):
    """Oracle and device descriptors of [m x width] windows into buffers whose rows lie `pitch` elements apart (row operands: one row)."""
    outb = kh.DTYPE_BYTES[out_dtype]
    want = np.full(m * pitch, 0x5a, dtype=np.uint8).repeat(outb).view(NP_OF[outb])[:m * pitch].copy()
    shape = lambda kind: (1, width) if kind == "row" else (m, 1) if kind == "col" else (m, width)
    pitch_of = lambda kind: 1 if kind == "col" else pitch
    o_ins = [ko.mk_global(a, shape(k)[0], shape(k)[1], pitch_of(k), 1, dt) for a, dt, k in zip(arrays, dtypes, kinds)]
    devs = [to_dev(a) for a in arrays]
    d_ins = [dglobal(t, shape(k)[0], shape(k)[1], pitch_of(k), 1, dt) for t, dt, k in zip(devs, dtypes, kinds)]
    return want, o_ins, d_ins, devs


@pytest.mark.parametrize("width", [9, 100, 1001, 8190])
@pytest.mark.parametrize("which", ["x*y+x 16-bit", "quantise f32->e4m3", "softmax", "layernorm"])
def test_ragged_widths_flat_and_rowwise(ko, width, which):
    """Rows start 8 elements apart but hold a width that is not a multiple of 8: the last vector of every row moves element
    by element, reduces skip the elements past the width, and nothing outside the window is written."""
    m, pitch = 11, (width + 7) // 8 * 8 + 8
    dt = kh.BF16
    if which == "x*y+x 16-bit":
        insts = [dict(op=L, dst=0, a=0), dict(op=L, dst=1, a=1), dict(op=MUL, dst=2, a=0, b=1), dict(op=ADD, dst=2, a=2, b=0), dict(op=ST, a=2)]
        arrays, dtypes, kinds, out_dt = [ko.fill_normal(m * pitch, dt, 3, 0), ko.fill_normal(m * pitch, dt, 3, 1)], [dt, dt], ["full", "full"], dt
    elif which == "quantise f32->e4m3":
        insts = [dict(op=L, dst=0, a=0), dict(op=L, dst=1, a=1), dict(op=MUL, dst=0, a=0, b=1), dict(op=CAST, dst=2, a=0, dtype=kh.F8E4M3, rmode=kh.RN), dict(op=ST, a=2)]
        arrays, dtypes, kinds, out_dt = [ko.fill_normal(m * pitch, kh.F32, 4, 0, 0.0, 50.0), ko.fill_uniform(m, kh.F32, 4, 1, 0.5, 4.0)], [kh.F32, kh.F32], ["full", "col"], kh.F8E4M3
    elif which == "softmax":
        insts, arrays, dtypes, kinds, out_dt = kh.softmax_insts(dt), [ko.fill_normal(m * pitch, dt, 5, 0, 0.0, 2.0)], [dt], ["full"], dt
    else:
        insts = kh.layernorm_insts(width, dt)
        arrays = [ko.fill_normal(m * pitch, dt, 6, 0, 0.0, 2.0), ko.fill_normal(pitch, dt, 6, 1, 1.0, 0.5), ko.fill_normal(pitch, dt, 6, 2, 0.0, 0.5)]
        dtypes, kinds, out_dt = [dt] * 3, ["full", "row", "row"], dt
    want, o_ins, d_ins, devs = _windows(ko, arrays, dtypes, out_dt, m, width, pitch, kinds)
    outb = kh.DTYPE_BYTES[out_dt]
    assert ko.elementwise(ko.program(insts), o_ins, ko.mk_global(want, m, width, pitch, 1, out_dt)) == 0
    dout = to_dev(np.full(m * pitch, 0x5a, dtype=np.uint8).repeat(outb).view(NP_OF[outb])[:m * pitch].copy())
    prog = kh.program(insts)
    kh.elementwise_specialize(prog, d_ins, dglobal(dout, m, width, pitch, 1, out_dt))
    before = kh.elementwise_specialize_stats()[1]
    kh.elementwise(prog, d_ins, dglobal(dout, m, width, pitch, 1, out_dt))
    sync()
    assert kh.elementwise_specialize_stats()[1] == before + 1
    got = to_host(dout, NP_OF[outb], (m, pitch))
    want = want.reshape(m, pitch)
    assert np.array_equal(got[:, width:], want[:, width:])          # the gap between rows keeps its fill
    if which in ("softmax", "layernorm"):
        _check_ulp_away_from_cancellation(np.ascontiguousarray(got[:, :width]), np.ascontiguousarray(want[:, :width]), dt)
    else:
        assert np.array_equal(got[:, :width], want[:, :width])


def test_strided_views_with_offsets(ko):
    """Operands and result are windows of larger buffers (row pitch above the width, a start inside the buffer)."""
    m, n, pitch = 20, 64, 96
    a = ko.fill_normal(m * pitch + 16, kh.BF16, 61, 0)
    b = ko.fill_normal(m * pitch + 16, kh.BF16, 61, 1)
    insts = [dict(op=L, dst=0, a=0), dict(op=L, dst=1, a=1), dict(op=MUL, dst=2, a=0, b=1), dict(op=ADD, dst=2, a=2, b=1),
             dict(op=MAX, dst=2, a=2, b=0), dict(op=ST, a=2)]
    want = np.full(m * pitch + 16, 0x1234, np.uint16)
    view = lambda mk, buf: mk(buf, m, n, pitch, 1, kh.BF16)
    def window(g):
        g.start1, g.end1 = 8, 8 + n
        return g
    assert ko.elementwise(ko.program(insts), [window(view(ko.mk_global, a)), window(view(ko.mk_global, b))], window(view(ko.mk_global, want))) == 0
    da, db = to_dev(a), to_dev(b)
    dview = lambda t: window(dglobal(t, m, n, pitch, 1, kh.BF16))
    prog = kh.program(insts)
    kh.elementwise_specialize(prog, [dview(da), dview(db)], dview(da))
    dout = to_dev(np.full(m * pitch + 16, 0x1234, np.uint16))
    before = kh.elementwise_specialize_stats()[1]
    kh.elementwise(prog, [dview(da), dview(db)], dview(dout))
    sync()
    assert kh.elementwise_specialize_stats()[1] == before + 1
    assert np.array_equal(to_host(dout, np.uint16, (m * pitch + 16,)), want)   # nothing outside the window is touched


def test_full_size_program_sampled_against_the_oracle(ko):
    """z = x*y + x on fp16 8192x8192: the whole result on the GPU, 32 rows spread over it against the oracle."""
    m = n = 8192
    x = ko.fill_normal(m * n, kh.F16, 0, 0).reshape(m, n)
    y = ko.fill_normal(m * n, kh.F16, 0, 1).reshape(m, n)
    insts = [dict(op=L, dst=0, a=0), dict(op=L, dst=1, a=1), dict(op=MUL, dst=2, a=0, b=1), dict(op=ADD, dst=2, a=2, b=0), dict(op=ST, a=2)]
    dx, dy, dz = to_dev(x), to_dev(y), dev_zeros(m * n, 2)
    prog = kh.program(insts)
    g = lambda t: dglobal(t, m, n, n, 1, kh.F16)
    kh.elementwise_specialize(prog, [g(dx), g(dy)], g(dz))
    before = kh.elementwise_specialize_stats()[1]
    kh.elementwise(prog, [g(dx), g(dy)], g(dz))
    sync()
    assert kh.elementwise_specialize_stats()[1] == before + 1
    got = to_host(dz, np.uint16, (m, n))
    rows = np.linspace(0, m - 1, 32).astype(int)
    xs, ys = np.ascontiguousarray(x[rows]), np.ascontiguousarray(y[rows])
    want = np.zeros((len(rows), n), np.uint16)
    assert ko.elementwise(ko.program(insts), [ko.mk_global(xs, len(rows), n, n, 1, kh.F16), ko.mk_global(ys, len(rows), n, n, 1, kh.F16)],
                          ko.mk_global(want, len(rows), n, n, 1, kh.F16)) == 0
    assert np.array_equal(got[rows], want)
    xf, yf = x.view(np.float16).astype(np.float64), y.view(np.float16).astype(np.float64)   # products and sums exact in fp64
    whole = ((xf * yf).astype(np.float16).astype(np.float64) + xf).astype(np.float16).view(np.uint16)
    nan = np.isnan(whole.view(np.float16))
    assert np.array_equal(got[~nan], whole[~nan])


# ---------------------------------------------------------------------------------------------------------
# Programs with reduces along the rows: compiled onto the row skeleton (a workgroup keeps the row in registers).
def _check_ulp_away_from_cancellation(got, want, dtype, floor=1e-6):
    """<= 2 ulp, except where gamma*xhat + beta cancels to almost nothing: there a sum taken in another order (1e-7 of the
    addends) is many ulp of the tiny result, so an absolute error below `floor` passes as well."""
    f = (lambda a: a.view(np.float16).astype(np.float64)) if dtype == kh.F16 else \
        (lambda a: (a.astype(np.uint32) << 16).view(np.float32).astype(np.float64))
    g, w = f(got), f(want)
    with np.errstate(invalid="ignore"):       # (inf - inf where both are infinite: not 'close', checked as ulp below)
        far = ~(np.abs(g - w) <= floor)
    _check_ulp(got[far], want[far], dtype)


def _row_both(ko, insts, dtype, m, n, seed, extra=0, std=2.0, col=False):
    x = ko.fill_normal(m * n, dtype, seed, std=std).reshape(m, n)
    rows = [ko.fill_normal(n, dtype, seed + 1 + k, mean=1.0 if k == 0 else 0.0, std=0.5) for k in range(extra)]
    ins, shapes = [x] + rows, [(m, n)] + [(1, n)] * extra
    if col:
        ins.append(ko.fill_uniform(m, dtype, seed + 9, 0, 0.5, 2.0))
        shapes.append((m, 1))
    return _both(ko, insts, ins, [dtype] * len(ins), dtype, m, n, in_shapes=shapes)


@pytest.mark.parametrize("dtype", [kh.F16, kh.BF16])
@pytest.mark.parametrize("m,n", [(7, 64), (5, 1000), (33, 4096), (700, 8192), (4, 12288), (3, 32768)])
def test_compiled_softmax_every_launch_shape(ko, dtype, m, n):
    _, compiled, want = _row_both(ko, kh.softmax_insts(dtype), dtype, m, n, 50 + n % 97)
    _check_ulp(compiled, want, dtype)


@pytest.mark.parametrize("dtype", [kh.F16, kh.BF16])
@pytest.mark.parametrize("m,n", [(12, 1024), (600, 8192), (5, 200), (3, 32768)])
def test_compiled_layernorm_and_rmsnorm(ko, dtype, m, n):
    """gamma and beta are parked in LDS where that fits 48 KiB (not at 32768 columns: read through L2 there)."""
    _, compiled, want = _row_both(ko, kh.layernorm_insts(n, dtype), dtype, m, n, 61, extra=2)
    _check_ulp_away_from_cancellation(compiled, want, dtype)
    _, compiled, want = _row_both(ko, kh.layernorm_insts(n, dtype, affine=False), dtype, m, n, 62)
    _check_ulp(compiled, want, dtype)
    _, compiled, want = _row_both(ko, kh.rmsnorm_insts(n, dtype), dtype, m, n, 63, extra=1)
    _check_ulp(compiled, want, dtype)


def test_compiled_row_program_with_special_values_reused_values_and_a_column_operand(ko):
    m, n = 6, 1024
    x = ko.fill_normal(m * n, kh.F16, 55, std=4.0).reshape(m, n)
    x[1, 3] = 0x7e00                 # a NaN poisons its row
    x[2, 9] = 0x7c00                 # +inf: inf - inf
    x[3, :] = 0xfc00                 # a row of -inf
    x[4, :] = 0x7bff                 # a row of the largest finite value: uniform 1/n
    _, compiled, want = _both(ko, kh.softmax_insts(kh.F16), [x], [kh.F16], kh.F16, m, n)
    _check_ulp(compiled, want, kh.F16)
    assert np.all(np.isnan(compiled[[1, 2, 3]].view(np.float16))) and np.all(compiled[4] == np.float16(1.0 / n).view(np.uint16))
    # (e / sum(e)) * e * col with e = exp(x): e is used three times, the per-row sum divides a row value, a [m x 1] operand scales rows
    insts = [dict(op=L, dst=0, a=0), dict(op=CAST, dst=1, a=0, dtype=kh.F32), dict(op=kh.EW_EXP, dst=1, a=1), dict(op=kh.EW_REDUCE_SUM, dst=2, a=1, b=1),
             dict(op=DIV, dst=3, a=1, b=2), dict(op=MUL, dst=3, a=3, b=1), dict(op=L, dst=5, a=1), dict(op=CAST, dst=5, a=5, dtype=kh.F32),
             dict(op=MUL, dst=3, a=3, b=5), dict(op=CAST, dst=4, a=3, dtype=kh.F16, rmode=kh.RN), dict(op=ST, a=4)]
    _, compiled, want = _row_both(ko, insts, kh.F16, 10, 2048, 71, std=1.0, col=True)
    _check_ulp(compiled, want, kh.F16)
    # the row maximum broadcast back (the stored value is a per-row value), and the sum of a per-row value (n times the maximum)
    prog = [dict(op=L, dst=0, a=0), dict(op=kh.EW_REDUCE_MAX, dst=1, a=0, b=1), dict(op=ST, a=1)]
    xs = ko.fill_normal(4 * 512, kh.F16, 72).reshape(4, 512)
    xs[1, 100], xs[2, 7] = 0x7e00, 0x7c00
    _, compiled, want = _both(ko, prog, [xs], [kh.F16], kh.F16, 4, 512)
    assert np.array_equal(compiled[[0, 2, 3]], want[[0, 2, 3]]) and np.all(np.isnan(compiled[1].view(np.float16)))
    prog = [dict(op=L, dst=0, a=0), dict(op=CAST, dst=0, a=0, dtype=kh.F32), dict(op=kh.EW_REDUCE_MAX, dst=1, a=0, b=1),
            dict(op=kh.EW_REDUCE_SUM, dst=2, a=1, b=1), dict(op=SUB, dst=0, a=0, b=2), dict(op=CAST, dst=3, a=0, dtype=kh.F16, rmode=kh.RN), dict(op=ST, a=3)]
    _, compiled, want = _both(ko, prog, [ko.fill_normal(8 * 256, kh.F16, 73).reshape(8, 256)], [kh.F16], kh.F16, 8, 256)
    _check_ulp(compiled, want, kh.F16)


def test_compiled_softmax_f32_in_and_out(ko):
    m, n = 8, 2048
    x = ko.fill_normal(m * n, kh.F32, 81, std=2.0).reshape(m, n)
    insts = [dict(op=L, dst=0, a=0), dict(op=kh.EW_REDUCE_MAX, dst=1, a=0, b=1), dict(op=SUB, dst=0, a=0, b=1),
             dict(op=kh.EW_EXP, dst=0, a=0), dict(op=kh.EW_REDUCE_SUM, dst=1, a=0, b=1), dict(op=DIV, dst=0, a=0, b=1), dict(op=ST, a=0)]
    _, compiled, want = _both(ko, insts, [x], [kh.F32], kh.F32, m, n)
    g, w = compiled.view(np.float32).astype(np.float64), want.view(np.float32).astype(np.float64)
    assert np.max(np.abs(g - w) / w) <= 4e-6        # fp32 exp (2 ulp) and a sum in another order
    assert np.allclose(g.sum(axis=1), 1.0, atol=1e-5)


def test_a_row_kernel_serves_only_its_own_width_class(ko):
    """Compiled for rows of 8192 elements (256 lanes x 4 vectors); rows of 1280 (64 lanes x 3 vectors, a shape no other
    test compiles softmax for) run the hand-written kernel until they get a compiled one of their own."""
    insts = kh.softmax_insts(kh.F16)
    _row_both(ko, insts, kh.F16, 16, 8192, 90)
    before = kh.elementwise_specialize_stats()
    m, n = 16, 1280
    x = ko.fill_normal(m * n, kh.F16, 91).reshape(m, n)
    want = np.zeros((m, n), np.uint16)
    assert ko.elementwise(ko.program(insts), [ko.mk_global(x, m, n, n, 1, kh.F16)], ko.mk_global(want, m, n, n, 1, kh.F16)) == 0
    dx, dout = to_dev(x), dev_zeros(m * n, 2)
    kh.elementwise(kh.program(insts), [dglobal(dx, m, n, n, 1, kh.F16)], dglobal(dout, m, n, n, 1, kh.F16))
    sync()
    assert kh.elementwise_specialize_stats() == before
    _check_ulp(to_host(dout, np.uint16, (m, n)), want, kh.F16)


def test_a_row_program_the_row_machine_refuses_is_compiled_on_its_first_call(ko):
    """Softmax over 100 columns of rows that lie 104 elements apart: the row machine wants a multiple of 8, so
    kapy_elementwise compiles a kernel for it instead of refusing (one more kernel loaded, the call ran it)."""
    m, width, pitch, dt = 9, 100, 104, kh.F16
    insts = kh.softmax_insts(dt)[:-2] + [dict(op=kh.EW_ABSF, dst=1, a=1)] + kh.softmax_insts(dt)[-2:]   # |softmax|: no other test's program
    x = ko.fill_normal(m * pitch, dt, 77, 0, 0.0, 2.0)
    want = np.full(m * pitch, 0x5a5a, np.uint16)
    assert ko.elementwise(ko.program(insts), [ko.mk_global(x, m, width, pitch, 1, dt)], ko.mk_global(want, m, width, pitch, 1, dt)) == 0
    dx, dout = to_dev(x), to_dev(np.full(m * pitch, 0x5a5a, np.uint16))
    loaded, launches = kh.elementwise_specialize_stats()
    kh.elementwise(kh.program(insts), [dglobal(dx, m, width, pitch, 1, dt)], dglobal(dout, m, width, pitch, 1, dt))
    sync()
    assert kh.elementwise_specialize_stats() == (loaded + 1, launches + 1)
    got, want = to_host(dout, np.uint16, (m, pitch)), want.reshape(m, pitch)
    assert np.array_equal(got[:, width:], want[:, width:])
    _check_ulp(np.ascontiguousarray(got[:, :width]), np.ascontiguousarray(want[:, :width]), dt)


def test_threads_specialising_the_same_program_load_one_kernel(ko):
    import threading
    m, n = 8, 64
    insts = [dict(op=L, dst=0, a=0), dict(op=kh.EW_SQRT, dst=1, a=0), dict(op=MUL, dst=1, a=1, b=0), dict(op=kh.EW_ABSF, dst=1, a=1), dict(op=ST, a=1)]
    x = to_dev(ko.fill_uniform(m * n, kh.F16, 88, 0, 0.5, 4.0))
    out = dev_zeros(m * n, 2)
    prog = kh.program(insts)
    loaded = kh.elementwise_specialize_stats()[0]
    errors = []
    def work():
        try:
            kh.elementwise_specialize(prog, [dglobal(x, m, n, n, 1, kh.F16)], dglobal(out, m, n, n, 1, kh.F16))
        except Exception as e:   # noqa: BLE001 - reported below
            errors.append(e)
    threads = [threading.Thread(target=work) for _ in range(4)]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    assert not errors, errors
    assert kh.elementwise_specialize_stats()[0] == loaded + 1


# ---------------------------------------------------------------------------------------------------------
# Column-major operands and results: the tiled skeleton (a load or store with swapped strides fused with the elementwise ops).
def _strided_case(ko, insts, specs, out_spec, m, n):
    """specs: per operand (dtype, kind) with kind in full / T (column-major) / row / col; out_spec: (dtype, 'full' | 'T')."""
    def layout(kind):   # (rows, cols, stride0, stride1, elements)
        return {"full": (m, n, n, 1, m * n), "T": (m, n, 1, m, m * n), "row": (1, n, n, 1, n), "col": (m, 1, 1, 1, m)}[kind]
    arrays, o_ins, d_ins, keep = [], [], [], []
    for k, (dt, kind) in enumerate(specs):
        r, c, s0, s1, count = layout(kind)
        a = ko.fill_uniform(count, dt, 101, k, 0.5, 2.0) if dt in (kh.F8E4M3, kh.F8E5M2) else ko.fill_normal(count, dt, 101, k)
        t = to_dev(a)
        arrays.append(a)      # the oracle's descriptor points into it
        keep.append(t)
        o_ins.append(ko.mk_global(a, r, c, s0, s1, dt))
        d_ins.append(dglobal(t, r, c, s0, s1, dt))
    out_dt, out_kind = out_spec
    r, c, s0, s1, count = layout(out_kind)
    outb = kh.DTYPE_BYTES[out_dt]
    want = np.zeros(count, dtype=NP_OF[outb])
    assert ko.elementwise(ko.program(insts), o_ins, ko.mk_global(want, r, c, s0, s1, out_dt)) == 0
    prog = kh.program(insts)
    dout = dev_zeros(count, outb)
    kh.elementwise_specialize(prog, d_ins, dglobal(dout, r, c, s0, s1, out_dt))
    before = kh.elementwise_specialize_stats()[1]
    kh.elementwise(prog, d_ins, dglobal(dout, r, c, s0, s1, out_dt))
    sync()
    assert kh.elementwise_specialize_stats()[1] == before + 1
    return to_host(dout, NP_OF[outb]), want


@pytest.mark.parametrize("m,n", [(64, 64), (128, 256), (72, 200), (8, 8), (1000, 520)])
def test_column_major_operands_are_staged_through_lds(ko, m, n):
    # z = x^T-view * y + bias_row, all f16, exactly rounded: bit-exact
    insts = [dict(op=L, dst=0, a=0), dict(op=L, dst=1, a=1), dict(op=L, dst=2, a=2), dict(op=MUL, dst=3, a=0, b=1), dict(op=ADD, dst=3, a=3, b=2), dict(op=ST, a=3)]
    got, want = _strided_case(ko, insts, [(kh.F16, "T"), (kh.F16, "full"), (kh.F16, "row")], (kh.F16, "full"), m, n)
    assert np.array_equal(got, want)
    # two column-major operands of different element sizes and a column operand, f32 arithmetic, bf16 result
    insts = [dict(op=L, dst=0, a=0), dict(op=CAST, dst=0, a=0, dtype=kh.F32), dict(op=L, dst=1, a=1), dict(op=L, dst=2, a=2), dict(op=CAST, dst=2, a=2, dtype=kh.F32),
             dict(op=FMA, dst=3, a=0, b=1, c=2), dict(op=CAST, dst=4, a=3, dtype=kh.BF16, rmode=kh.RN), dict(op=ST, a=4)]
    got, want = _strided_case(ko, insts, [(kh.BF16, "T"), (kh.F32, "T"), (kh.BF16, "col")], (kh.BF16, "full"), m, n)
    assert np.array_equal(got, want)


@pytest.mark.parametrize("m,n", [(64, 128), (200, 80), (512, 1008)])   # (the fp8 operand is read 16 elements at a time along n)
def test_column_major_result_is_the_transposed_problem(ko, m, n):
    # the transpose fused with GELU: out (column-major) = gelu(x*0.5 + bias_row) of a row-major x
    insts = [dict(op=L, dst=0, a=0), dict(op=CAST, dst=0, a=0, dtype=kh.F32), dict(op=SPL, dst=1, dtype=kh.F32, imm=0.5), dict(op=MUL, dst=0, a=0, b=1),
             dict(op=L, dst=2, a=1), dict(op=CAST, dst=2, a=2, dtype=kh.F32), dict(op=ADD, dst=0, a=0, b=2), dict(op=kh.EW_GELU_TANH, dst=0, a=0),
             dict(op=CAST, dst=3, a=0, dtype=kh.F16, rmode=kh.RN), dict(op=ST, a=3)]
    got, want = _strided_case(ko, insts, [(kh.F16, "full"), (kh.F16, "row")], (kh.F16, "T"), m, n)
    _check_ulp(got.reshape(n, m), want.reshape(n, m), kh.F16)
    # dequantise-and-transpose: e4m3 row-major in, bf16 column-major out, scaled per original row
    insts = [dict(op=L, dst=0, a=0), dict(op=CAST, dst=0, a=0, dtype=kh.F32), dict(op=L, dst=1, a=1), dict(op=MUL, dst=0, a=0, b=1),
             dict(op=CAST, dst=2, a=0, dtype=kh.BF16, rmode=kh.RN), dict(op=ST, a=2)]
    got, want = _strided_case(ko, insts, [(kh.F8E4M3, "full"), (kh.F32, "col")], (kh.BF16, "T"), m, n)
    assert np.array_equal(got, want)


def test_auto_specialize_switch_compiles_on_the_first_call(ko):
    """KAPY_EW_AUTO_SPECIALIZE=1 (read once per process, so tried in a process of its own): a program outside the hand-written
    kernels is compiled by its first kapy_elementwise call; the result equals the oracle's."""
    import os
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    code = r'''
import sys
sys.path[:0] = [%r, %r, %r]
import numpy as np, torch, kapy_hip as kh, ko
from gpu_util import dev_zeros, dglobal, sync, to_dev, to_host
m, n = 16, 256
a, b = ko.fill_normal(m * n, kh.F16, 5, 0).reshape(m, n), ko.fill_normal(m * n, kh.F16, 5, 1).reshape(m, n)
L, ADD, MUL, ST = kh.EW_LD_GLOBAL, kh.EW_ADDF, kh.EW_MULF, kh.EW_ST_GLOBAL
insts = [dict(op=L, dst=0, a=0), dict(op=L, dst=1, a=1), dict(op=MUL, dst=2, a=0, b=1), dict(op=ADD, dst=2, a=2, b=0), dict(op=ST, a=2)]
want = np.zeros((m, n), np.uint16)
assert ko.elementwise(ko.program(insts), [ko.mk_global(a, m, n, n, 1, kh.F16), ko.mk_global(b, m, n, n, 1, kh.F16)], ko.mk_global(want, m, n, n, 1, kh.F16)) == 0
da, db, dz = to_dev(a), to_dev(b), dev_zeros(m * n, 2)
g = lambda t: dglobal(t, m, n, n, 1, kh.F16)
for call in range(2):
    kh.elementwise(kh.program(insts), [g(da), g(db)], g(dz)); sync()
    assert kh.elementwise_specialize_stats() == (1, call + 1), kh.elementwise_specialize_stats()
assert np.array_equal(to_host(dz, np.uint16, (m, n)), want)
kh.elementwise(kh.gelu_program(kh.F16), [g(da), dglobal(db, 1, n, n, 1, kh.F16)], g(dz)); sync()     # a matched program stays on its kernel
assert kh.elementwise_specialize_stats() == (1, 2)
print("auto ok")
''' % (os.path.join(root, "kapy-lang_amd", "python"), os.path.join(root, "oracle"), os.path.join(root, "tests"))
    env = dict(os.environ, KAPY_EW_AUTO_SPECIALIZE="1")
    out = subprocess.run([sys.executable, "-c", code], env=env, capture_output=True, text=True, timeout=110)
    assert out.returncode == 0 and "auto ok" in out.stdout, out.stdout + out.stderr



def test_by_default_a_program_is_compiled_when_it_comes_back(ko):
    """Without the switch (in a process of its own, where nothing was compiled before): the first call of a program outside the
    hand-written kernels runs on the stepwise machines, the second compiles it, later ones launch the compiled kernel; another
    operand signature of the same program starts counting again; a captured call never compiles; results equal the oracle's
    whichever path served the call.  KAPY_EW_AUTO_SPECIALIZE=0: never."""
    import os
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    code = r'''
import os, sys
sys.path[:0] = [%r, %r, %r]
import numpy as np, torch, kapy_hip as kh, ko
from gpu_util import dev_zeros, dglobal, sync, to_dev, to_host
never = os.environ.get("KAPY_EW_AUTO_SPECIALIZE") == "0"
m, n = 64, 512
a, b = ko.fill_normal(m * n, kh.F16, 5, 0).reshape(m, n), ko.fill_normal(m * n, kh.F16, 5, 1).reshape(m, n)
L, ADD, MUL, ST = kh.EW_LD_GLOBAL, kh.EW_ADDF, kh.EW_MULF, kh.EW_ST_GLOBAL
insts = [dict(op=L, dst=0, a=0), dict(op=L, dst=1, a=1), dict(op=MUL, dst=2, a=0, b=1), dict(op=ADD, dst=2, a=2, b=0), dict(op=ST, a=2)]
want = np.zeros((m, n), np.uint16)
assert ko.elementwise(ko.program(insts), [ko.mk_global(a, m, n, n, 1, kh.F16), ko.mk_global(b, m, n, n, 1, kh.F16)], ko.mk_global(want, m, n, n, 1, kh.F16)) == 0
da, db, dz = to_dev(a), to_dev(b), dev_zeros(m * n, 2)
g = lambda t: dglobal(t, m, n, n, 1, kh.F16)
expect = [(0, 0), (1, 1), (1, 2), (1, 3)]
for call in range(4):
    dz.zero_()
    kh.elementwise(kh.program(insts), [g(da), g(db)], g(dz)); sync()
    assert kh.elementwise_specialize_stats() == ((0, 0) if never else expect[call]), (call, kh.elementwise_specialize_stats())
    assert np.array_equal(to_host(dz, np.uint16, (m, n)), want), call
if not never:
    # the same program with a row operand in place of the second full one: another signature, counted from one again
    grow = dglobal(db, 1, n, n, 1, kh.F16)
    kh.elementwise(kh.program(insts), [g(da), grow], g(dz)); sync()
    assert kh.elementwise_specialize_stats() == (1, 3)
    # under capture nothing is compiled: its second call is recorded on the stepwise machine and replays correctly
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            kh.elementwise(kh.program(insts), [g(da), grow], g(dz), stream=side.cuda_stream)
    assert kh.elementwise_specialize_stats() == (1, 3)
    want_row = np.zeros((m, n), np.uint16)
    assert ko.elementwise(ko.program(insts), [ko.mk_global(a, m, n, n, 1, kh.F16), ko.mk_global(b, 1, n, n, 1, kh.F16)], ko.mk_global(want_row, m, n, n, 1, kh.F16)) == 0
    for rep in range(2):
        dz.zero_(); sync(); graph.replay(); sync()
        assert np.array_equal(to_host(dz, np.uint16, (m, n)), want_row)
print("default ok")
''' % (os.path.join(root, "kapy-lang_amd", "python"), os.path.join(root, "oracle"), os.path.join(root, "tests"))
    for value in (None, "0"):
        env = {k: v for k, v in os.environ.items() if k != "KAPY_EW_AUTO_SPECIALIZE"}
        if value is not None:
            env["KAPY_EW_AUTO_SPECIALIZE"] = value
        out = subprocess.run([sys.executable, "-c", code], env=env, capture_output=True, text=True, timeout=110)
        assert out.returncode == 0 and "default ok" in out.stdout, out.stdout + out.stderr


def test_full_size_transpose_fused_with_gelu(ko):
    """y = gelu_tanh(x^T*0.5 + bias) on fp16 8192x8192 through the tiled skeleton: the whole result against the two
    hand-written kernels run one after the other (transpose, then the fused GELU; <= 2 ulp: one contracts x*s + b into an
    fma, the other rounds twice), and 32 rows spread over it against the oracle."""
    n = 8192
    x = ko.fill_normal(n * n, kh.F16, 0, 0).reshape(n, n)
    bias = ko.fill_normal(n, kh.F16, 0, 1)
    dx, db, dy, dt_, d2 = to_dev(x), to_dev(bias), dev_zeros(n * n, 2), dev_zeros(n * n, 2), dev_zeros(n * n, 2)
    prog = kh.gelu_program(kh.F16, 0.5)
    gT, g, gb = dglobal(dx, n, n, 1, n, kh.F16), (lambda t: dglobal(t, n, n, n, 1, kh.F16)), dglobal(db, 1, n, n, 1, kh.F16)
    kh.elementwise_specialize(prog, [gT, gb], g(dy))
    before = kh.elementwise_specialize_stats()[1]
    kh.elementwise(prog, [gT, gb], g(dy))
    kh.copy(g(dx), g(dt_), transpose=True)
    kh.elementwise(prog, [g(dt_), gb], g(d2))
    sync()
    assert kh.elementwise_specialize_stats()[1] == before + 1      # only the call with the swapped strides ran compiled code
    got, two_step = to_host(dy, np.uint16, (n, n)), to_host(d2, np.uint16, (n, n))
    assert ulp_diff_f16(got, two_step).max() <= 2
    rows = np.linspace(0, n - 1, 32).astype(int)
    xs = np.ascontiguousarray(x[:, rows].T)                        # rows of the transposed view
    want = np.zeros((len(rows), n), np.uint16)
    assert ko.elementwise(ko.program(_gelu_insts()), [ko.mk_global(xs, len(rows), n, n, 1, kh.F16), ko.mk_global(bias, 1, n, n, 1, kh.F16)],
                          ko.mk_global(want, len(rows), n, n, 1, kh.F16)) == 0
    _check_ulp(got[rows], want, kh.F16)


def _gelu_insts():
    """The chain of kh.gelu_program(F16, 0.5) spelled out (the oracle takes the same instruction list)."""
    return [dict(op=L, dst=0, a=0), dict(op=CAST, dst=1, a=0, dtype=kh.F32), dict(op=SPL, dst=2, dtype=kh.F32, imm=0.5), dict(op=MUL, dst=1, a=1, b=2),
            dict(op=L, dst=4, a=1), dict(op=CAST, dst=4, a=4, dtype=kh.F32), dict(op=ADD, dst=1, a=1, b=4), dict(op=kh.EW_GELU_TANH, dst=1, a=1),
            dict(op=CAST, dst=5, a=1, dtype=kh.F16, rmode=kh.RN), dict(op=ST, a=5)]


def test_a_damaged_cached_code_object_is_replaced(ko, tmp_path, monkeypatch):
    """KAPY_EW_CACHE_DIR holds code objects keyed by a hash of their source.  A file there that is not a loadable code object
    (damaged, foreign) must not poison the program for good: the load fails, the file is thrown away and the source is
    compiled again."""
    import os
    monkeypatch.setenv("KAPY_EW_CACHE_DIR", str(tmp_path))
    m, n = 24, 136
    insts = [dict(op=L, dst=0, a=0), dict(op=L, dst=1, a=1), dict(op=SUB, dst=2, a=0, b=1), dict(op=MIN, dst=2, a=2, b=1),
             dict(op=kh.EW_ABSF, dst=2, a=2), dict(op=ST, a=2)]
    a, b = ko.fill_normal(m * n, kh.F16, 91, 0).reshape(m, n), ko.fill_normal(m * n, kh.F16, 91, 1).reshape(m, n)
    want = np.zeros((m, n), np.uint16)
    og = lambda x: ko.mk_global(x, m, n, n, 1, kh.F16)
    assert ko.elementwise(ko.program(insts), [og(a), og(b)], og(want)) == 0
    da, db, dz = to_dev(a), to_dev(b), dev_zeros(m * n, 2)
    g = lambda t: dglobal(t, m, n, n, 1, kh.F16)
    prog = kh.program(insts)
    _, size = kh.elementwise_source(prog, [g(da), g(db)], g(dz), compile=True)          # compiles and fills the cache
    files = os.listdir(tmp_path)
    assert len(files) == 1 and os.path.getsize(tmp_path / files[0]) == size
    with open(tmp_path / files[0], "wb") as f:
        f.write(b"not a code object " * 64)
    loaded_before, _ = kh.elementwise_specialize_stats()
    kh.elementwise_specialize(prog, [g(da), g(db)], g(dz))                              # reads the damaged file, recovers
    assert kh.elementwise_specialize_stats()[0] == loaded_before + 1
    assert os.path.getsize(tmp_path / files[0]) == size
    kh.elementwise(prog, [g(da), g(db)], g(dz))
    sync()
    assert np.array_equal(to_host(dz, np.uint16, (m, n)), want)
