"""GPU parity for fused elementwise programs: max |err| <= 2 ulp of the 16-bit result type against
the oracle (the tolerance the benchmark definition states), bit-exact where the op is exactly rounded."""
import ctypes as C

import numpy as np
import pytest

import kapy_hip as kh
from gpu_util import dev_zeros, dglobal, sync, to_dev, to_host, ulp_diff_f16

pytestmark = pytest.mark.gpu
ULP_TOL = 2


def _check_ulp(got, want, dtype):
    f = (lambda a: a.view(np.float16).astype(np.float64)) if dtype == kh.F16 else \
        (lambda a: (a.astype(np.uint32) << 16).view(np.float32).astype(np.float64))
    gn, wn = np.isnan(f(got)), np.isnan(f(want))
    bad = np.argwhere(gn != wn)
    assert len(bad) == 0, "NaN pattern differs at %s: got %s want %s" % (bad[:8].tolist(), [hex(int(got[tuple(b)])) for b in bad[:8]],
                                                                       [hex(int(want[tuple(b)])) for b in bad[:8]])
    d = ulp_diff_f16(got[~gn], want[~wn])
    assert d.max(initial=0) <= ULP_TOL, "max ulp error %d" % d.max()
    return d


def _gelu_case(ko, dtype, m, n, seed, specials=False):
    x = ko.fill_normal(m * n, dtype, seed, 0).reshape(m, n)
    bias = ko.fill_normal(n, dtype, seed + 1, 0)
    if specials:
        enc = (lambda v: np.array(v, dtype=np.float16).view(np.uint16)) if dtype == kh.F16 else \
            (lambda v: (np.array(v, dtype=np.float32).view(np.uint32) >> 16).astype(np.uint16))
        sp = enc([0.0, -0.0, np.inf, -np.inf, np.nan, 60000.0, -60000.0, 1e-7, -8.0, 8.0, -3.0, 3.0])
        x.ravel()[:len(sp)] = sp
        bias[:len(sp)] = 0
    want = np.zeros((m, n), dtype=np.uint16)
    go = ko.mk_global(want, m, n, n, 1, dtype)
    assert ko.elementwise(ko.gelu_program(dtype, dtype), [ko.mk_global(x, m, n, n, 1, dtype), ko.mk_global(bias, 1, n, n, 1, dtype)], go) == 0
    dx, db, dy = to_dev(x), to_dev(bias), dev_zeros(m * n, 2)
    kh.elementwise(kh.gelu_program(dtype), [dglobal(dx, m, n, n, 1, dtype), dglobal(db, 1, n, n, 1, dtype)], dglobal(dy, m, n, n, 1, dtype))
    sync()
    return to_host(dy, np.uint16, (m, n)), want


@pytest.mark.parametrize("dtype", [kh.F16, kh.BF16])
@pytest.mark.parametrize("m,n", [(64, 256), (33, 1000), (7, 24)])
def test_gelu_bias_scale_fused(ko, dtype, m, n):
    got, want = _gelu_case(ko, dtype, m, n, 0, specials=True)
    _check_ulp(got, want, dtype)


def test_gelu_unaligned_shape_takes_the_interpreter(ko):
    got, want = _gelu_case(ko, kh.F16, 19, 37, 5)   # 37 % 8 != 0: not the vector path
    _check_ulp(got, want, kh.F16)


def test_config2_gelu_8192_sampled_against_oracle(ko):
    """benchmark configuration 2: y = GELU_tanh(x*0.5 + bias), x fp16 8192x8192 normal(0,1) seed 0, bias seed 1.
    The whole result is produced on the GPU; the oracle checks 64 full rows spread over the matrix, and
    a row-broadcast invariant (rows with equal x rows give equal y rows) covers the rest."""
    n = 8192
    x = ko.fill_normal(n * n, ko.F16, 0, 0).reshape(n, n)
    bias = ko.fill_normal(n, ko.F16, 1, 0)
    x[5000] = x[17]                                    # planted duplicate row
    dx, db, dy = to_dev(x), to_dev(bias), dev_zeros(n * n, 2)
    kh.elementwise(kh.gelu_program(kh.F16), [dglobal(dx, n, n, n, 1, kh.F16), dglobal(db, 1, n, n, 1, kh.F16)],
                   dglobal(dy, n, n, n, 1, kh.F16))
    sync()
    got = to_host(dy, np.uint16, (n, n))
    rows = np.unique(np.concatenate([np.arange(0, n, 131), [n - 1, 17, 5000]]))
    xs = np.ascontiguousarray(x[rows])
    want = np.zeros_like(xs)
    m = len(rows)
    assert ko.elementwise(ko.gelu_program(), [ko.mk_global(xs, m, n, n, 1, ko.F16), ko.mk_global(bias, 1, n, n, 1, ko.F16)],
                          ko.mk_global(want, m, n, n, 1, ko.F16)) == 0
    d = _check_ulp(got[rows], want, kh.F16)
    assert (d > 0).mean() < 0.02                       # almost every element is bit-identical
    assert np.array_equal(got[5000], got[17])
    assert not np.any(np.isnan(got.view(np.float16)))


def _run_prog(ko, insts, ins_np, in_dtypes, out_dtype, m, n, in_shapes=None):
    outb = kh.DTYPE_BYTES[out_dtype]
    np_out = {1: np.uint8, 2: np.uint16, 4: np.uint32}[outb]
    want = np.zeros((m, n), dtype=np_out)
    in_shapes = in_shapes or [(m, n)] * len(ins_np)
    gos = [ko.mk_global(a, s[0], s[1], s[1], 1, dt) for a, s, dt in zip(ins_np, in_shapes, in_dtypes)]
    assert ko.elementwise(ko.program(insts), gos, ko.mk_global(want, m, n, n, 1, out_dtype)) == 0
    devs = [to_dev(a) for a in ins_np]
    dout = dev_zeros(m * n, outb)
    kh.elementwise(kh.program(insts), [dglobal(t, s[0], s[1], s[1], 1, dt) for t, s, dt in zip(devs, in_shapes, in_dtypes)],
                   dglobal(dout, m, n, n, 1, out_dtype))
    sync()
    return to_host(dout, np_out, (m, n)), want


def test_bf16_and_f16_arithmetic_is_exactly_rounded(ko):
    m, n = 32, 96
    for dt in (kh.BF16, kh.F16):
        a = ko.fill_normal(m * n, dt, 2, 0).reshape(m, n)
        b = ko.fill_normal(m * n, dt, 2, 1).reshape(m, n)
        insts = [dict(op=kh.EW_LD_GLOBAL, dst=0, a=0), dict(op=kh.EW_LD_GLOBAL, dst=1, a=1),
                 dict(op=kh.EW_MULF, dst=2, a=0, b=1), dict(op=kh.EW_ADDF, dst=2, a=2, b=0),
                 dict(op=kh.EW_SUBF, dst=3, a=2, b=1), dict(op=kh.EW_MAXIMUMF, dst=3, a=3, b=0),
                 dict(op=kh.EW_FMA, dst=3, a=3, b=1, c=0), dict(op=kh.EW_ST_GLOBAL, a=3)]
        got, want = _run_prog(ko, insts, [a, b], [dt, dt], dt, m, n)
        assert np.array_equal(got, want)       # +,-,*,max,fma: one rounding each, bit-exact


def test_explicit_tanh_chain_equals_the_fused_gelu_within_tolerance(ko):
    """GELU written out in kapy ops (mulf/addf/fma/tanh) against the oracle of the same chain."""
    m, n = 16, 256
    x = ko.fill_normal(m * n, kh.F16, 9, 0).reshape(m, n)
    c = lambda r, v: dict(op=kh.EW_SPLAT, dst=r, dtype=kh.F32, imm=v)
    insts = [dict(op=kh.EW_LD_GLOBAL, dst=0, a=0), dict(op=kh.EW_FPTOFP, dst=1, a=0, dtype=kh.F32),
             dict(op=kh.EW_MULF, dst=2, a=1, b=1), dict(op=kh.EW_MULF, dst=2, a=2, b=1),     # v^3
             c(3, 0.044715), dict(op=kh.EW_FMA, dst=2, a=2, b=3, c=1),                       # v + 0.044715 v^3
             c(3, 0.7978845608028654), dict(op=kh.EW_MULF, dst=2, a=2, b=3),
             dict(op=kh.EW_TANH, dst=2, a=2), c(3, 1.0), dict(op=kh.EW_ADDF, dst=2, a=2, b=3),
             c(3, 0.5), dict(op=kh.EW_MULF, dst=4, a=1, b=3), dict(op=kh.EW_MULF, dst=2, a=2, b=4),
             dict(op=kh.EW_FPTOFP, dst=5, a=2, dtype=kh.F16, rmode=kh.RN), dict(op=kh.EW_ST_GLOBAL, a=5)]
    got, want = _run_prog(ko, insts, [x], [kh.F16], kh.F16, m, n)
    _check_ulp(got, want, kh.F16)


@pytest.mark.parametrize("op", [kh.EW_EXP, kh.EW_EXP2, kh.EW_LOG, kh.EW_LOG2, kh.EW_SQRT, kh.EW_RSQRT, kh.EW_TANH,
                                kh.EW_ERF, kh.EW_ABSF, kh.EW_NEGF, kh.EW_GELU_TANH])
def test_unary_math_ops_within_2_ulp_of_16bit_result(ko, op):
    m, n = 8, 512
    x = ko.fill_uniform(m * n, kh.F16, 4, 0, 0.01 if op in (kh.EW_LOG, kh.EW_LOG2, kh.EW_SQRT, kh.EW_RSQRT) else -6.0, 6.0).reshape(m, n)
    insts = [dict(op=kh.EW_LD_GLOBAL, dst=0, a=0), dict(op=kh.EW_FPTOFP, dst=1, a=0, dtype=kh.F32),
             dict(op=op, dst=1, a=1), dict(op=kh.EW_FPTOFP, dst=2, a=1, dtype=kh.F16, rmode=kh.RN),
             dict(op=kh.EW_ST_GLOBAL, a=2)]
    got, want = _run_prog(ko, insts, [x], [kh.F16], kh.F16, m, n)
    _check_ulp(got, want, kh.F16)


@pytest.mark.parametrize("src,dst,rmode", [(kh.F32, kh.F16, kh.RN), (kh.F32, kh.F16, kh.RZ), (kh.F32, kh.BF16, kh.RN),
                                           (kh.F32, kh.BF16, kh.RZ), (kh.F32, kh.F8E4M3, kh.RN), (kh.F32, kh.F8E5M2, kh.RN),
                                           (kh.F16, kh.F8E4M3, kh.RN), (kh.F16, kh.F8E5M2, kh.RZ), (kh.BF16, kh.F8E4M3, kh.RN),
                                           (kh.F8E4M3, kh.F16, kh.RN), (kh.F8E5M2, kh.BF16, kh.RN), (kh.F8E4M3, kh.F32, kh.RN),
                                           (kh.F16, kh.F32, kh.RN), (kh.BF16, kh.F32, kh.RN)])
def test_fptofp_bit_exact(ko, src, dst, rmode):
    """kapy.fptofp over whole tensors: every cast is an exactly-rounded op, so results are bit-exact."""
    m, n = 64, 1024
    sb, db = kh.DTYPE_BYTES[src], kh.DTYPE_BYTES[dst]
    if sb == 1:
        x = (np.arange(m * n) % 256).astype(np.uint8)
    elif sb == 2:
        x = np.arange(m * n, dtype=np.uint32).astype(np.uint16)            # every 16-bit pattern
    else:
        rng = np.random.default_rng(0)
        x = np.concatenate([rng.normal(0, 1, m * n // 2), rng.normal(0, 300, m * n // 4),
                            rng.normal(0, 1e-3, m * n // 4)]).astype(np.float32)
        x[:8] = [0, -0.0, np.inf, -np.inf, np.nan, 448.0, 464.0, 57344.0]
        h = np.arange(0, 0x7F, dtype=np.uint8)                             # e4m3 midpoints: ties
        v = np.array([ko.lib().ko_e4m3_to_f64(int(b)) for b in h])
        x[8:8 + len(v) - 1] = ((v[:-1] + v[1:]) / 2).astype(np.float32)
    want = ko.fptofp(x, src, dst, rmode)
    dx, dy = to_dev(x), dev_zeros(m * n, db)
    kh.fptofp(dglobal(dx, m, n, n, 1, src), dglobal(dy, m, n, n, 1, dst), rmode)
    sync()
    got = to_host(dy, want.dtype)
    if dst in (kh.F16, kh.BF16, kh.F32) and src != kh.F32:
        pass
    wf, gf = ko.decode(want, dst), ko.decode(got.view(want.dtype), dst)
    nan = np.isnan(wf)
    assert np.array_equal(np.isnan(gf), nan)
    assert np.array_equal(got.view(want.dtype)[~nan], want[~nan])


def test_broadcast_column_vector_and_padding(ko):
    m, n = 48, 64
    x = ko.fill_normal(m * n, kh.F16, 1, 0).reshape(m, n)
    col = ko.fill_normal(m, kh.F16, 1, 1)
    insts = [dict(op=kh.EW_LD_GLOBAL, dst=0, a=0), dict(op=kh.EW_LD_GLOBAL, dst=1, a=1),
             dict(op=kh.EW_ADDF, dst=2, a=0, b=1), dict(op=kh.EW_ST_GLOBAL, a=2)]
    got, want = _run_prog(ko, insts, [x, col], [kh.F16, kh.F16], kh.F16, m, n, in_shapes=[(m, n), (m, 1)])
    assert np.array_equal(got, want)
    # column-broadcast bias through the fused path
    prog = [dict(op=kh.EW_LD_GLOBAL, dst=0, a=0), dict(op=kh.EW_LD_GLOBAL, dst=1, a=1),
            dict(op=kh.EW_FPTOFP, dst=2, a=0, dtype=kh.F32), dict(op=kh.EW_FPTOFP, dst=3, a=1, dtype=kh.F32),
            dict(op=kh.EW_ADDF, dst=2, a=2, b=3), dict(op=kh.EW_EXP, dst=2, a=2),
            dict(op=kh.EW_FPTOFP, dst=4, a=2, dtype=kh.F16, rmode=kh.RN), dict(op=kh.EW_ST_GLOBAL, a=4)]
    got, want = _run_prog(ko, prog, [x, col], [kh.F16, kh.F16], kh.F16, m, n, in_shapes=[(m, n), (m, 1)])
    _check_ulp(got, want, kh.F16)


def test_register_stack_kernel_tree_shapes_and_operand_kinds(ko):
    """Programs that are not the act(x*s+bias) chain run on the in-register stack machine when every operand can be
    read 8 elements at a time: reversed subtraction / division (deeper operand on the right), a depth-3 tree, an fma
    of three subtrees, row / column / scalar operands, f32 and fp8 operands and results; exactly rounded ops must be
    bit-exact against the oracle, the same programs at a width that is not a multiple of 8 take the interpreter."""
    L, ADD, SUB, MUL, DIV, FMA, MAX, ST, CAST, SPL = (kh.EW_LD_GLOBAL, kh.EW_ADDF, kh.EW_SUBF, kh.EW_MULF, kh.EW_DIVF, kh.EW_FMA,
                                                      kh.EW_MAXIMUMF, kh.EW_ST_GLOBAL, kh.EW_FPTOFP, kh.EW_SPLAT)
    for (m, n) in ((16, 256), (16, 252)):
        a = ko.fill_normal(m * n, kh.F16, 21, 0).reshape(m, n)
        b = ko.fill_uniform(m * n, kh.F16, 21, 1, 0.5, 2.0).reshape(m, n)
        row = ko.fill_normal(n, kh.F16, 21, 2)
        col = ko.fill_normal(m, kh.F16, 21, 3)
        one = ko.fill_normal(1, kh.F16, 21, 4)
        # (a - (b*row)) / ((a + col) max (b - one)), all in f16: reversed sub and div, depth 3, every operand kind
        insts = [dict(op=L, dst=0, a=0), dict(op=L, dst=1, a=1), dict(op=L, dst=2, a=2), dict(op=L, dst=3, a=3), dict(op=L, dst=4, a=4),
                 dict(op=MUL, dst=5, a=1, b=2), dict(op=SUB, dst=5, a=0, b=5), dict(op=ADD, dst=6, a=0, b=3), dict(op=SUB, dst=7, a=1, b=4),
                 dict(op=MAX, dst=6, a=6, b=7), dict(op=DIV, dst=5, a=5, b=6), dict(op=ST, a=5)]
        got, want = _run_prog(ko, insts, [a, b, row, col, one], [kh.F16] * 5, kh.F16, m, n, [(m, n), (m, n), (1, n), (m, 1), (1, 1)])
        _check_ulp(got, want, kh.F16)     # division is within 2 ulp of f32 (div.full), the rest exact
        # fma(a*b, b - a, a + b) in f32 from f16 operands, f32 result
        insts = [dict(op=L, dst=0, a=0), dict(op=L, dst=1, a=1), dict(op=CAST, dst=2, a=0, dtype=kh.F32), dict(op=CAST, dst=3, a=1, dtype=kh.F32),
                 dict(op=MUL, dst=4, a=2, b=3), dict(op=SUB, dst=5, a=3, b=2), dict(op=ADD, dst=6, a=2, b=3), dict(op=FMA, dst=7, a=4, b=5, c=6),
                 dict(op=ST, a=7)]
        got, want = _run_prog(ko, insts, [a, b], [kh.F16] * 2, kh.F32, m, n)
        assert np.array_equal(got, want)
        # quantise: f32 operand scaled by a splat, rounded to e4m3; and back: e4m3 operand widened to bf16
        x32 = ko.fill_normal(m * n, kh.F32, 22, 0).reshape(m, n)
        insts = [dict(op=L, dst=0, a=0), dict(op=SPL, dst=1, dtype=kh.F32, imm=37.5), dict(op=MUL, dst=0, a=0, b=1),
                 dict(op=CAST, dst=2, a=0, dtype=kh.F8E4M3, rmode=kh.RN), dict(op=ST, a=2)]
        q, wantq = _run_prog(ko, insts, [x32], [kh.F32], kh.F8E4M3, m, n)
        assert np.array_equal(q, wantq)
        insts = [dict(op=L, dst=0, a=0), dict(op=CAST, dst=1, a=0, dtype=kh.BF16), dict(op=ST, a=1)]
        got, want = _run_prog(ko, insts, [wantq], [kh.F8E4M3], kh.BF16, m, n)
        assert np.array_equal(got, want)


@pytest.mark.parametrize("width", [8, 9, 15, 1001, 2046])
@pytest.mark.parametrize("which", ["gelu row bias", "gelu full bias", "x + y", "x*y + x"])
def test_rows_with_a_ragged_last_vector_keep_the_fast_kernels_and_stay_inside_the_view(ko, width, which):
    """Views whose rows start 16-byte aligned but whose width is not a multiple of 8 (a sub-view of a wider tensor): the
    last vector of every row moves element by element; nothing outside the view is read into the result or written."""
    m, pitch = 37, 2048
    xp = ko.fill_normal(m * pitch, kh.F16, 101).reshape(m, pitch)
    yp = ko.fill_normal(m * pitch, kh.F16, 102).reshape(m, pitch)
    bias = ko.fill_normal(pitch, kh.F16, 103)
    sentinel = 0x1234
    want_p = np.full((m, pitch), sentinel, np.uint16)
    view = lambda lib, a, rows=m: lib.mk_global(a, rows, width, pitch, 1, kh.F16)
    if which.startswith("gelu"):
        insts_k, insts_o = kh.gelu_program(kh.F16, 0.5), ko.gelu_program(kh.F16, kh.F16)
        second_np, second_rows = (bias, 1) if which == "gelu row bias" else (yp, m)
    else:
        body = [dict(op=kh.EW_ADDF, dst=2, a=0, b=1)] if which == "x + y" else [dict(op=kh.EW_MULF, dst=2, a=0, b=1), dict(op=kh.EW_ADDF, dst=2, a=2, b=0)]
        insts = [dict(op=kh.EW_LD_GLOBAL, dst=0, a=0), dict(op=kh.EW_LD_GLOBAL, dst=1, a=1)] + body + [dict(op=kh.EW_ST_GLOBAL, a=2)]
        insts_k, insts_o = kh.program(insts), ko.program(insts)
        second_np, second_rows = yp, m
    assert ko.elementwise(insts_o, [view(ko, xp), view(ko, second_np, second_rows)], view(ko, want_p)) == 0
    dx, d2, dout = to_dev(xp), to_dev(second_np), dev_zeros(m * pitch, 2, fill=sentinel)
    dv = lambda t, rows=m: dglobal(t, rows, width, pitch, 1, kh.F16)
    kh.elementwise(insts_k, [dv(dx), dv(d2, second_rows)], dv(dout))
    sync()
    got = to_host(dout, np.uint16, (m, pitch))
    assert np.all(got[:, width:] == sentinel)
    if which.startswith("gelu"):
        _check_ulp(got[:, :width], want_p[:, :width], kh.F16)
    else:
        assert np.array_equal(got[:, :width], want_p[:, :width])


@pytest.mark.parametrize("dtype", [kh.F16, kh.BF16])
@pytest.mark.parametrize("op", ["EW_ADDF", "EW_SUBF", "EW_MULF", "EW_MAXIMUMF", "EW_MINIMUMF"])
def test_plain_binary_programs_are_bit_exact_in_every_operand_shape(ko, dtype, op):
    """z = x op y on the 16-bit type (addf: the reference's elementwise_add fixture) with the second or the first operand
    full, a row or a column: the correctly rounded result of the type, NaN and infinity included."""
    m, n = 24, 256
    full = ko.fill_normal(m * n, dtype, 91, std=30.0).reshape(m, n)
    other = ko.fill_normal(m * n, dtype, 92, std=0.01).reshape(m, n)
    enc = (lambda v: np.array(v, dtype=np.float16).view(np.uint16)) if dtype == kh.F16 else \
        (lambda v: (np.array(v, dtype=np.float32).view(np.uint32) >> 16).astype(np.uint16))
    sp = enc([np.nan, np.inf, -np.inf, 0.0, -0.0, 65504.0, -65504.0, 6e-8])
    full.ravel()[:len(sp)] = sp
    other.ravel()[3:3 + len(sp)] = sp
    for shape in ((m, n), (1, n), (m, 1)):
        y = np.ascontiguousarray(other[:shape[0], :shape[1]])
        for swapped in (False, True):
            insts = [dict(op=kh.EW_LD_GLOBAL, dst=0, a=0), dict(op=kh.EW_LD_GLOBAL, dst=1, a=1),
                     dict(op=getattr(kh, op), dst=2, a=1 if swapped else 0, b=0 if swapped else 1), dict(op=kh.EW_ST_GLOBAL, a=2)]
            got, want = _run_prog(ko, insts, [full, y], [dtype, dtype], dtype, m, n, in_shapes=[(m, n), shape])
            nan = np.isnan(_as_f64(want, dtype))
            assert np.array_equal(np.isnan(_as_f64(got, dtype)), nan)
            assert np.array_equal(got[~nan], want[~nan]), (op, shape, swapped)


def _as_f64(bits, dtype):
    return bits.view(np.float16).astype(np.float64) if dtype == kh.F16 else (bits.astype(np.uint32) << 16).view(np.float32).astype(np.float64)


# ---------------------------------------------------------------------------------------------------------
# Row-wise fusions: programs with a reduce along the rows run with the row resident on chip.
def _row_case(ko, insts, dtype, m, n, seed, extra=(), std=2.0):
    x = ko.fill_normal(m * n, dtype, seed, std=std).reshape(m, n)
    rows = [ko.fill_normal(n, dtype, seed + 1 + k, mean=1.0 if k == 0 else 0.0, std=0.5) for k in range(len(extra))]
    ins = [x] + rows
    shapes = [(m, n)] + [(1, n)] * len(rows)
    return _run_prog(ko, insts, ins, [dtype] * len(ins), dtype, m, n, in_shapes=shapes)


@pytest.fixture(params=["fused kernel", "row machine"])
def row_path(request, monkeypatch):
    """The named row programs have kernels of their own; KAPY_ROW_FUSED=0 sends them through the row machine."""
    if request.param == "row machine":
        monkeypatch.setenv("KAPY_ROW_FUSED", "0")
    return request.param


@pytest.mark.parametrize("dtype", [kh.F16, kh.BF16])
@pytest.mark.parametrize("m,n", [(7, 64), (5, 1000), (33, 4096), (9, 8192), (4, 12288), (3, 32768)])
def test_softmax_rows_every_launch_shape(ko, row_path, dtype, m, n):
    got, want = _row_case(ko, kh.softmax_insts(dtype), dtype, m, n, 50 + n % 97)
    _check_ulp(got, want, dtype)


@pytest.mark.parametrize("dtype", [kh.F16, kh.BF16])
@pytest.mark.parametrize("m,n", [(60000, 64), (50000, 200), (3001, 24), (70, 128), (1000, 256), (9000, 1000), (7000, 4096), (6500, 8192), (6200, 5000)])
def test_softmax_many_rows(ko, dtype, m, n):
    """With many times more rows than workgroups fit on the device, softmax takes one workgroup per row instead of resident
    workgroups that walk the rows, and rows of up to 256 elements share a wave (8, 16 or 32 lanes per row).  The device
    computes every row; the checker a spread sample of them (rows are independent), and the first rows are compared
    against a short launch, which takes the walking kernel (another order of the fp32 sums: within the tolerance)."""
    x = ko.fill_normal(m * n, dtype, 58 + n % 89, std=2.0).reshape(m, n)
    insts = kh.softmax_insts(dtype)
    dout = dev_zeros(m * n, 2)
    kh.elementwise(kh.program(insts), [dglobal(to_dev(x), m, n, n, 1, dtype)], dglobal(dout, m, n, n, 1, dtype))
    sync()
    got = to_host(dout, np.uint16, (m, n))
    rows = np.unique(np.concatenate([np.arange(0, m, max(1, m // 61)), [m - 1, m - 2, 1]]))
    xs = np.ascontiguousarray(x[rows])
    want = np.zeros((len(rows), n), np.uint16)
    assert ko.elementwise(ko.program(insts), [ko.mk_global(xs, len(rows), n, n, 1, dtype)], ko.mk_global(want, len(rows), n, n, 1, dtype)) == 0
    _check_ulp(got[rows], want, dtype)
    few = 40
    dfew = dev_zeros(few * n, 2)
    kh.elementwise(kh.program(insts), [dglobal(to_dev(np.ascontiguousarray(x[:few])), few, n, n, 1, dtype)], dglobal(dfew, few, n, n, 1, dtype))
    sync()
    _check_ulp(to_host(dfew, np.uint16, (few, n)), got[:few], dtype)


@pytest.mark.parametrize("dtype", [kh.F16, kh.BF16])
@pytest.mark.parametrize("m,n", [(40000, 64), (3001, 24), (70, 128), (5000, 200), (1000, 256)])
def test_norms_many_short_rows(ko, dtype, m, n):
    """Layer norm and RMS norm over rows that share a wave, every row against the checker."""
    got, want = _row_case(ko, kh.layernorm_insts(n, dtype), dtype, m, n, 64, extra=("gamma", "beta"))
    # x^ * gamma + beta cancels here and there among a million elements, and what another order of the fp32 sums changes
    # in the last place of x^ * gamma is then many last places of the result: bounded in units of the terms instead
    g, w = _as_f64(got, dtype), _as_f64(want, dtype)
    eps = 2.0 ** -10 if dtype == kh.F16 else 2.0 ** -7
    assert np.array_equal(np.isnan(g), np.isnan(w)) and np.all(np.abs(g - w)[~np.isnan(w)] <= 2 * eps * np.maximum(np.abs(w[~np.isnan(w)]), 1.0))
    assert np.mean(got == want) > 0.98
    got, want = _row_case(ko, kh.layernorm_insts(n, dtype, affine=False), dtype, m, n, 65)
    _check_ulp(got, want, dtype)
    got, want = _row_case(ko, kh.rmsnorm_insts(n, dtype), dtype, m, n, 66, extra=("gamma",))
    _check_ulp(got, want, dtype)


def test_softmax_special_rows(ko, row_path):
    m, n = 6, 1024
    x = ko.fill_normal(m * n, kh.F16, 55, std=4.0).reshape(m, n)
    x[1, 3] = 0x7e00                 # a NaN poisons its row
    x[2, 9] = 0x7c00                 # +inf: inf - inf
    x[3, :] = 0xfc00                 # a row of -inf
    x[4, :] = 0x7bff                 # a row of the largest finite value: uniform 1/n
    insts = kh.softmax_insts(kh.F16)
    got, want = _run_prog(ko, insts, [x], [kh.F16], kh.F16, m, n)
    _check_ulp(got, want, kh.F16)
    assert np.all(np.isnan(got[[1, 2, 3]].view(np.float16))) and np.all(got[4] == np.float16(1.0 / n).view(np.uint16))


@pytest.mark.parametrize("dtype", [kh.F16, kh.BF16])
@pytest.mark.parametrize("m,n", [(12, 1024), (6, 8192), (5, 200)])
def test_layernorm_and_rmsnorm_rows(ko, row_path, dtype, m, n):
    got, want = _row_case(ko, kh.layernorm_insts(n, dtype), dtype, m, n, 61, extra=("gamma", "beta"))
    _check_ulp(got, want, dtype)
    got, want = _row_case(ko, kh.layernorm_insts(n, dtype, affine=False), dtype, m, n, 62)
    _check_ulp(got, want, dtype)
    got, want = _row_case(ko, kh.rmsnorm_insts(n, dtype), dtype, m, n, 63, extra=("gamma",))
    _check_ulp(got, want, dtype)


def test_row_program_value_read_back_from_lds_and_special_values(ko):
    # e / sum(e) * e: when the last factor is wanted the value is no longer on the stack below and comes back from LDS
    insts = [dict(op=kh.EW_LD_GLOBAL, dst=0, a=0), dict(op=kh.EW_FPTOFP, dst=1, a=0, dtype=kh.F32),
             dict(op=kh.EW_EXP, dst=1, a=1), dict(op=kh.EW_REDUCE_SUM, dst=2, a=1, b=1), dict(op=kh.EW_DIVF, dst=3, a=1, b=2),
             dict(op=kh.EW_MULF, dst=3, a=3, b=1), dict(op=kh.EW_FPTOFP, dst=4, a=3, dtype=kh.F16, rmode=kh.RN),
             dict(op=kh.EW_ST_GLOBAL, a=4)]
    got, want = _row_case(ko, insts, kh.F16, 10, 2048, 71, std=1.0)
    _check_ulp(got, want, kh.F16)
    # a NaN poisons its own row only; an infinity makes the row's maximum infinite
    m, n = 4, 512
    x = ko.fill_normal(m * n, kh.F16, 72).reshape(m, n)
    x[1, 100] = 0x7e00
    x[2, 7] = 0x7c00
    prog = [dict(op=kh.EW_LD_GLOBAL, dst=0, a=0), dict(op=kh.EW_REDUCE_MAX, dst=1, a=0, b=1), dict(op=kh.EW_ST_GLOBAL, a=1)]
    got, want = _run_prog(ko, prog, [x], [kh.F16], kh.F16, m, n)
    assert np.array_equal(got[[0, 2, 3]], want[[0, 2, 3]]) and np.all(got[2] == 0x7c00)
    assert np.all(np.isnan(got[1].view(np.float16))) and np.all(np.isnan(want[1].view(np.float16)))


def test_softmax_f32_in_and_out(ko):
    m, n = 8, 2048
    x = ko.fill_normal(m * n, kh.F32, 81, std=2.0).reshape(m, n)
    insts = [dict(op=kh.EW_LD_GLOBAL, dst=0, a=0), dict(op=kh.EW_REDUCE_MAX, dst=1, a=0, b=1), dict(op=kh.EW_SUBF, dst=0, a=0, b=1),
             dict(op=kh.EW_EXP, dst=0, a=0), dict(op=kh.EW_REDUCE_SUM, dst=1, a=0, b=1), dict(op=kh.EW_DIVF, dst=0, a=0, b=1),
             dict(op=kh.EW_ST_GLOBAL, a=0)]
    got, want = _run_prog(ko, insts, [x], [kh.F32], kh.F32, m, n)
    g, w = got.view(np.float32).astype(np.float64), want.view(np.float32).astype(np.float64)
    assert np.max(np.abs(g - w) / w) <= 4e-6        # fp32 exp (2 ulp) and a sum in another order
    assert np.allclose(g.sum(axis=1), 1.0, atol=1e-5)


def test_row_programs_outside_the_fused_kernel_are_refused(ko):
    def run(m, n, axis=1):
        x = to_dev(ko.fill_normal(m * n, kh.F16, 1))
        prog = [dict(op=kh.EW_LD_GLOBAL, dst=0, a=0), dict(op=kh.EW_REDUCE_SUM, dst=1, a=0, b=axis), dict(op=kh.EW_ST_GLOBAL, a=1)]
        kh.elementwise(kh.program(prog), [dglobal(x, m, n, n, 1, kh.F16)], dglobal(dev_zeros(m * n, 2), m, n, n, 1, kh.F16))
    for args in ((2, 32776), (4, 100)):                       # longer than 32768; not a multiple of 8
        with pytest.raises(kh.KapyError) as e:
            run(*args)
        assert e.value.status == -3 and "reduce" in e.value.message


# ---------------------------------------------------------------------------------------------------------
# Reduces along axis 0 inside a program: the column machine.
def _along_columns(insts):
    return [dict(i, b=0) if i["op"] in (kh.EW_REDUCE_SUM, kh.EW_REDUCE_MAX) else i for i in insts]


@pytest.mark.parametrize("dtype", [kh.F16, kh.BF16])
@pytest.mark.parametrize("m,n", [(64, 64), (1, 40), (7, 100), (255, 192), (256, 65), (1000, 130), (4096, 64)])
def test_softmax_columns_every_launch_shape(ko, dtype, m, n):
    got, want = _row_case(ko, _along_columns(kh.softmax_insts(dtype)), dtype, m, n, 150 + n % 97)
    _check_ulp(got, want, dtype)
    # every column sums to one
    sums = _as_f64(got, dtype).sum(axis=0)
    assert np.allclose(sums, 1.0, atol=m * 2.0 ** (-11 if dtype == kh.F16 else -8) * 0.05 + 2e-2)


@pytest.mark.parametrize("dtype", [kh.F16, kh.BF16])
@pytest.mark.parametrize("m,n", [(5000, 512), (70000, 64), (64, 2048), (3000, 264), (129, 8)])
def test_column_programs_run_as_phases_over_the_whole_device(ko, dtype, m, n):
    """Widths that are multiples of 8 and at least 64 rows: every reduce is a launch of its own over strips x row chunks with
    its per-column results kept in memory for the phases after it.  Softmax, and a program whose second reduce depends on
    the first and on a column operand, in 16-bit arithmetic (the per-column results are then 16-bit too)."""
    got, want = _row_case(ko, _along_columns(kh.softmax_insts(dtype)), dtype, m, n, 160 + n % 97)
    _check_ulp(got, want, dtype)
    # y = (x - max_col(x)) * c[row] - max_col((x - max_col(x)) * c[row]), all in `dtype`
    insts = [dict(op=kh.EW_LD_GLOBAL, dst=0, a=0), dict(op=kh.EW_REDUCE_MAX, dst=1, a=0, b=0), dict(op=kh.EW_SUBF, dst=0, a=0, b=1),
             dict(op=kh.EW_LD_GLOBAL, dst=2, a=1), dict(op=kh.EW_MULF, dst=0, a=0, b=2), dict(op=kh.EW_REDUCE_MAX, dst=3, a=0, b=0),
             dict(op=kh.EW_SUBF, dst=0, a=0, b=3), dict(op=kh.EW_ST_GLOBAL, a=0)]
    x = ko.fill_normal(m * n, dtype, 161, std=2.0).reshape(m, n)
    c = ko.fill_normal(m, dtype, 162, mean=1.0, std=0.25)
    got, want = _run_prog(ko, insts, [x, c], [dtype, dtype], dtype, m, n, in_shapes=[(m, n), (m, 1)])
    assert np.array_equal(got, want)            # max and single roundings only: bit-exact


def test_column_program_equals_the_row_program_on_the_transposed_problem(ko):
    # the same numbers through the other machine: transposing the operand and the result turns columns into rows;
    # max is exact and the sums differ by the order of the fp32 additions only
    m, n = 96, 200
    x = ko.fill_normal(m * n, kh.F16, 171, std=2.0).reshape(m, n)
    by_cols, _ = _run_prog(ko, _along_columns(kh.softmax_insts(kh.F16)), [x], [kh.F16], kh.F16, m, n)
    by_rows, _ = _run_prog(ko, kh.softmax_insts(kh.F16), [np.ascontiguousarray(x.T)], [kh.F16], kh.F16, n, m)
    assert ulp_diff_f16(by_cols, np.ascontiguousarray(by_rows.T)).max() <= 1


def test_column_reduces_with_broadcast_operands_special_values_and_views(ko):
    m, n = 50, 70
    # (x * scale[row] + shift[col]) centred on its column mean, in f32, stored as bf16
    insts = [dict(op=kh.EW_LD_GLOBAL, dst=0, a=0), dict(op=kh.EW_FPTOFP, dst=0, a=0, dtype=kh.F32),
             dict(op=kh.EW_LD_GLOBAL, dst=1, a=1), dict(op=kh.EW_FPTOFP, dst=1, a=1, dtype=kh.F32),
             dict(op=kh.EW_LD_GLOBAL, dst=2, a=2), dict(op=kh.EW_FPTOFP, dst=2, a=2, dtype=kh.F32),
             dict(op=kh.EW_FMA, dst=0, a=0, b=1, c=2), dict(op=kh.EW_REDUCE_SUM, dst=3, a=0, b=0),
             dict(op=kh.EW_SPLAT, dst=4, dtype=kh.F32, imm=1.0 / m), dict(op=kh.EW_MULF, dst=3, a=3, b=4),
             dict(op=kh.EW_SUBF, dst=0, a=0, b=3), dict(op=kh.EW_FPTOFP, dst=5, a=0, dtype=kh.BF16, rmode=kh.RN),
             dict(op=kh.EW_ST_GLOBAL, a=5)]
    x = ko.fill_normal(m * n, kh.F16, 181).reshape(m, n)
    scale = ko.fill_normal(m, kh.F16, 182, mean=1.0, std=0.25).reshape(m, 1)
    shift = ko.fill_normal(n, kh.F16, 183).reshape(1, n)
    got, want = _run_prog(ko, insts, [x, scale, shift], [kh.F16] * 3, kh.BF16, m, n, in_shapes=[(m, n), (m, 1), (1, n)])
    g, w = _as_f64(got, kh.BF16), _as_f64(want, kh.BF16)
    assert np.max(np.abs(g - w)) <= 2.0 ** -7 * np.max(np.abs(w)) and np.mean(got == want) > 0.9
    # a max along columns is exact; a NaN poisons its own column, an infinity owns its column, -0 stays below +0
    x = ko.fill_normal(m * n, kh.F16, 184).reshape(m, n)
    x[3, 5] = 0x7e00
    x[9, 6] = 0x7c00
    x[:, 7] = 0x8000
    x[:, 8] = 0x8000
    x[11, 8] = 0x0000
    prog = [dict(op=kh.EW_LD_GLOBAL, dst=0, a=0), dict(op=kh.EW_REDUCE_MAX, dst=1, a=0, b=0), dict(op=kh.EW_ST_GLOBAL, a=1)]
    got, want = _run_prog(ko, prog, [x], [kh.F16], kh.F16, m, n)
    keep = np.arange(n) != 5
    assert np.array_equal(got[:, keep], want[:, keep]) and np.all(np.isnan(got[:, 5].view(np.float16)))
    assert np.all(got[:, 6] == 0x7c00) and np.all(got[:, 7] == 0x8000) and np.all(got[:, 8] == 0x0000)
    # a sum of -0 only is -0
    prog[1] = dict(op=kh.EW_REDUCE_SUM, dst=1, a=0, b=0)
    got, want = _run_prog(ko, prog, [x[:, 7:8].copy()], [kh.F16], kh.F16, m, 1)
    assert np.all(got == 0x8000) and np.array_equal(got, want)


@pytest.mark.parametrize("narrow", [kh.F16, kh.BF16])
@pytest.mark.parametrize("m,n", [(256, 64), (4096, 512), (40, 64), (256, 65)])
def test_a_down_cast_right_before_a_column_sum_is_rounded(ko, narrow, m, n):
    """reduce_sum(fptofp(x, f32 -> 16 bit), axis 0): the sum adds the ROUNDED values, on the launches-per-reduce path (at least
    64 rows, width a multiple of 8) and on the one-launch column machine alike.  Rows come in pairs +a + e, -a + e with a in
    [0.5, 1) on the 16-bit grid and e below half a grid step: rounded, every column sums to exactly zero; unrounded, to m * e."""
    rng = np.random.default_rng(7 + m + n)
    step = 2.0 ** (-11 if narrow == kh.F16 else -8)
    a = 0.5 + step * rng.integers(0, int(0.5 / step), size=(m // 2, n))
    e = step / 8
    xf = np.concatenate([a + e, -a + e]).astype(np.float32)
    xf = xf[rng.permutation(m)]
    assert np.all(np.abs(xf.astype(np.float64)) % step != 0)            # e survives in fp32
    x = xf.view(np.uint32)
    insts = [dict(op=kh.EW_LD_GLOBAL, dst=0, a=0), dict(op=kh.EW_FPTOFP, dst=1, a=0, dtype=narrow, rmode=kh.RN),
             dict(op=kh.EW_REDUCE_SUM, dst=2, a=1, b=0), dict(op=kh.EW_ST_GLOBAL, a=2)]
    got, want = _run_prog(ko, insts, [x], [kh.F32], narrow, m, n)
    assert np.array_equal(got, want)
    assert not (got & 0x7FFF).any()              # +-0 everywhere: m * e (a 16-bit value of its own) would show


def test_column_program_on_strided_views_and_f32(ko):
    # operand and result are windows of wider buffers; f32 throughout
    m, n, ld = 300, 90, 128
    x = ko.fill_normal(m * ld, kh.F32, 191, std=2.0).reshape(m, ld)
    insts = _along_columns([dict(op=kh.EW_LD_GLOBAL, dst=0, a=0), dict(op=kh.EW_REDUCE_MAX, dst=1, a=0, b=1), dict(op=kh.EW_SUBF, dst=0, a=0, b=1),
                            dict(op=kh.EW_EXP, dst=0, a=0), dict(op=kh.EW_REDUCE_SUM, dst=1, a=0, b=1), dict(op=kh.EW_DIVF, dst=0, a=0, b=1),
                            dict(op=kh.EW_ST_GLOBAL, a=0)])
    want = np.zeros((m, ld), np.uint32)
    go = lambda a: ko.mk_global(a, m, ld, ld, 1, kh.F32)
    sub = lambda g: ko.sv_global(g, 0, m, 16, 16 + n)
    assert ko.elementwise(ko.program(insts), [sub(go(x))], sub(go(want))) == 0
    dx, dout = to_dev(x), dev_zeros(m * ld, 4)
    dsub = lambda t: kh.sv_global(dglobal(t, m, ld, ld, 1, kh.F32), 0, m, 16, 16 + n)
    kh.elementwise(kh.program(insts), [dsub(dx)], dsub(dout))
    sync()
    got = to_host(dout, np.uint32, (m, ld))
    assert not got[:, :16].any() and not got[:, 16 + n:].any()          # nothing outside the window is written
    g, w = got[:, 16:16 + n].view(np.float32).astype(np.float64), want[:, 16:16 + n].view(np.float32).astype(np.float64)
    assert np.max(np.abs(g - w) / w) <= 4e-6 and np.allclose(g.sum(axis=0), 1.0, atol=1e-5)


def test_reduces_along_both_axes_in_one_program_are_refused(ko):
    m, n = 8, 64
    x = to_dev(ko.fill_normal(m * n, kh.F16, 1))
    prog = [dict(op=kh.EW_LD_GLOBAL, dst=0, a=0), dict(op=kh.EW_REDUCE_SUM, dst=1, a=0, b=0), dict(op=kh.EW_REDUCE_SUM, dst=2, a=1, b=1),
            dict(op=kh.EW_ST_GLOBAL, a=2)]
    with pytest.raises(kh.KapyError) as e:
        kh.elementwise(kh.program(prog), [dglobal(x, m, n, n, 1, kh.F16)], dglobal(dev_zeros(m * n, 2), m, n, n, 1, kh.F16))
    assert e.value.status == -3 and "same axis" in e.value.message
    five = [dict(op=kh.EW_LD_GLOBAL, dst=0, a=0)] + [dict(op=kh.EW_REDUCE_MAX, dst=0, a=0, b=0)] * 5 + [dict(op=kh.EW_ST_GLOBAL, a=0)]
    with pytest.raises(kh.KapyError) as e:
        kh.elementwise(kh.program(five), [dglobal(x, m, n, n, 1, kh.F16)], dglobal(dev_zeros(m * n, 2), m, n, n, 1, kh.F16))
    assert e.value.status == -3 and "at most 4" in e.value.message


# ---------------------------------------------------------------------------------------------------------
# The ops of the reference's elementwise list beyond the arithmetic ones: floor, ceil, sin, cos, maxnumf, minnumf, remf.
@pytest.mark.parametrize("dtype", [kh.F16, kh.BF16, kh.F32])
def test_floor_ceil_maxnum_minnum_rem_are_exact(ko, dtype):
    m, n = 24, 200
    x = ko.fill_normal(m * n, dtype, 201, 0, 0.0, 6.0).reshape(m, n)
    y = ko.fill_normal(m * n, dtype, 201, 1, 0.0, 2.0).reshape(m, n)
    specials = {kh.F16: [0x7e00, 0x3c00, 0x8000, 0x0000, 0x7c00, 0xfc00, 0x4580, 0xc580], kh.BF16: [0x7fc0, 0x3f80, 0x8000, 0x0000, 0x7f80, 0xff80, 0x40b0, 0xc0b0]}
    others = {kh.F16: [0x4000, 0x7e00, 0x0000, 0x8000, 0x4200, 0x3800, 0x4000, 0x4000], kh.BF16: [0x4000, 0x7fc0, 0x0000, 0x8000, 0x4040, 0x3f00, 0x4000, 0x4000]}
    if dtype != kh.F32:
        x.ravel()[:8] = specials[dtype]
        y.ravel()[:8] = others[dtype]
    else:
        x.ravel()[:8] = [np.nan, 1.0, -0.0, 0.0, np.inf, -np.inf, 5.5, -5.5]
        y.ravel()[:8] = [2.0, np.nan, 0.0, -0.0, 3.0, 0.5, 2.0, 2.0]
    L0, L1 = dict(op=kh.EW_LD_GLOBAL, dst=0, a=0), dict(op=kh.EW_LD_GLOBAL, dst=1, a=1)
    for op in (kh.EW_FLOOR, kh.EW_CEIL):
        got, want = _run_prog(ko, [L0, dict(op=op, dst=2, a=0), dict(op=kh.EW_ST_GLOBAL, a=2)], [x], [dtype], dtype, m, n)
        assert _same_bits_or_nan(got, want, dtype), op
    for op in (kh.EW_MAXNUMF, kh.EW_MINNUMF, kh.EW_REMF):
        got, want = _run_prog(ko, [L0, L1, dict(op=op, dst=2, a=0, b=1), dict(op=kh.EW_ST_GLOBAL, a=2)], [x, y], [dtype, dtype], dtype, m, n)
        assert _same_bits_or_nan(got, want, dtype), op


def _same_bits_or_nan(got, want, dtype):
    if dtype == kh.F32:
        g, w = got.view(np.float32), want.view(np.float32)
        nan = np.isnan(w)
        return np.array_equal(np.isnan(g), nan) and np.array_equal(got.view(np.uint32)[~nan], want.view(np.uint32)[~nan])
    nan = np.isnan(_as_f64(want, dtype))
    return np.array_equal(np.isnan(_as_f64(got, dtype)), nan) and np.array_equal(got[~nan], want[~nan])


@pytest.mark.parametrize("dtype", [kh.F16, kh.BF16])
def test_sin_cos_within_two_ulp(ko, dtype):
    m, n = 32, 256
    x = ko.fill_normal(m * n, dtype, 211, 0, 0.0, 4.0).reshape(m, n)
    for op in (kh.EW_SIN, kh.EW_COS):
        insts = [dict(op=kh.EW_LD_GLOBAL, dst=0, a=0), dict(op=kh.EW_FPTOFP, dst=1, a=0, dtype=kh.F32), dict(op=op, dst=1, a=1),
                 dict(op=kh.EW_FPTOFP, dst=2, a=1, dtype=dtype, rmode=kh.RN), dict(op=kh.EW_ST_GLOBAL, a=2)]
        got, want = _run_prog(ko, insts, [x], [dtype], dtype, m, n)
        _check_ulp(got, want, dtype)


def test_division_keeps_the_sign_of_a_zero_dividend(ko):
    """-0 / y is -0 for y > 0: the lean division corrects its quotient by the remainder, and adding a +0 remainder would
    lose the sign.  Through the stack machine, the row machine (division by a per-row value) and a compiled kernel."""
    m, n = 16, 128
    x = ko.fill_normal(m * n, kh.F32, 221, 0, 0.0, 1.0).reshape(m, n)
    x[:, ::3] = -0.0
    x[:, 1::7] = 0.0
    y = np.abs(ko.fill_normal(m * n, kh.F32, 221, 1, 0.0, 1.0)).reshape(m, n) + np.float32(0.5)
    L0, L1, ST = dict(op=kh.EW_LD_GLOBAL, dst=0, a=0), dict(op=kh.EW_LD_GLOBAL, dst=1, a=1), dict(op=kh.EW_ST_GLOBAL, a=2)
    insts = [L0, L1, dict(op=kh.EW_DIVF, dst=2, a=0, b=1), ST]
    got, want = _run_prog(ko, insts, [x, y], [kh.F32, kh.F32], kh.F32, m, n)
    assert np.array_equal(got, want) and np.array_equal(np.signbit(got.view(np.float32)), np.signbit(x / y))
    # x / rowmax(y): the row machine's division of a row by one value
    insts = [L0, L1, dict(op=kh.EW_REDUCE_MAX, dst=1, a=1, b=1), dict(op=kh.EW_DIVF, dst=2, a=0, b=1), ST]
    got, want = _run_prog(ko, insts, [x, y], [kh.F32, kh.F32], kh.F32, m, n)
    assert np.array_equal(np.signbit(got.view(np.float32)), np.signbit(want.view(np.float32)))
    assert np.max(np.abs(got.view(np.float32) - want.view(np.float32))) <= 1e-6
    # compiled
    insts = [L0, L1, dict(op=kh.EW_DIVF, dst=2, a=0, b=1), dict(op=kh.EW_NEGF, dst=2, a=2), dict(op=kh.EW_NEGF, dst=2, a=2), ST]
    dx, dy, dz = to_dev(x), to_dev(y), dev_zeros(m * n, 4)
    g = lambda t: dglobal(t, m, n, n, 1, kh.F32)
    try:
        kh.elementwise_specialize(kh.program(insts), [g(dx), g(dy)], g(dz))
    except kh.KapyError as e:
        assert e.status == kh.ERR_UNSUPPORTED      # no runtime compiler on this machine
        return
    kh.elementwise(kh.program(insts), [g(dx), g(dy)], g(dz))
    sync()
    out = to_host(dz, np.float32, (m, n))
    assert np.array_equal(out, x / y) and np.array_equal(np.signbit(out), np.signbit(x / y))


@pytest.mark.parametrize("dtype", [kh.F16, kh.BF16, kh.F32])
@pytest.mark.parametrize("m,n", [(301, 501), (17, 3), (2, 7), (64, 1001), (1000, 9)])
def test_dense_operands_with_odd_widths_run_as_one_line(ko, dtype, m, n):
    """Dense matrices of one shape whose rows are not whole vectors: the program runs over all elements as one line (and once
    more over the last few); a scalar operand rides along.  Bit-exact (one rounding per op), guard words intact."""
    eb = kh.DTYPE_BYTES[dtype]
    a, b = ko.fill_normal(m * n, dtype, 91, 0), ko.fill_normal(m * n, dtype, 91, 1)
    c = ko.fill_normal(1, dtype, 92, 0)
    insts = [dict(op=kh.EW_LD_GLOBAL, dst=0, a=0), dict(op=kh.EW_LD_GLOBAL, dst=1, a=1), dict(op=kh.EW_LD_GLOBAL, dst=2, a=2),
             dict(op=kh.EW_MULF, dst=3, a=0, b=1), dict(op=kh.EW_ADDF, dst=3, a=3, b=2), dict(op=kh.EW_MAXIMUMF, dst=3, a=3, b=1),
             dict(op=kh.EW_ST_GLOBAL, a=3)]
    np_t = {2: np.uint16, 4: np.uint32}[eb]
    want = np.zeros(m * n, np_t)
    gos = [ko.mk_global(a, m, n, n, 1, dtype), ko.mk_global(b, m, n, n, 1, dtype), ko.mk_global(c, 1, 1, 1, 1, dtype)]
    assert ko.elementwise(ko.program(insts), gos, ko.mk_global(want, m, n, n, 1, dtype)) == 0
    da, db_, dc = to_dev(a), to_dev(b), to_dev(c)
    dout = dev_zeros(m * n + 32, eb, fill=0x5A5A)
    kh.elementwise(kh.program(insts), [dglobal(da, m, n, n, 1, dtype), dglobal(db_, m, n, n, 1, dtype), dglobal(dc, 1, 1, 1, 1, dtype)],
                   dglobal(dout, m, n, n, 1, dtype))
    sync()
    got = to_host(dout, np_t)
    assert np.array_equal(got[:m * n], want.view(np_t)) and np.all(got[m * n:] == got[-1]) and got[-1] != 0


@pytest.mark.parametrize("dtype", [kh.F16, kh.F32])
def test_column_major_result_runs_as_the_transposed_problem(ko, dtype):
    """Result and full operands column-major, a [1 x n] and a [m x 1] operand beside them: the call is the row-major program on
    the transposed problem (the row operand becomes a column operand and the other way round).  Bit-exact."""
    m, n = 200, 136
    eb = kh.DTYPE_BYTES[dtype]
    np_t = {2: np.uint16, 4: np.uint32}[eb]
    a, b = ko.fill_normal(m * n, dtype, 95, 0), ko.fill_normal(m * n, dtype, 95, 1)
    r, c = ko.fill_normal(n, dtype, 96, 0), ko.fill_normal(m, dtype, 96, 1)
    insts = [dict(op=kh.EW_LD_GLOBAL, dst=0, a=0), dict(op=kh.EW_LD_GLOBAL, dst=1, a=1), dict(op=kh.EW_LD_GLOBAL, dst=2, a=2),
             dict(op=kh.EW_LD_GLOBAL, dst=3, a=3), dict(op=kh.EW_MULF, dst=4, a=0, b=2), dict(op=kh.EW_FMA, dst=4, a=1, b=3, c=4),
             dict(op=kh.EW_ST_GLOBAL, a=4)]
    want = np.zeros(m * n, np_t)
    shapes = [(m, n, 1, m), (m, n, 1, m), (1, n, n, 1), (m, 1, 1, 1)]      # (rows, cols, stride0, stride1): a, b column-major
    gos = [ko.mk_global(t, *sh, dtype) for t, sh in zip((a, b, r, c), shapes)]
    assert ko.elementwise(ko.program(insts), gos, ko.mk_global(want, m, n, 1, m, dtype)) == 0
    devs = [to_dev(t) for t in (a, b, r, c)]
    dout = dev_zeros(m * n + 32, eb, fill=0x5A5A)
    kh.elementwise(kh.program(insts), [dglobal(t, *sh, dtype) for t, sh in zip(devs, shapes)], dglobal(dout, m, n, 1, m, dtype))
    sync()
    got = to_host(dout, np_t)
    assert np.array_equal(got[:m * n], want.view(np_t)) and np.all(got[m * n:] == got[-1]) and got[-1] != 0


@pytest.mark.parametrize("dtype", [kh.F16, kh.BF16])
@pytest.mark.parametrize("axis", [1, 0])
def test_softmax_of_large_magnitudes(ko, dtype, axis):
    """Lines whose maximum is large (6e4 in f16, 1e6 and 3e38 in bf16) and whose other elements lie within a few units of it: the
    exponent (x - max) * log2(e) must be formed from the difference - a product max * log2(e) of its own carries a rounding of
    0.4 % (f16) to several per cent, or overflows - through the row kernels and the column kernels alike."""
    m, n = (64, 2048) if axis == 1 else (2048, 64)
    rng = np.random.default_rng(axis)
    top = 60000.0 if dtype == kh.F16 else 1.0e6
    x = (top - np.abs(rng.standard_normal((m, n))) * (16.0 if dtype == kh.F16 else 3.0e4)).astype(np.float32)
    if dtype == kh.BF16:
        line = (slice(None), 3) if axis == 0 else (3, slice(None))
        x[line] = 3.0e38 - np.abs(rng.standard_normal(x[line].shape)) * 1.0e37     # max * log2(e) overflows fp32
    bits = ko.fptofp(np.ascontiguousarray(x), ko.F32, dtype).reshape(m, n)
    insts = kh.softmax_insts(dtype) if axis == 1 else _along_columns(kh.softmax_insts(dtype))
    got, want = _run_prog(ko, insts, [bits], [dtype], dtype, m, n, in_shapes=[(m, n)])
    _check_ulp(got, want, dtype)
