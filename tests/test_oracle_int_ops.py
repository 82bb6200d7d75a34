"""Pins the checker's integer, compare, select and conversion ops (arith.addi ... arith.select, kapy.arange; the reference's
conversion list, ElementwiseOpToLLVM.cpp:1178-1215) against numpy's integer arithmetic: wrapping results per width, truncating
and flooring division, arithmetic and logical shifts, signed and unsigned orderings, MLIR's compare predicates, one-rounding
int -> float conversions.  The values MLIR leaves undefined are pinned to what the header documents."""
import numpy as np
import pytest

NP_INT = {"I8": np.int8, "I16": np.int16, "I32": np.int32}
BITS = {"I8": 8, "I16": 16, "I32": 32}


def _run(ko, insts, ins, in_dtypes, out_dtype, m, n, shapes=None):
    shapes = shapes or [(m, n)] * len(ins)
    out = np.zeros((m, n), ko.NP_STORAGE[out_dtype])
    gs = [ko.mk_global(a, s[0], s[1], s[1], 1, dt) for a, s, dt in zip(ins, shapes, in_dtypes)]
    rc = ko.elementwise(ko.program(insts), gs, ko.mk_global(out, m, n, n, 1, out_dtype))
    assert rc == 0, rc
    return out


def _operands(rng, name, m, n):
    """Random values of the width with the interesting ones mixed in: 0, +-1, the extremes."""
    t, bits = NP_INT[name], BITS[name]
    lo, hi = -(1 << (bits - 1)), (1 << (bits - 1)) - 1
    special = np.array([0, 1, -1, 2, -2, lo, hi, lo + 1, 3, 7, bits - 1, bits, bits + 1], np.int64)
    def one():
        a = rng.integers(lo, hi + 1, size=m * n, dtype=np.int64)
        small = rng.integers(-9, 10, size=m * n, dtype=np.int64)
        pick = rng.integers(0, 4, size=m * n)
        a = np.where(pick == 0, small, a)
        a = np.where(pick == 1, special[rng.integers(0, len(special), size=m * n)], a)
        return a.reshape(m, n)
    return one().astype(t), one().astype(t)


def _wrap(v, name):
    return v.astype(np.int64).astype(NP_INT[name]) if name != "I32" else (v.astype(np.int64) & 0xFFFFFFFF).astype(np.uint32).view(np.int32).reshape(v.shape)


def _trunc_div(a, b):
    q = np.abs(a) // np.maximum(np.abs(b), 1)
    return np.where((a < 0) != (b < 0), -q, q)


@pytest.mark.parametrize("name", ["I8", "I16", "I32"])
def test_integer_binary_ops_against_numpy(ko, name):
    rng = np.random.default_rng(BITS[name])
    m, n = 40, 50
    x, y = _operands(rng, name, m, n)
    dt = getattr(ko, name)
    bits = BITS[name]
    a, b = x.astype(np.int64), y.astype(np.int64)
    mask = (1 << bits) - 1
    ua, ub = a & mask, b & mask
    nz = b != 0
    safe_b = np.where(nz, b, 1)
    safe_ub = np.where(nz, ub, 1)
    sh = np.minimum(ub, bits - 1)
    want = {
        ko.EW_ADDI: a + b, ko.EW_SUBI: a - b, ko.EW_MULI: a * b,
        ko.EW_DIVSI: np.where(nz, _trunc_div(a, safe_b), 0),
        ko.EW_DIVUI: np.where(nz, ua // safe_ub, 0),
        ko.EW_FLOORDIVSI: np.where(nz, a // safe_b, 0),
        ko.EW_CEILDIVSI: np.where(nz, -((-a) // safe_b), 0),
        ko.EW_CEILDIVUI: np.where(nz, (ua + safe_ub - 1) // safe_ub, 0),
        ko.EW_REMSI: np.where(nz, a - _trunc_div(a, safe_b) * safe_b, 0),
        ko.EW_REMUI: np.where(nz, ua % safe_ub, 0),
        ko.EW_ANDI: ua & ub, ko.EW_ORI: ua | ub, ko.EW_XORI: ua ^ ub,
        ko.EW_SHLI: np.where(ub >= bits, 0, ua << np.minimum(ub, 63)),
        ko.EW_SHRUI: np.where(ub >= bits, 0, ua >> np.minimum(ub, 63)),
        ko.EW_SHRSI: a >> sh,
        ko.EW_MAXSI: np.maximum(a, b), ko.EW_MINSI: np.minimum(a, b),
        ko.EW_MAXUI: np.maximum(ua, ub), ko.EW_MINUI: np.minimum(ua, ub),
    }
    for op, w in want.items():
        insts = [dict(op=ko.EW_LD_GLOBAL, dst=0, a=0), dict(op=ko.EW_LD_GLOBAL, dst=1, a=1), dict(op=op, dst=2, a=0, b=1), dict(op=ko.EW_ST_GLOBAL, a=2)]
        got = _run(ko, insts, [x, y], [dt, dt], dt, m, n)
        assert np.array_equal(got, _wrap(w, name)), "op %d on %s" % (op, name)
    # the documented corner cases, spelled out
    lo = -(1 << (bits - 1))
    xs = np.array([[lo, lo, 5, -5, 7, -7, 1, -1]], NP_INT[name])
    ys = np.array([[-1, 0, 0, 0, -2, 2, bits, bits]], NP_INT[name])
    prog = lambda op: [dict(op=ko.EW_LD_GLOBAL, dst=0, a=0), dict(op=ko.EW_LD_GLOBAL, dst=1, a=1), dict(op=op, dst=2, a=0, b=1), dict(op=ko.EW_ST_GLOBAL, a=2)]
    div = _run(ko, prog(ko.EW_DIVSI), [xs, ys], [dt, dt], dt, 1, 8)[0]
    assert list(div[:6]) == [lo, 0, 0, 0, -3, -3]                      # min / -1 wraps, x / 0 = 0, truncation toward zero
    rem = _run(ko, prog(ko.EW_REMSI), [xs, ys], [dt, dt], dt, 1, 8)[0]
    assert list(rem[:6]) == [0, 0, 0, 0, 1, -1]                        # the remainder takes the dividend's sign
    fl = _run(ko, prog(ko.EW_FLOORDIVSI), [xs, ys], [dt, dt], dt, 1, 8)[0]
    ce = _run(ko, prog(ko.EW_CEILDIVSI), [xs, ys], [dt, dt], dt, 1, 8)[0]
    assert list(fl[4:6]) == [-4, -4] and list(ce[4:6]) == [-3, -3]
    assert list(_run(ko, prog(ko.EW_SHLI), [xs, ys], [dt, dt], dt, 1, 8)[0][6:]) == [0, 0]       # a shift by the width
    assert list(_run(ko, prog(ko.EW_SHRSI), [xs, ys], [dt, dt], dt, 1, 8)[0][6:]) == [0, -1]
    assert list(_run(ko, prog(ko.EW_SHRUI), [xs, ys], [dt, dt], dt, 1, 8)[0][6:]) == [0, 0]


@pytest.mark.parametrize("name", ["I8", "I16", "I32"])
def test_cmpi_select_absi_and_integer_casts(ko, name):
    rng = np.random.default_rng(100 + BITS[name])
    m, n = 30, 40
    x, y = _operands(rng, name, m, n)
    y = np.where(rng.integers(0, 3, size=(m, n)) == 0, x, y).astype(NP_INT[name])   # some equal pairs
    dt, bits = getattr(ko, name), BITS[name]
    a, b = x.astype(np.int64), y.astype(np.int64)
    ua, ub = a & ((1 << bits) - 1), b & ((1 << bits) - 1)
    preds = {ko.CMPI_EQ: a == b, ko.CMPI_NE: a != b, ko.CMPI_SLT: a < b, ko.CMPI_SLE: a <= b, ko.CMPI_SGT: a > b, ko.CMPI_SGE: a >= b,
             ko.CMPI_ULT: ua < ub, ko.CMPI_ULE: ua <= ub, ko.CMPI_UGT: ua > ub, ko.CMPI_UGE: ua >= ub}
    ld2 = [dict(op=ko.EW_LD_GLOBAL, dst=0, a=0), dict(op=ko.EW_LD_GLOBAL, dst=1, a=1)]
    for pred, w in preds.items():
        got = _run(ko, ld2 + [dict(op=ko.EW_CMPI, dst=2, a=0, b=1, c=pred), dict(op=ko.EW_ST_GLOBAL, a=2)], [x, y], [dt, dt], ko.I1, m, n)
        assert np.array_equal(got, w.astype(np.uint8)), pred
        # select(cmp, x, y) and extui / extsi of the i1
        got = _run(ko, ld2 + [dict(op=ko.EW_CMPI, dst=2, a=0, b=1, c=pred), dict(op=ko.EW_SELECT, dst=3, a=2, b=0, c=1), dict(op=ko.EW_ST_GLOBAL, a=3)],
                   [x, y], [dt, dt], dt, m, n)
        assert np.array_equal(got, np.where(w, x, y))
    for op, w in ((ko.EW_EXTUI, (a < b).astype(np.int64)), (ko.EW_EXTSI, -(a < b).astype(np.int64))):
        got = _run(ko, ld2 + [dict(op=ko.EW_CMPI, dst=2, a=0, b=1, c=ko.CMPI_SLT), dict(op=op, dst=3, a=2, dtype=dt), dict(op=ko.EW_ST_GLOBAL, a=3)],
                   [x, y], [dt, dt], dt, m, n)
        assert np.array_equal(got, w.astype(NP_INT[name]))
    got = _run(ko, [dict(op=ko.EW_LD_GLOBAL, dst=0, a=0), dict(op=ko.EW_ABSI, dst=1, a=0), dict(op=ko.EW_ST_GLOBAL, a=1)], [x], [dt], dt, m, n)
    assert np.array_equal(got, _wrap(np.abs(a), name))                  # |most negative| wraps to itself
    for other in ("I8", "I16", "I32"):
        if other == name:
            continue
        od = getattr(ko, other)
        if BITS[other] < bits:
            got = _run(ko, [dict(op=ko.EW_LD_GLOBAL, dst=0, a=0), dict(op=ko.EW_TRUNCI, dst=1, a=0, dtype=od), dict(op=ko.EW_ST_GLOBAL, a=1)], [x], [dt], od, m, n)
            assert np.array_equal(got, _wrap(a, other))
        else:
            for op, w in ((ko.EW_EXTSI, a), (ko.EW_EXTUI, ua)):
                got = _run(ko, [dict(op=ko.EW_LD_GLOBAL, dst=0, a=0), dict(op=op, dst=1, a=0, dtype=od), dict(op=ko.EW_ST_GLOBAL, a=1)], [x], [dt], od, m, n)
                assert np.array_equal(got, _wrap(w, other))


def test_cmpf_predicates_with_nan_and_signed_zero(ko):
    vals = np.array([0.0, -0.0, 1.0, -1.0, 2.5, np.inf, -np.inf, np.nan], np.float32)
    a, b = np.meshgrid(vals, vals, indexing="ij")
    a, b = np.ascontiguousarray(a), np.ascontiguousarray(b)
    un = np.isnan(a) | np.isnan(b)
    with np.errstate(invalid="ignore"):
        ordered = {ko.CMPF_OEQ: a == b, ko.CMPF_OGT: a > b, ko.CMPF_OGE: a >= b, ko.CMPF_OLT: a < b, ko.CMPF_OLE: a <= b, ko.CMPF_ONE: (a != b) & ~un}
    want = dict(ordered)
    want.update({ko.CMPF_UEQ: ordered[ko.CMPF_OEQ] | un, ko.CMPF_UGT: ordered[ko.CMPF_OGT] | un, ko.CMPF_UGE: ordered[ko.CMPF_OGE] | un,
                 ko.CMPF_ULT: ordered[ko.CMPF_OLT] | un, ko.CMPF_ULE: ordered[ko.CMPF_OLE] | un, ko.CMPF_UNE: ordered[ko.CMPF_ONE] | un,
                 ko.CMPF_ORD: ~un, ko.CMPF_UNO: un, ko.CMPF_FALSE: np.zeros_like(un), ko.CMPF_TRUE: np.ones_like(un)})
    for pred, w in want.items():
        got = _run(ko, [dict(op=ko.EW_LD_GLOBAL, dst=0, a=0), dict(op=ko.EW_LD_GLOBAL, dst=1, a=1), dict(op=ko.EW_CMPF, dst=2, a=0, b=1, c=pred),
                        dict(op=ko.EW_ST_GLOBAL, a=2)], [a.view(np.uint32), b.view(np.uint32)], [ko.F32, ko.F32], ko.I1, 8, 8)
        assert np.array_equal(got, w.astype(np.uint8)), pred


def _round_to_bits(v, keep):
    """v (float64, exact integers) rounded to `keep` significant bits, ties to even."""
    mant, exp = np.frexp(v)
    return np.ldexp(np.rint(mant * (1 << keep)), exp - keep)


def test_sitofp_rounds_once_fptosi_truncates_and_saturates(ko):
    rng = np.random.default_rng(5)
    m, n = 64, 64
    x = rng.integers(-(1 << 31), 1 << 31, size=(m, n), dtype=np.int64)
    x[0, :8] = [0, 1, -1, (1 << 24) + 1, (1 << 24) + 3, 0x7FFFFFFF, -(1 << 31), 0x7FFFFF80]
    x[1, :4] = [0x00808000, 0x00818000, 0x00808001, -0x00808000]         # exact ties and near-ties of the 8-bit significand
    xi = x.astype(np.int32)
    cast = lambda dt: [dict(op=ko.EW_LD_GLOBAL, dst=0, a=0), dict(op=ko.EW_SITOFP, dst=1, a=0, dtype=dt), dict(op=ko.EW_ST_GLOBAL, a=1)]
    got = _run(ko, cast(ko.F32), [xi], [ko.I32], ko.F32, m, n).view(np.float32)
    assert np.array_equal(got, xi.astype(np.float32))
    got = _run(ko, cast(ko.BF16), [xi], [ko.I32], ko.BF16, m, n)
    want = _round_to_bits(x.astype(np.float64), 8).astype(np.float32).view(np.uint32) >> 16
    assert np.array_equal(got, want.astype(np.uint16))
    small = (x % 200001 - 100000).astype(np.int32)                        # f16's range and beyond (to infinity)
    got = _run(ko, cast(ko.F16), [small], [ko.I32], ko.F16, m, n)
    with np.errstate(over="ignore"):
        assert np.array_equal(got, small.astype(np.float64).astype(np.float16).view(np.uint16))
    # fptosi: toward zero; beyond i32 saturates, NaN gives 0; a narrower result keeps the low bits of the i32
    f = (rng.standard_normal((m, n)) * 10.0 ** rng.integers(-1, 11, size=(m, n))).astype(np.float32)
    f[0, :6] = [np.nan, np.inf, -np.inf, 2147483648.0, -2147483904.0, -0.75]
    i32 = np.where(np.isnan(f), 0, np.clip(np.trunc(f.astype(np.float64)), -(1 << 31), (1 << 31) - 1)).astype(np.int64)
    for name in ("I32", "I16", "I8"):
        dt = getattr(ko, name)
        got = _run(ko, [dict(op=ko.EW_LD_GLOBAL, dst=0, a=0), dict(op=ko.EW_FPTOSI, dst=1, a=0, dtype=dt), dict(op=ko.EW_ST_GLOBAL, a=1)],
                   [f.view(np.uint32)], [ko.F32], dt, m, n)
        assert np.array_equal(got, _wrap(i32, name)), name


def test_bitcast_arange_and_integer_splat(ko):
    rng = np.random.default_rng(6)
    m, n = 16, 24
    bits = rng.integers(0, 1 << 16, size=(m, n)).astype(np.uint16)
    bits = np.where((bits & 0x7C00) == 0x7C00, bits & 0x83FF, bits).astype(np.uint16)   # no infinities / NaNs: their payloads may be quieted
    got = _run(ko, [dict(op=ko.EW_LD_GLOBAL, dst=0, a=0), dict(op=ko.EW_BITCAST, dst=1, a=0, dtype=ko.I16), dict(op=ko.EW_ST_GLOBAL, a=1)], [bits], [ko.F16], ko.I16, m, n)
    assert np.array_equal(got.view(np.uint16), bits)
    got = _run(ko, [dict(op=ko.EW_LD_GLOBAL, dst=0, a=0), dict(op=ko.EW_BITCAST, dst=1, a=0, dtype=ko.F16), dict(op=ko.EW_ST_GLOBAL, a=1)], [bits.view(np.int16)], [ko.I16], ko.F16, m, n)
    assert np.array_equal(got, bits)
    w = rng.integers(-(1 << 31), 1 << 31, size=(m, n)).astype(np.int32)
    w = np.where((w.view(np.uint32) & 0x7F800000) == 0x7F800000, w & ~0x7F800000 | 0x3F000000, w).astype(np.int32)
    got = _run(ko, [dict(op=ko.EW_LD_GLOBAL, dst=0, a=0), dict(op=ko.EW_BITCAST, dst=1, a=0, dtype=ko.F32), dict(op=ko.EW_ST_GLOBAL, a=1)], [w], [ko.I32], ko.F32, m, n)
    assert np.array_equal(got.view(np.int32), w)
    # arange along either axis plus an integer splat: (start + index) * 3, the causal mask j <= i
    for axis in (0, 1):
        got = _run(ko, [dict(op=ko.EW_ARANGE, dst=0, a=-5, b=axis), dict(op=ko.EW_SPLAT, dst=1, dtype=ko.I32, a=3), dict(op=ko.EW_MULI, dst=2, a=0, b=1),
                        dict(op=ko.EW_ST_GLOBAL, a=2)], [], [], ko.I32, m, n)
        idx = np.arange(m)[:, None] + np.zeros((1, n), np.int64) if axis == 0 else np.arange(n)[None, :] + np.zeros((m, 1), np.int64)
        assert np.array_equal(got, ((idx - 5) * 3).astype(np.int32))
    got = _run(ko, [dict(op=ko.EW_ARANGE, dst=0, a=0, b=0), dict(op=ko.EW_ARANGE, dst=1, a=0, b=1), dict(op=ko.EW_CMPI, dst=2, a=1, b=0, c=ko.CMPI_SLE),
                    dict(op=ko.EW_ST_GLOBAL, a=2)], [], [], ko.I1, m, n)
    assert np.array_equal(got, np.tril(np.ones((m, n), np.uint8)))
    for name in ("I8", "I16"):
        dt = getattr(ko, name)
        got = _run(ko, [dict(op=ko.EW_SPLAT, dst=0, dtype=dt, a=1000003), dict(op=ko.EW_ST_GLOBAL, a=0)], [], [], dt, 2, 8)
        assert np.all(got == _wrap(np.array([1000003]), name)[0])


def test_typing_rules_of_the_integer_ops(ko):
    x = np.zeros((4, 8), np.int32)
    f = np.zeros((4, 8), np.uint32)
    ld = [dict(op=ko.EW_LD_GLOBAL, dst=0, a=0), dict(op=ko.EW_LD_GLOBAL, dst=1, a=1)]
    bad = [
        ld + [dict(op=ko.EW_ADDI, dst=2, a=0, b=1), dict(op=ko.EW_ST_GLOBAL, a=2)],                        # addi of an int and a float
        ld + [dict(op=ko.EW_ADDF, dst=2, a=0, b=0), dict(op=ko.EW_ST_GLOBAL, a=2)],                        # addf on integers
        ld + [dict(op=ko.EW_SELECT, dst=2, a=0, b=0, c=0), dict(op=ko.EW_ST_GLOBAL, a=2)],                 # the condition is not an i1
        ld + [dict(op=ko.EW_EXTSI, dst=2, a=0, dtype=ko.I16), dict(op=ko.EW_ST_GLOBAL, a=2)],              # "widening" to a narrower type
        ld + [dict(op=ko.EW_BITCAST, dst=2, a=0, dtype=ko.F16), dict(op=ko.EW_ST_GLOBAL, a=2)],            # widths differ
        ld + [dict(op=ko.EW_CMPI, dst=2, a=0, b=0, c=10), dict(op=ko.EW_ST_GLOBAL, a=2)],                  # no such predicate
    ]
    gs = [ko.mk_global(x, 4, 8, 8, 1, ko.I32), ko.mk_global(f, 4, 8, 8, 1, ko.F32)]
    for insts in bad:
        out = np.zeros((4, 8), np.int32)
        assert ko.elementwise(ko.program(insts), gs, ko.mk_global(out, 4, 8, 8, 1, ko.I32)) != 0
