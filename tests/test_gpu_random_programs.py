"""Seeded random elementwise programs built from exactly rounded ops only (add, sub, mul, div, rem, max, min, maxnum, minnum, fma, neg, abs, sqrt, floor, ceil and
casts between every float type), over random operand kinds (full, column-major, row, column, scalar) and shapes: the machines
and the compiled kernels must both reproduce the oracle bit for bit (NaNs compared as NaNs)."""
import numpy as np
import pytest

import kapy_hip as kh
from gpu_util import dev_zeros, dglobal, sync, to_dev, to_host

pytestmark = pytest.mark.gpu
NP_OF = {1: np.uint8, 2: np.uint16, 4: np.uint32}
L, ST, CAST = kh.EW_LD_GLOBAL, kh.EW_ST_GLOBAL, kh.EW_FPTOFP


def _random_case(rng):
    m, n = [(16, 64), (40, 200), (64, 64), (8, 1000), (136, 72)][rng.randint(5)]
    compute = [kh.F16, kh.BF16, kh.F32][rng.randint(3)]
    n_ins = 1 + rng.randint(3)
    kinds = ["full"] + [["full", "T", "row", "col", "scalar"][rng.randint(5)] for _ in range(n_ins - 1)]
    if rng.randint(3) == 0:
        kinds[0] = "T"
    in_dtypes = [[kh.F16, kh.BF16, kh.F32, kh.F8E4M3, kh.F8E5M2][rng.randint(5)] for _ in range(n_ins)]
    insts, regs, r = [], [], 0
    for k in range(n_ins):
        insts.append(dict(op=L, dst=r, a=k))
        if in_dtypes[k] != compute:
            insts.append(dict(op=CAST, dst=r, a=r, dtype=compute, rmode=kh.RN if rng.randint(2) or (in_dtypes[k] == kh.BF16 and False) else kh.RZ))
        regs.append(r)
        r += 1
    binary = [kh.EW_ADDF, kh.EW_SUBF, kh.EW_MULF, kh.EW_DIVF, kh.EW_MAXIMUMF, kh.EW_MINIMUMF, kh.EW_MAXNUMF, kh.EW_MINNUMF, kh.EW_REMF]
    unary = [kh.EW_NEGF, kh.EW_ABSF, kh.EW_SQRT, kh.EW_FLOOR, kh.EW_CEIL]
    for _ in range(2 + rng.randint(7)):
        pick = lambda: regs[rng.randint(len(regs))]
        kind = rng.randint(10)
        if kind < 6:
            insts.append(dict(op=binary[rng.randint(len(binary))], dst=r, a=pick(), b=pick()))
        elif kind < 8:
            insts.append(dict(op=unary[rng.randint(len(unary))], dst=r, a=pick()))
        elif kind == 8 and compute != kh.BF16:       # (a bf16 fma is an fp32 fma rounded again: not exactly rounded)
            insts.append(dict(op=kh.EW_FMA, dst=r, a=pick(), b=pick(), c=pick()))
        else:
            insts.append(dict(op=kh.EW_SPLAT, dst=r, dtype=compute, imm=float(rng.choice([0.0, 1.0, -2.5, 0.333, 1e4, 3e-5]))))
        regs.append(r)
        r = min(r + 1, 14)       # (16 registers: the last ones get reused)
    out_dtype = [kh.F16, kh.BF16, kh.F32, kh.F8E4M3, kh.F8E5M2][rng.randint(5)]
    last = regs[-1]
    if out_dtype != compute:
        narrowing = kh.DTYPE_BYTES[out_dtype] < kh.DTYPE_BYTES[compute]
        rmode = kh.RZ if narrowing and rng.randint(3) == 0 and not (compute == kh.BF16 and out_dtype in (kh.F8E4M3, kh.F8E5M2)) else kh.RN
        insts.append(dict(op=CAST, dst=15, a=last, dtype=out_dtype, rmode=rmode))
        last = 15
    insts.append(dict(op=ST, a=last))
    out_kind = "T" if rng.randint(4) == 0 else "full"
    return m, n, insts, kinds, in_dtypes, out_dtype, out_kind


def _layout(kind, m, n):
    return {"full": (m, n, n, 1, m * n), "T": (m, n, 1, m, m * n), "row": (1, n, n, 1, n), "col": (m, 1, 1, 1, m), "scalar": (1, 1, 1, 1, 1)}[kind]


def _same(got, want, dtype):
    if dtype == kh.F32:
        g, w = got.view(np.float32), want.view(np.float32)
        nan = np.isnan(w)
        return np.array_equal(np.isnan(g), nan) and np.array_equal(got[~nan], want[~nan])
    if dtype in (kh.F16, kh.BF16):
        is_nan = (lambda a: (a & 0x7fff) > 0x7c00) if dtype == kh.F16 else (lambda a: (a & 0x7fff) > 0x7f80)
        nan = is_nan(want)
        return np.array_equal(is_nan(got), nan) and np.array_equal(got[~nan], want[~nan])
    is_nan = (lambda a: (a & 0x7f) == 0x7f) if dtype == kh.F8E4M3 else (lambda a: (a & 0x7f) > 0x7c)     # (the sign of a NaN is not part of the result)
    nan = is_nan(want)
    return np.array_equal(is_nan(got), nan) and np.array_equal(got[~nan], want[~nan])


@pytest.mark.parametrize("seed", list(range(100)) + [212])      # (98 and 212 once differed: min(+0, -0) in the oracle, an fma folded into the cast after it)
def test_random_exact_program(ko, seed):
    rng = np.random.RandomState(1000 + seed)
    m, n, insts, kinds, in_dtypes, out_dtype, out_kind = _random_case(rng)
    arrays, o_ins, d_ins, devs = [], [], [], []
    for k, (kind, dt) in enumerate(zip(kinds, in_dtypes)):
        r, c, s0, s1, count = _layout(kind, m, n)
        a = ko.fill_uniform(count, dt, seed, k, -4.0, 4.0) if dt in (kh.F8E4M3, kh.F8E5M2) else ko.fill_normal(count, dt, seed, k, 0.0, 2.0)
        arrays.append(a)
        devs.append(to_dev(a))
        o_ins.append(ko.mk_global(a, r, c, s0, s1, dt))
        d_ins.append(dglobal(devs[-1], r, c, s0, s1, dt))
    r, c, s0, s1, count = _layout(out_kind, m, n)
    outb = kh.DTYPE_BYTES[out_dtype]
    want = np.zeros(count, NP_OF[outb])
    rc = ko.elementwise(ko.program(insts), o_ins, ko.mk_global(want, r, c, s0, s1, out_dtype))
    assert rc == 0, "the oracle refuses the program: %s" % insts
    prog = kh.program(insts)
    describe = "seed %d: %dx%d kinds %s dtypes %s -> %s %s, program %s" % (seed, m, n, kinds, in_dtypes, out_dtype, out_kind, insts)
    dout = dev_zeros(count, outb)
    kh.elementwise(prog, d_ins, dglobal(dout, r, c, s0, s1, out_dtype))
    sync()
    assert _same(to_host(dout, NP_OF[outb]), want, out_dtype), "machines differ from the oracle; " + describe
    try:
        kh.elementwise_specialize(prog, d_ins, dglobal(dout, r, c, s0, s1, out_dtype))
    except kh.KapyError as e:
        assert e.status == kh.ERR_UNSUPPORTED, describe
        return                                   # (e.g. an fp8 column-major operand whose extent is not a multiple of 16)
    dout2 = dev_zeros(count, outb)
    kh.elementwise(prog, d_ins, dglobal(dout2, r, c, s0, s1, out_dtype))
    sync()
    assert _same(to_host(dout2, NP_OF[outb]), want, out_dtype), "the compiled kernel differs from the oracle; " + describe


@pytest.mark.parametrize("seed", range(40))
def test_random_exact_program_with_column_maxima(ko, seed):
    """The same random programs with two dependent reduces along axis 0 put before the store: t = min(v, max_col(u)),
    result = t - max_col(t).  A maximum is exact in any order, so the column machine must match the oracle bit for bit."""
    rng = np.random.RandomState(5000 + seed)
    m, n, insts, kinds, in_dtypes, out_dtype, out_kind = _random_case(rng)
    tail = []
    while insts[-1]["op"] in (ST, CAST) and (insts[-1]["op"] == ST or insts[-1]["dst"] == 15):
        tail.insert(0, insts.pop())
    v = tail[0]["a"]                                                           # the value the program was going to cast / store
    u = insts[rng.randint(len(insts))]["dst"]
    insts += [dict(op=kh.EW_REDUCE_MAX, dst=13, a=u, b=0), dict(op=kh.EW_MINIMUMF, dst=14, a=v, b=13),
              dict(op=kh.EW_REDUCE_MAX, dst=13, a=14, b=0), dict(op=kh.EW_SUBF, dst=14, a=14, b=13)]
    tail[0] = dict(tail[0], a=14)
    insts += tail
    arrays, o_ins, d_ins, devs = [], [], [], []
    for k, (kind, dt) in enumerate(zip(kinds, in_dtypes)):
        r, c, s0, s1, count = _layout(kind, m, n)
        a = ko.fill_uniform(count, dt, seed, k, -4.0, 4.0) if dt in (kh.F8E4M3, kh.F8E5M2) else ko.fill_normal(count, dt, seed, k, 0.0, 2.0)
        arrays.append(a)                       # (the oracle's descriptor holds a bare pointer: the array has to outlive it)
        devs.append(to_dev(a))
        o_ins.append(ko.mk_global(a, r, c, s0, s1, dt))
        d_ins.append(dglobal(devs[-1], r, c, s0, s1, dt))
    r, c, s0, s1, count = _layout(out_kind, m, n)
    outb = kh.DTYPE_BYTES[out_dtype]
    want = np.zeros(count, NP_OF[outb])
    assert ko.elementwise(ko.program(insts), o_ins, ko.mk_global(want, r, c, s0, s1, out_dtype)) == 0, "the oracle refuses the program: %s" % insts
    dout = dev_zeros(count, outb)
    kh.elementwise(kh.program(insts), d_ins, dglobal(dout, r, c, s0, s1, out_dtype))
    sync()
    assert _same(to_host(dout, NP_OF[outb]), want, out_dtype), "seed %d: %dx%d kinds %s dtypes %s -> %s %s, program %s" % (
        seed, m, n, kinds, in_dtypes, out_dtype, out_kind, insts)
