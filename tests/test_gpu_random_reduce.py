"""Seeded random kapy.reduce calls and batched layout moves: random extents (multiples of the vector widths and not), both
axes, sum and max, row- or column-major windows into larger buffers with pitches that keep or break 16-byte alignment, every
pairing of f16 / bf16 / f32 source and result.  max is bit-exact against the oracle; sum is accumulated in fp32 on the device
and in double by the oracle, so it is held to the fp32 accumulation bound plus one rounding of the result's type.  Nothing
outside the result window may change."""
import ctypes as C

import numpy as np
import pytest

import kapy_hip as kh
from gpu_util import dglobal, sync, to_dev, to_host

pytestmark = pytest.mark.gpu
NP = {1: np.uint8, 2: np.uint16, 4: np.uint32}
VALUE = {kh.F16: np.uint16, kh.BF16: np.uint16, kh.F32: np.float32}     # the storage type the oracle's decode expects
EPS = {kh.F16: 2.0 ** -11, kh.BF16: 2.0 ** -8, kh.F32: 2.0 ** -24}
INF = {kh.F16: 0x7c00, kh.BF16: 0x7f80, kh.F32: np.inf}     # as an element of the array ko.fill_normal returns for the type
SHAPES = [(2, 256), (64, 1000), (300, 128), (1024, 64), (37, 2048), (5, 520), (1000, 96), (130, 50), (1, 4096), (256, 1),
          (33, 33), (8, 512), (512, 8), (96, 1536), (2048, 32), (7, 7)]


def _window(rng, rows, cols, itemsize):
    """(buffer elements, offset, strides) of a rows x cols window, row- or column-major, pitch >= extent."""
    col_major = rng.randint(3) == 0
    lead, other = (rows, cols) if col_major else (cols, rows)
    pitch = lead + [0, 0, 8, 16 // itemsize, 3, 1][rng.randint(6)]
    offset = [0, 0, 16 // itemsize, 5][rng.randint(4)]
    return offset + pitch * other + 8, offset, ((1, pitch) if col_major else (pitch, 1))


@pytest.mark.parametrize("seed", range(64))
def test_random_reduce(ko, seed):
    rng = np.random.RandomState(9000 + seed)
    sdt = [kh.F16, kh.BF16, kh.F32][rng.randint(3)]
    ddt = [kh.F32, sdt, kh.F16, kh.BF16][rng.randint(4)]
    sb, db = kh.DTYPE_BYTES[sdt], kh.DTYPE_BYTES[ddt]
    m, n = SHAPES[rng.randint(len(SHAPES))]
    axis, kind = int(rng.randint(2)), int(rng.randint(2))
    om, on = (m, 1) if axis == 1 else (1, n)
    s_count, s_off, s_str = _window(rng, m, n, sb)
    d_count, d_off, d_str = _window(rng, om, on, db)
    scale = [1.0, 0.05, 30.0][rng.randint(3)]
    src = ko.fill_normal(s_count, sdt, 9000 + seed, 0, 0.0, scale)
    fill = 0x5A5A5A5A & (2 ** (8 * db) - 1)
    want = np.full(d_count, fill, NP[db])
    so = ko.mk_global(src[s_off:], m, n, s_str[0], s_str[1], sdt)
    do = ko.mk_global(want[d_off:], om, on, d_str[0], d_str[1], ddt)
    describe = "seed %d: %s of dtype %d -> %d, %dx%d along axis %d, src strides %s offset %d, dst strides %s offset %d" % (
        seed, "max" if kind else "sum", sdt, ddt, m, n, axis, s_str, s_off, d_str, d_off)
    assert ko.lib().ko_reduce(C.byref(so), C.byref(do), axis, kind) == 0, describe
    d_src, d_dst = to_dev(src), to_dev(np.full(d_count, fill, NP[db]))
    kh.reduce(dglobal(d_src, m, n, s_str[0], s_str[1], sdt, dynamic_offset=s_off),
              dglobal(d_dst, om, on, d_str[0], d_str[1], ddt, dynamic_offset=d_off), axis, kind)
    sync()
    got = to_host(d_dst, NP[db])
    inside = np.zeros(d_count, bool)
    idx = d_off + (np.arange(om)[:, None] * d_str[0] + np.arange(on)[None, :] * d_str[1]).ravel()
    inside[idx] = True
    assert np.array_equal(got[~inside], want[~inside]), describe + ": wrote outside the result window"
    if kind == 1:
        bad = np.flatnonzero(got != want)
        assert len(bad) == 0, "%s: %d results differ, first at %d (got %#x want %#x)" % (describe, len(bad), bad[0], got[bad[0]], want[bad[0]])
        return
    g = ko.decode(got[idx].view(VALUE[ddt]), ddt)
    w = ko.decode(want[idx].view(VALUE[ddt]), ddt)
    # the magnitude the accumulation error scales with: sum of |x| along the reduced axis
    vals = np.abs(ko.decode(src.view(VALUE[sdt]), sdt))
    sidx = s_off + np.arange(m)[:, None] * s_str[0] + np.arange(n)[None, :] * s_str[1]
    mass = vals[sidx].sum(axis=axis).ravel()
    bound = 2.0 ** -22 * mass + 2.0 * EPS[ddt] * np.abs(w) + 1e-30
    worst = np.argmax(np.abs(g - w) - bound)
    assert np.all(np.abs(g - w) <= bound), "%s: result %d is %r, oracle %r, bound %g" % (describe, worst, g[worst], w[worst], bound[worst])


@pytest.mark.parametrize("dtype", [kh.F16, kh.BF16, kh.F32])
@pytest.mark.parametrize("m,n,axis", [(64, 1024, 1), (16, 520, 1), (300, 128, 0), (1024, 64, 0), (8, 40, 1), (33, 33, 0)])
def test_reduce_of_lines_with_nan_infinities_and_signed_zeros(ko, dtype, m, n, axis):
    """Lines holding a NaN, +inf, -inf, only -0, and -0 next to +0 under negative values: max and sum treat them as the ops they
    fold with do (maximumf: NaN wins, -0 below +0; addf: inf - inf is NaN).  Bit-exact for max and for the special results."""
    rng = np.random.RandomState(m * 131 + n)
    x = rng.normal(0, 1, (m, n)).astype(np.float32)
    lines = x if axis == 1 else x.T                  # a view: line k is reduced to result k
    lines[1, 3] = np.nan
    lines[2, :] = -0.0
    lines[3, 5] = np.inf
    lines[4, 6], lines[4, 7] = np.inf, -np.inf
    lines[5, 7] = -np.inf
    lines[6, :] = -np.abs(lines[6, :]) - 1
    lines[6, 1], lines[6, 2] = -0.0, 0.0
    lines[7, :] = -np.abs(lines[7, :]) - 1
    lines[7, 1], lines[7, 2] = 0.0, -0.0
    store = np.ascontiguousarray((x.view(np.uint32) >> 16).astype(np.uint16) if dtype == kh.BF16 else
                                 x.astype(np.float16).view(np.uint16) if dtype == kh.F16 else x.view(np.uint32))
    om, on = (m, 1) if axis == 1 else (1, n)
    dx = to_dev(store)
    for kind in (0, 1):
        want = np.zeros(om * on, np.uint32)
        assert ko.lib().ko_reduce(C.byref(ko.mk_global(store, m, n, n, 1, dtype)), C.byref(ko.mk_global(want, om, on, 1, om, ko.F32)), axis, kind) == 0
        dd = to_dev(np.zeros(om * on, np.uint32))
        kh.reduce(dglobal(dx, m, n, n, 1, dtype), dglobal(dd, om, on, 1, om, kh.F32), axis, kind)
        sync()
        got = to_host(dd, np.uint32)
        gf, wf = got.view(np.float32), want.view(np.float32)
        assert np.array_equal(np.isnan(gf), np.isnan(wf)) and np.isnan(wf[1]) and (kind == 1 or np.isnan(wf[4]))
        exact = ~np.isnan(wf) & (~np.isfinite(wf) | (wf == 0) | (kind == 1))
        assert np.array_equal(got[exact], want[exact]), (kind, np.flatnonzero(exact & (got != want))[:5])
        assert np.allclose(gf[~np.isnan(wf) & ~exact], wf[~np.isnan(wf) & ~exact], rtol=1e-5, atol=1e-3)
        if axis == 1 and n % 8 == 0:
            # the same reduce as an instruction of a row program (its result on every element of the row, in the row's type)
            prog = [dict(op=kh.EW_LD_GLOBAL, dst=0, a=0), dict(op=kh.EW_REDUCE_MAX if kind else kh.EW_REDUCE_SUM, dst=1, a=0, b=1),
                    dict(op=kh.EW_ST_GLOBAL, a=1)]
            pw = np.zeros(m * n, store.dtype)
            assert ko.elementwise(ko.program(prog), [ko.mk_global(store, m, n, n, 1, dtype)], ko.mk_global(pw, m, n, n, 1, dtype)) == 0
            dp = to_dev(np.zeros(m * n, store.dtype))
            kh.elementwise(kh.program(prog), [dglobal(dx, m, n, n, 1, dtype)], dglobal(dp, m, n, n, 1, dtype))
            sync()
            pg = to_host(dp, store.dtype)
            pgf, pwf = ko.decode(pg.view(VALUE[dtype]), dtype), ko.decode(pw.view(VALUE[dtype]), dtype)
            assert np.array_equal(np.isnan(pgf), np.isnan(pwf))
            exact = ~np.isnan(pwf) & (~np.isfinite(pwf) | (pwf == 0) | (kind == 1))
            assert np.array_equal(pg[exact], pw[exact]), (kind, np.flatnonzero(exact & (pg != pw))[:5])
            rest = ~np.isnan(pwf) & ~exact
            assert np.all(np.abs(pgf[rest] - pwf[rest]) <= 2 * EPS[dtype] * np.abs(pwf[rest]) + 1e-3)


@pytest.mark.parametrize("dtype", [kh.F16, kh.BF16, kh.F32])
@pytest.mark.parametrize("m,n", [(100000, 64), (20000, 200), (5000, 4096), (4097, 72), (300000, 8), (129, 8192), (70000, 4), (3000, 36)])
def test_reduce_along_axis0_of_tall_matrices(ko, dtype, m, n):
    """Few kept indices and many reduced ones: the reduced axis is shared out over workgroups, whose fp32 partial lines a second
    pass folds in a fixed order.  max bit-exact, sum within the fp32 accumulation bound, twice with the same bits, and the
    result type's rounding when the result is 16-bit."""
    x = ko.fill_normal(m * n, dtype, 77 + n, 0)
    x.reshape(m, n)[m // 3, 3] = INF[dtype]   # one +inf: its column sums and maximises to +inf
    dx = to_dev(x)
    for kind in (0, 1):
        for ddt in (kh.F32, dtype):
            db = kh.DTYPE_BYTES[ddt]
            want = np.zeros(n, NP[db])
            assert ko.lib().ko_reduce(C.byref(ko.mk_global(x, m, n, n, 1, dtype)), C.byref(ko.mk_global(want, 1, n, n, 1, ddt)), 0, kind) == 0
            runs = []
            for _ in range(2):
                dd = to_dev(np.full(n + 16, 0x5A5A, NP[db]))
                kh.reduce(dglobal(dx, m, n, n, 1, dtype), dglobal(dd, 1, n, n, 1, ddt), 0, kind)
                sync()
                runs.append(to_host(dd, NP[db]))
            got = runs[0]
            assert np.array_equal(runs[0], runs[1]) and np.all(got[n:] == 0x5A5A)
            got = got[:n]
            if kind == 1:
                assert np.array_equal(got, want)
                continue
            g, w = ko.decode(got.view(VALUE[ddt]), ddt), ko.decode(want.view(VALUE[ddt]), ddt)
            assert np.isinf(w[3]) and g[3] == w[3]
            mass = np.abs(ko.decode(x.view(VALUE[dtype]), dtype)).reshape(m, n).sum(axis=0)
            rest = np.isfinite(w)
            assert np.all(np.abs(g[rest] - w[rest]) <= (2.0 ** -22 * mass + 2.0 * EPS[ddt] * np.abs(w) + 1e-30)[rest])


@pytest.mark.parametrize("dtype", [kh.F16, kh.BF16, kh.F32])
@pytest.mark.parametrize("m,n", [(100000, 64), (30000, 200), (1000, 512), (7, 8), (4099, 24), (3, 1 << 20), (64, 65536), (5, 40000), (300, 16384), (5000, 4), (900, 260)])
def test_reduce_along_axis1_of_short_and_of_few_long_lines(ko, dtype, m, n):
    """Lines of up to 512 elements share a wave; few long lines are shared out over workgroups in chunks whose fp32 partial
    results a second launch folds.  max bit-exact, sum within the fp32 accumulation bound, twice with the same bits."""
    x = ko.fill_normal(m * n, dtype, 79 + n, 0)
    x.reshape(m, n)[m // 2, n // 3] = INF[dtype]
    dx = to_dev(x)
    for kind in (0, 1):
        for ddt in (kh.F32, dtype):
            db = kh.DTYPE_BYTES[ddt]
            want = np.zeros(m, NP[db])
            assert ko.lib().ko_reduce(C.byref(ko.mk_global(x, m, n, n, 1, dtype)), C.byref(ko.mk_global(want, m, 1, 1, 1, ddt)), 1, kind) == 0
            runs = []
            for _ in range(2):
                dd = to_dev(np.full(m + 16, 0x5A5A, NP[db]))
                kh.reduce(dglobal(dx, m, n, n, 1, dtype), dglobal(dd, m, 1, 1, 1, ddt), 1, kind)
                sync()
                runs.append(to_host(dd, NP[db]))
            got = runs[0]
            assert np.array_equal(runs[0], runs[1]) and np.all(got[m:] == 0x5A5A)
            got = got[:m]
            if kind == 1:
                assert np.array_equal(got, want)
                continue
            g, w = ko.decode(got.view(VALUE[ddt]), ddt), ko.decode(want.view(VALUE[ddt]), ddt)
            assert np.isinf(w[m // 2]) and g[m // 2] == w[m // 2]
            mass = np.abs(ko.decode(x.view(VALUE[dtype]), dtype)).reshape(m, n).sum(axis=1)
            rest = np.isfinite(w)
            assert np.all(np.abs(g[rest] - w[rest]) <= (2.0 ** -22 * mass + 2.0 * EPS[ddt] * np.abs(w) + 1e-30)[rest])


def test_tall_reduces_on_two_streams_with_a_workspace_each():
    """Launches that share a reduced axis out over workgroups meet in a workspace; calls that may overlap in time (two streams)
    get one each.  Every result has the same bits as the call made alone on the library's own array."""
    import torch
    m, n = 60000, 64
    xs = [torch.randn(m, n, device="cuda").half() for _ in range(6)]
    alone = []
    for x in xs:
        d = torch.zeros(n, device="cuda", dtype=torch.float32)
        kh.reduce(dglobal(x, m, n, n, 1, kh.F16), dglobal(d, 1, n, n, 1, kh.F32), 0, 0)
        sync()
        alone.append(d.clone())
    streams = [torch.cuda.Stream(), torch.cuda.Stream()]
    spaces = [torch.zeros(kh.lib().kapy_reduce_workspace_bytes(), dtype=torch.uint8, device="cuda") for _ in streams]
    sync()
    for st in streams:
        st.wait_stream(torch.cuda.current_stream())
    for rep in range(5):
        outs = [torch.zeros(n, device="cuda", dtype=torch.float32) for _ in xs]
        for k, (x, d) in enumerate(zip(xs, outs)):
            with torch.cuda.stream(streams[k % 2]):
                kh.reduce_ex(dglobal(x, m, n, n, 1, kh.F16), dglobal(d, 1, n, n, 1, kh.F32), 0, kh.REDUCE_ADDF, workspace=spaces[k % 2],
                             stream=streams[k % 2].cuda_stream)
        for st in streams:
            st.synchronize()
        for d, a in zip(outs, alone):
            assert torch.equal(d, a)
    for ws in spaces:
        assert not ws[:16384].any()                    # the arrival counters are back at zero


def test_a_captured_reduce_equals_the_eager_call():
    """Nothing about the call depends on the stream being captured: the graph's replays give the eager call's bits."""
    import torch
    for m, n, axis in ((60000, 64, 0), (8192, 2048, 0), (64, 262144, 1)):
        x = torch.randn(m, n, device="cuda").half()
        k = n if axis == 0 else m
        shape, strides = ((1, n), (n, 1)) if axis == 0 else ((m, 1), (1, m))
        eager = torch.zeros(k, device="cuda", dtype=torch.float32)
        kh.reduce(dglobal(x, m, n, n, 1, kh.F16), dglobal(eager, shape[0], shape[1], strides[0], strides[1], kh.F32), axis, 0)
        sync()
        out = torch.zeros(k, device="cuda", dtype=torch.float32)
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.stream(side):
            with torch.cuda.graph(graph, stream=side):
                kh.reduce(dglobal(x, m, n, n, 1, kh.F16), dglobal(out, shape[0], shape[1], strides[0], strides[1], kh.F32), axis, 0, stream=side.cuda_stream)
        for rep in range(3):
            out.fill_(-1.0)
            sync()
            graph.replay()
            sync()
            assert torch.equal(out, eager), (m, n, axis, rep)


FLOAT_KINDS = [kh.REDUCE_ADDF, kh.REDUCE_MAXIMUMF, kh.REDUCE_MINIMUMF, kh.REDUCE_MULF, kh.REDUCE_MAXNUMF, kh.REDUCE_MINNUMF]


@pytest.mark.parametrize("dtype", [kh.F16, kh.BF16, kh.F32])
@pytest.mark.parametrize("m,n,axis", [(64, 1024, 1), (16, 520, 1), (4, 262144, 1), (300, 128, 0), (20000, 64, 0), (4096, 2048, 0), (33, 33, 0), (7, 100, 1)])
def test_every_float_combiner_on_every_kernel_shape(ko, dtype, m, n, axis):
    """minimumf, mulf, maxnumf and minnumf beside addf and maximumf, through the short-line, long-line, shared-out, strip and
    element kernels; lines with NaNs for the four orderings (bit-exact), products of values near one."""
    x = ko.fill_normal(m * n, dtype, 700 + m + n, 0, 0.0, 1.0).reshape(m, n)
    nan = {kh.F16: 0x7e00, kh.BF16: 0x7fc0, kh.F32: np.float32(np.nan)}[dtype]
    rng = np.random.default_rng(m)
    if dtype == kh.F32:
        x = x.copy()
    x[rng.integers(0, m), rng.integers(0, n)] = nan
    if axis == 1:
        x[m // 2, :] = nan
    else:
        x[:, n // 2] = nan
    sb = kh.DTYPE_BYTES[dtype]
    om, on = (m, 1) if axis == 1 else (1, n)
    for kind in FLOAT_KINDS:
        src = x
        if kind in (kh.REDUCE_ADDF, kh.REDUCE_MULF):                      # finite operands; products of 1 + small
            src = ko.fill_normal(m * n, dtype, 800 + m, 0, 1.0 if kind == kh.REDUCE_MULF else 0.0, 2.0 ** -9 if kind == kh.REDUCE_MULF else 1.0).reshape(m, n)
        want = np.zeros(om * on, NP[sb])
        assert ko.lib().ko_reduce(C.byref(ko.mk_global(src, m, n, n, 1, dtype)), C.byref(ko.mk_global(want, om, on, on, 1, dtype)), axis, kind) == 0
        d_dst = to_dev(np.zeros(om * on, NP[sb]))
        kh.reduce_ex(dglobal(to_dev(src), m, n, n, 1, dtype), dglobal(d_dst, om, on, on, 1, dtype), axis, kind)
        sync()
        got = to_host(d_dst, NP[sb])
        if kind in (kh.REDUCE_ADDF, kh.REDUCE_MULF):
            g, w = ko.decode(got.view(VALUE[dtype]), dtype), ko.decode(want.view(VALUE[dtype]), dtype)
            scale = np.abs(ko.decode(src.view(VALUE[dtype]), dtype)).sum(axis=axis).ravel() if kind == kh.REDUCE_ADDF else np.abs(w)
            n_red = n if axis == 1 else m          # a product's rounding errors add up along the line (about their square root on random data)
            rel = 8.0 * np.sqrt(n_red) * 2.0 ** -24 if kind == kh.REDUCE_MULF else 2.0 ** -22
            assert np.all(np.abs(g - w) <= rel * scale + 2.0 * EPS[dtype] * np.abs(w) + 1e-30), kind
        else:
            gv, wv = got.view(VALUE[dtype]), want.view(VALUE[dtype])
            same = gv == wv
            if dtype == kh.F32:
                same |= np.isnan(gv) & np.isnan(wv)
            else:
                both_nan = (ko.decode(gv, dtype) != ko.decode(gv, dtype)) & (ko.decode(wv, dtype) != ko.decode(wv, dtype))
                same |= both_nan
            assert np.all(same), "combiner %d: %d results differ" % (kind, int((~same).sum()))


@pytest.mark.parametrize("dt,np_t", [(kh.I8, np.int8), (kh.I16, np.int16), (kh.I32, np.int32)])
@pytest.mark.parametrize("m,n,axis", [(37, 53, 0), (37, 53, 1), (3000, 64, 0), (8, 5000, 1)])
def test_integer_combiners_are_bit_exact(ko, dt, np_t, m, n, axis):
    rng = np.random.default_rng(m + n + axis)
    info = np.iinfo(np_t)
    x = rng.integers(info.min, info.max + 1, size=(m, n), dtype=np.int64).astype(np_t)
    om, on = (m, 1) if axis == 1 else (1, n)
    for kind in range(kh.REDUCE_ADDI, kh.REDUCE_XORI + 1):
        want = np.zeros((om, on), np_t)
        assert ko.lib().ko_reduce(C.byref(ko.mk_global(x, m, n, n, 1, dt)), C.byref(ko.mk_global(want, om, on, on, 1, dt)), axis, kind) == 0
        d_dst = to_dev(np.zeros(om * on, np_t))
        kh.reduce_ex(dglobal(to_dev(x), m, n, n, 1, dt), dglobal(d_dst, om, on, on, 1, dt), axis, kind)
        sync()
        assert np.array_equal(to_host(d_dst, np_t, (om, on)), want), kind


@pytest.mark.parametrize("dtype", [kh.F16, kh.BF16, kh.F32])
@pytest.mark.parametrize("shape,axis,loops,row_major", [((2, 256), 1, None, True), ((4, 512), 1, (1, 8), True), ((64, 8), 0, (1, 1), False),
                                                          ((128, 16), 0, (2, 1), False), ((16, 64), 1, (1, 2), True), ((32, 32), 0, (1, 1), True),
                                                          ((1, 4096), 1, (1, 4), True)])
def test_reference_arithmetic_equals_the_checker_bit_for_bit(ko, dtype, shape, axis, loops, row_major):
    """KAPY_REDUCE_REFERENCE: partial results rounded to the element type, lane-serial fold then butterfly, on a wavefront's tile
    under a given fragments layout (None: the default one) - the same bits as the checker's walk of that order, for sums (where
    the order shows), maxima and an integer fold."""
    m, n = shape
    lay = None
    klay = None
    if loops is not None:
        lay = ko.Fragments()
        ko.lib().ko_fragments_default((C.c_int64 * 2)(*loops), (C.c_int64 * 2)(*shape), 1 if row_major else 0, 64, C.byref(lay))
        klay = kh.Fragments.make([lay.lane_array[0], lay.lane_array[1]], [lay.lane_loops[0], lay.lane_loops[1]], lay.minor_axis, lay.major_axis)
    sb = kh.DTYPE_BYTES[dtype]
    om, on = (m, 1) if axis == 1 else (1, n)
    x = ko.fill_normal(m * n, dtype, 900 + m, 0, 0.0, 30.0).reshape(m, n)
    differs = 0
    for kind in (kh.REDUCE_ADDF, kh.REDUCE_MAXIMUMF, kh.REDUCE_MULF):
        src = x if kind != kh.REDUCE_MULF else ko.fill_normal(m * n, dtype, 901, 0, 1.0, 0.01).reshape(m, n)
        want, wide = np.zeros(om * on, NP[sb]), np.zeros(om * on, NP[sb])
        g, o = ko.mk_global(src, m, n, n, 1, dtype), ko.mk_global(want, om, on, on, 1, dtype)
        assert ko.lib().ko_reduce_reference(C.byref(g), C.byref(o), axis, kind, C.byref(lay) if lay is not None else None, 64) == 0
        assert ko.lib().ko_reduce(C.byref(g), C.byref(ko.mk_global(wide, om, on, on, 1, dtype)), axis, kind) == 0
        d_dst = to_dev(np.zeros(om * on, NP[sb]))
        kh.reduce_ex(dglobal(to_dev(src), m, n, n, 1, dtype), dglobal(d_dst, om, on, on, 1, dtype), axis, kind, arithmetic=kh.REDUCE_REFERENCE, layout=klay)
        sync()
        assert np.array_equal(to_host(d_dst, NP[sb]), want), kind
        differs += int((want != wide).sum())
    if dtype != kh.F32 and max(m, n) >= 256:
        assert differs > 0        # 16-bit partial sums are not the once-rounded sum: the mode is not a no-op
    xi = (np.arange(m * n, dtype=np.int64).reshape(m, n) * 2654435761 % 65521 - 30000).astype(np.int16)
    want = np.zeros((om, on), np.int16)
    assert ko.lib().ko_reduce_reference(C.byref(ko.mk_global(xi, m, n, n, 1, kh.I16)), C.byref(ko.mk_global(want, om, on, on, 1, kh.I16)), axis, kh.REDUCE_ADDI,
                                        C.byref(lay) if lay is not None else None, 64) == 0
    d_dst = to_dev(np.zeros(om * on, np.int16))
    kh.reduce_ex(dglobal(to_dev(xi), m, n, n, 1, kh.I16), dglobal(d_dst, om, on, on, 1, kh.I16), axis, kh.REDUCE_ADDI, arithmetic=kh.REDUCE_REFERENCE, layout=klay)
    sync()
    assert np.array_equal(to_host(d_dst, np.int16, (om, on)), want) and np.array_equal(want.ravel(), xi.astype(np.int64).sum(axis=axis).astype(np.int16))


def test_reduce_refusals():
    import torch
    x = torch.zeros(64 * 64, device="cuda", dtype=torch.int32)
    g = lambda m, n, dt: dglobal(x, m, n, n, 1, dt)
    for args, kw, words in (((g(64, 64, kh.F16), g(64, 1, kh.F16), 1, 15), {}, "unknown combiner"),
                            ((g(64, 64, kh.F16), g(64, 1, kh.F16), 1, kh.REDUCE_ADDI), {}, "integer combiner"),
                            ((g(64, 64, kh.I32), g(64, 1, kh.I32), 1, kh.REDUCE_ADDF), {}, "float combiner"),
                            ((g(64, 64, kh.I32), g(64, 1, kh.I16), 1, kh.REDUCE_ADDI), {}, "one type"),
                            ((g(48, 64, kh.F16), g(48, 1, kh.F16), 1, kh.REDUCE_ADDF), dict(arithmetic=kh.REDUCE_REFERENCE), "power-of-two"),
                            ((g(64, 64, kh.F16), g(64, 1, kh.F32), 1, kh.REDUCE_ADDF), dict(arithmetic=kh.REDUCE_REFERENCE), "source's element type")):
        with pytest.raises(kh.KapyError) as e:
            kh.reduce_ex(*args, **kw)
        assert words in e.value.message, e.value.message


@pytest.mark.parametrize("seed", range(32))
def test_random_batched_copy(ko, seed):
    """A b x h grid of tiles moved between two 4-D layouts (any of the two orders of the grid axes on either side), with or
    without a transpose of the tile itself: bit-exact against the oracle and against numpy's transpose of the same array."""
    rng = np.random.RandomState(9500 + seed)
    dtype = [kh.F16, kh.BF16, kh.F32, kh.F8E4M3][rng.randint(4)]
    eb = kh.DTYPE_BYTES[dtype]
    b, h = int(rng.randint(1, 4)), int(rng.randint(1, 6))
    s, d = [(40, 64), (64, 64), (17, 24), (128, 32), (33, 128), (8, 8), (100, 16)][rng.randint(7)]
    transpose = bool(rng.randint(2))
    src_bhsd, dst_bhsd = bool(rng.randint(2)), bool(rng.randint(2))
    ds, dd_ = (d, s) if transpose else (s, d)
    src = rng.randint(0, 2 ** (8 * min(eb, 4) - (1 if eb == 4 else 0)), size=b * h * s * d).astype(NP[eb])

    def layout(bhsd, rows, cols):
        """(row stride, offsets along b and h) of a [b,h,rows,cols] (bhsd) or [b,rows,h,cols] array."""
        return (cols, h * rows * cols, rows * cols) if bhsd else (h * cols, rows * h * cols, cols)

    s_row, s_b, s_h = layout(src_bhsd, s, d)
    d_row, d_b, d_h = layout(dst_bhsd, ds, dd_)
    describe = "seed %d: dtype %d grid %dx%d tile %dx%d%s, source %s, result %s" % (
        seed, dtype, b, h, s, d, " transposed" if transpose else "", "bhsd" if src_bhsd else "bshd", "bhsd" if dst_bhsd else "bshd")
    want = np.zeros(b * h * s * d, NP[eb])
    assert ko.lib().ko_copy_batched(C.byref(ko.mk_global(src, s, d, s_row, 1, dtype)), C.byref(ko.mk_global(want, ds, dd_, d_row, 1, dtype)),
                                    int(transpose), 0, b, h, s_b, s_h, d_b, d_h) == 0, describe
    d_src, d_dst = to_dev(src), to_dev(np.zeros(b * h * s * d, NP[eb]))
    kh.copy_batched(dglobal(d_src, s, d, s_row, 1, dtype), dglobal(d_dst, ds, dd_, d_row, 1, dtype), (b, h, s_b, s_h, d_b, d_h),
                    transpose=transpose)
    sync()
    got = to_host(d_dst, NP[eb])
    assert np.array_equal(got, want), describe
    a = src.reshape(b, h, s, d) if src_bhsd else src.reshape(b, s, h, d).transpose(0, 2, 1, 3)      # -> [b,h,s,d]
    if transpose:
        a = a.transpose(0, 1, 3, 2)
    expect = a if dst_bhsd else a.transpose(0, 2, 1, 3)
    assert np.array_equal(got.reshape(expect.shape), expect), describe + " (numpy transpose)"
