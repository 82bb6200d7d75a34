"""Pins the checker's kapy.reduce (Ops.td:441-457, ReduceOpToLLVM.cpp:51-172): every combiner against numpy on both axes, NaN and
signed-zero rules of the four float orderings, wrapping integer folds, and the lowering's own arithmetic and order (element-type
partial results, lane-serial fold, butterfly at ascending lane distances) against a hand-computed answer and an independent
numpy float16 walk of the same order."""
import ctypes as C

import numpy as np
import pytest


def _reduce(ko, x, dtype, axis, kind, out_dtype=None):
    m, n = x.shape
    out_dtype = dtype if out_dtype is None else out_dtype
    out = np.zeros((m, 1) if axis == 1 else (1, n), ko.NP_STORAGE[out_dtype])
    g = ko.mk_global(np.ascontiguousarray(x), m, n, n, 1, dtype)
    o = ko.mk_global(out, out.shape[0], out.shape[1], out.shape[1], 1, out_dtype)
    assert ko.lib().ko_reduce(C.byref(g), C.byref(o), axis, kind) == 0
    return out


@pytest.mark.parametrize("axis", [0, 1])
def test_float_combiners_against_numpy(ko, axis):
    rng = np.random.default_rng(axis)
    x = rng.standard_normal((37, 53)).astype(np.float32)
    xu = x.view(np.uint32)
    f = lambda a: a.view(np.float32).astype(np.float64)
    keep = dict(axis=axis, keepdims=True)
    assert np.allclose(f(_reduce(ko, xu, ko.F32, axis, 0)), x.astype(np.float64).sum(**keep), rtol=1e-6)
    assert np.array_equal(f(_reduce(ko, xu, ko.F32, axis, 1)), x.max(**keep))
    assert np.array_equal(f(_reduce(ko, xu, ko.F32, axis, 2)), x.min(**keep))
    small = (1.0 + 0.01 * x).astype(np.float32)
    assert np.allclose(f(_reduce(ko, small.view(np.uint32), ko.F32, axis, 3)), small.astype(np.float64).prod(**keep), rtol=1e-6)
    # NaN: maximumf / minimumf are poisoned, maxnumf / minnumf skip it unless the whole line is NaN
    y = x.copy()
    y[3, 5] = np.nan
    y[7, :] = np.nan
    y[:, 9] = np.nan
    yu = y.view(np.uint32)
    for kind, fn in ((1, np.max), (2, np.min)):
        assert np.array_equal(f(_reduce(ko, yu, ko.F32, axis, kind)), fn(y, **keep), equal_nan=True)
    for kind, fn in ((4, np.nanmax), (5, np.nanmin)):
        with np.errstate(all="ignore"), pytest.warns(RuntimeWarning):
            want = fn(y, **keep)
        assert np.array_equal(f(_reduce(ko, yu, ko.F32, axis, kind)), want, equal_nan=True)


def test_signed_zero_and_once_rounded_sums(ko):
    z = np.array([[-0.0, 0.0, -0.0], [-0.0, -0.0, -0.0], [0.0, -0.0, 0.0]], np.float32)
    zu = z.view(np.uint32)
    sign = lambda a: np.signbit(a.view(np.float32)).ravel().tolist()
    assert sign(_reduce(ko, zu, ko.F32, 1, 1)) == [False, True, False]      # max: -0 below +0
    assert sign(_reduce(ko, zu, ko.F32, 1, 2)) == [True, True, True]        # min
    assert sign(_reduce(ko, zu, ko.F32, 1, 4)) == [False, True, False] and sign(_reduce(ko, zu, ko.F32, 1, 5)) == [True, True, True]
    assert sign(_reduce(ko, zu, ko.F32, 1, 0)) == [False, True, False]      # a line of only -0 sums to -0
    ones = np.full((1, 2056), 0x3C00, np.uint16)                            # 2056 ones in f16: the exact sum, rounded once, is 2056
    assert _reduce(ko, ones, ko.F16, 1, 0).view(np.float16)[0, 0] == 2056.0
    assert _reduce(ko, ones, ko.F16, 1, 0, ko.F32).view(np.float32)[0, 0] == 2056.0


@pytest.mark.parametrize("name,np_t", [("I8", np.int8), ("I16", np.int16), ("I32", np.int32)])
def test_integer_combiners_wrap(ko, name, np_t):
    rng = np.random.default_rng(11)
    info = np.iinfo(np_t)
    x = rng.integers(info.min, info.max + 1, size=(19, 23), dtype=np.int64).astype(np_t)
    dt = getattr(ko, name)
    bits = info.bits
    for axis in (0, 1):
        keep = dict(axis=axis, keepdims=True)
        wide = x.astype(np.int64)
        uns = wide & ((1 << bits) - 1)
        wrap = lambda v: (np.asarray(v, np.int64) & ((1 << bits) - 1)).astype(np.uint64).astype({8: np.uint8, 16: np.uint16, 32: np.uint32}[bits]).view(np_t)
        prod = np.ones_like(wide.sum(**keep))
        for k in range(x.shape[axis]):
            prod = (prod * np.take(wide, [k], axis=axis)) & 0xFFFFFFFF    # python-int free: stays within 64 bits
        want = {6: wrap(wide.sum(**keep)), 7: wrap(prod), 8: x.max(**keep), 9: x.min(**keep), 10: wrap(uns.max(**keep)), 11: wrap(uns.min(**keep)),
                12: np.bitwise_and.reduce(x, **keep), 13: np.bitwise_or.reduce(x, **keep), 14: np.bitwise_xor.reduce(x, **keep)}
        for kind, w in want.items():
            assert np.array_equal(_reduce(ko, x, dt, axis, kind), w), (kind, axis)


def _reference(ko, x, dtype, axis, kind, layout=None, lanes=64):
    m, n = x.shape
    out = np.zeros((m, 1) if axis == 1 else (1, n), ko.NP_STORAGE[dtype])
    g = ko.mk_global(np.ascontiguousarray(x), m, n, n, 1, dtype)
    o = ko.mk_global(out, out.shape[0], out.shape[1], out.shape[1], 1, dtype)
    assert ko.lib().ko_reduce_reference(C.byref(g), C.byref(o), axis, kind, C.byref(layout) if layout is not None else None, lanes) == 0
    return out


def test_reference_arithmetic_known_answer(ko):
    """f16 row of 256: 2048 followed by 255 ones, on 64 lanes (lane l holds columns l, l + 64, l + 128, l + 192).  Lane 0 folds
    2048 + 1 + 1 + 1 = 2048 in f16 (each 2049 is a tie that goes to the even 2048), every other lane 4; the butterfly then adds
    4, 8, 16, 32, 64, 128 - all exact: 2300.  The exact sum 2303 rounds to 2304."""
    x = np.full((1, 256), 0x3C00, np.uint16)
    x[0, 0] = np.float16(2048.0).view(np.uint16)
    assert _reference(ko, x, ko.F16, 1, 0).view(np.float16)[0, 0] == 2300.0
    assert _reduce(ko, x, ko.F16, 1, 0).view(np.float16)[0, 0] == 2304.0
    # the same line on 32 lanes (the reference's warp): lane 0 holds 8 elements, 2048 + 7 ones stays 2048; others 8 -> 2048 + 8 * 31 = 2296
    assert _reference(ko, x, ko.F16, 1, 0, lanes=32).view(np.float16)[0, 0] == 2296.0


@pytest.mark.parametrize("shape,axis,loops,row_major", [((2, 256), 1, (1, 1), True), ((4, 512), 1, (1, 8), True), ((64, 8), 0, (1, 1), False),
                                                          ((128, 16), 0, (2, 1), False), ((16, 64), 1, (1, 2), True), ((32, 32), 0, (1, 1), True)])
def test_reference_order_against_an_independent_walk(ko, shape, axis, loops, row_major):
    """numpy float16 arithmetic in the order ReduceOpToLLVM.cpp:76-119 spells out, over the element positions of the reference's
    own diagram rule (lane id contiguous along the major axis, `loops` consecutive elements per lane, tiles of the lane array
    repeated over the tensor)."""
    rng = np.random.default_rng(shape[0] * 7 + shape[1])
    x = (rng.standard_normal(shape) * 30.0).astype(np.float16)
    lay = ko.Fragments()
    fl = (C.c_int64 * 2)(*loops)
    sh = (C.c_int64 * 2)(*shape)
    ko.lib().ko_fragments_default(fl, sh, 1 if row_major else 0, 64, C.byref(lay))
    got = _reference(ko, x.view(np.uint16), ko.F16, axis, 0, layout=lay).view(np.float16)
    a0, a1 = lay.lane_array[0], lay.lane_array[1]
    l0, l1 = loops
    # which lane owns element (i, j), and in which order a lane meets its elements along the reduced axis: increasing index
    lane_of = lambda i, j: ((i % (a0 * l0)) // l0) * a1 + (j % (a1 * l1)) // l1 if row_major else ((i % (a0 * l0)) // l0) + ((j % (a1 * l1)) // l1) * a0
    n_keep, n_red = (shape[0], shape[1]) if axis == 1 else (shape[1], shape[0])
    lane_offset = 1 if (1 if row_major else 0) == axis else (a0 if axis == 1 else a1)
    for k in range(n_keep):
        acc = {}
        for r in range(n_red):
            i, j = (k, r) if axis == 1 else (r, k)
            ln = lane_of(i, j)
            acc[ln] = x[i, j] if ln not in acc else np.float16(acc[ln] + x[i, j])
        owners = sorted(acc)
        rounds = int(np.log2(len(owners)))
        for t in range(rounds):
            acc = {ln: np.float16(acc[ln] + acc[ln ^ (lane_offset << t)]) for ln in owners}
        want = acc[owners[0]]
        assert all(acc[ln] == want for ln in owners)      # the combiner commutes, so every lane of a butterfly ends with the same value
        g = got[k, 0] if axis == 1 else got[0, k]
        assert g == acc[lane_of(*((k, 0) if axis == 1 else (0, k)))], (k, g, want)
