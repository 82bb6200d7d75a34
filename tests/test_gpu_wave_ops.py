"""GPU parity for the cross-lane ops: kgpu.change (bit-exact re-layout) and kapy.reduce."""
import ctypes as C

import numpy as np
import pytest

import kapy_hip as kh
from gpu_util import dev_zeros, dglobal, sync, to_dev, to_host

pytestmark = pytest.mark.gpu


def _change_case(ko, src, dst, shape, seed=1):
    fs, fd = kh.Fragments.make(*src), kh.Fragments.make(*dst)
    os_, od = ko.Fragments.make(*src), ko.Fragments.make(*dst)
    s1, s2 = kh.A2(0, 0), kh.A2(0, 0)
    kh.lib().kapy_fragments_loops(C.byref(fs), kh.A2(*shape), kh.A2(0, 0), s1)
    kh.lib().kapy_fragments_loops(C.byref(fd), kh.A2(*shape), kh.A2(0, 0), s2)
    ns, nd = s1[0] * s1[1], s2[0] * s2[1]
    vals = np.random.default_rng(seed).integers(0, 2 ** 32, size=(64, ns), dtype=np.uint64).astype(np.uint32)
    # make the input a consistent distribution of one tile (replicated elements hold equal values)
    tile = np.random.default_rng(seed + 1000).integers(0, 2 ** 32, size=shape, dtype=np.uint64).astype(np.uint32)
    for lane in range(64):
        for iv in range(ns):
            o = kh.A2(0, 0)
            kh.lib().kapy_fragments_map(C.byref(fs), kh.A2(*shape), 1, kh.A2(lane, iv), o)
            vals[lane, iv] = tile[o[0], o[1]]
    want = np.zeros((64, nd), dtype=np.uint32)
    ko.lib().ko_change_tile(vals.ctypes.data_as(C.c_void_p), C.byref(os_), C.byref(od), kh.A2(*shape), 4, 64,
                            want.ctypes.data_as(C.c_void_p))
    din, dout = to_dev(vals), dev_zeros(64 * nd, 4)
    kh.change(din.data_ptr(), fs, fd, shape, dout.data_ptr())
    sync()
    got = to_host(dout, np.uint32, (64, nd))
    assert np.array_equal(got, want)
    # closed form: the value of the element the result layout places at (lane, iv).  Where that layout is larger than the
    # tensor, positions past the tensor's edge name no element (they hold a replica if the source layout reaches as far, zero
    # otherwise: the comparison with the oracle above covers them)
    for lane in (0, 17, 63):
        for iv in range(nd):
            o = kh.A2(0, 0)
            kh.lib().kapy_fragments_map(C.byref(fd), kh.A2(*shape), 2, kh.A2(lane, iv), o)
            inside = o[0] < shape[0] and o[1] < shape[1]
            assert not inside or got[lane, iv] == tile[o[0], o[1]], (lane, iv, o[0], o[1])



@pytest.mark.parametrize("src,dst,shape", [
    (([8, 8], [1, 2], 0, 1), ([16, 4], [1, 8], 0, 1), (16, 32)),
    (([2, 32], [4, 1], 0, 1), ([8, 8], [1, 4], 0, 1), (32, 32)),      # MFMA accumulator -> 8-byte store layout
    (([8, 8], [2, 2], 0, 1), ([8, 8], [2, 2], 1, 0), (16, 16)),       # exchange axes: a lane-grid transpose
    (([32, 2], [1, 8], 1, 0), ([8, 8], [4, 2], 0, 1), (32, 16)),       # MFMA lhs operand -> row-major 4x2 blocks
])
def test_change_matches_oracle(ko, src, dst, shape):
    _change_case(ko, src, dst, shape)


@pytest.mark.parametrize("seed", range(48))
def test_random_change(ko, seed):
    """Random pairs of fragments layouts over one wavefront (lane grid a0 x a1 = 64, 1-8 values per lane and axis, either axis
    minor) and random power-of-two tile shapes, tiles smaller than a layout's footprint (replicated elements) included."""
    rng = np.random.RandomState(12000 + seed)

    def layout():
        a0 = 1 << rng.randint(7)
        return ([a0, 64 // a0], [1 << rng.randint(3), 1 << rng.randint(3)]) + ((0, 1) if rng.randint(2) else (1, 0))

    src, dst = layout(), layout()
    shape = (1 << rng.randint(3, 7), 1 << rng.randint(3, 7))
    def per_lane(lay, shp):
        n = kh.A2(0, 0)
        kh.lib().kapy_fragments_loops(C.byref(kh.Fragments.make(*lay)), kh.A2(*shp), kh.A2(0, 0), n)
        return n[0] * n[1]

    while max(per_lane(src, shape), per_lane(dst, shape)) > 64:      # what kapy_change accepts per lane
        shape = (shape[0] // 2, shape[1]) if shape[0] >= shape[1] else (shape[0], shape[1] // 2)
    _change_case(ko, src, dst, shape, seed)


@pytest.mark.parametrize("dt", [kh.F32, kh.F16, kh.BF16])
def test_reduce_matches_oracle(ko, dt):
    """reduce_sum.mlir fixture shape (2x256 -> 2x1 column-major) and larger, both axes, sum and max."""
    for (m, n, axis) in ((2, 256, 1), (64, 1000, 1), (300, 128, 0), (4096, 64, 0), (37, 8192, 1), (5, 520, 1), (1000, 96, 0), (130, 50, 0)):
        x = ko.fill_normal(m * n, dt, 3, 0)
        for kind in (0, 1):
            om, on = (m, 1) if axis == 1 else (1, n)
            want = np.zeros(om * on, dtype=np.float32)
            assert ko.lib().ko_reduce(C.byref(ko.mk_global(x, m, n, n, 1, dt)), C.byref(ko.mk_global(want, om, on, 1, om, ko.F32)),
                                      axis, kind) == 0
            dx, dd = to_dev(x), dev_zeros(om * on, 4)
            kh.reduce(dglobal(dx, m, n, n, 1, dt), dglobal(dd, om, on, 1, om, kh.F32), axis, kind)
            sync()
            got = to_host(dd, np.float32)
            if kind == 1:
                assert np.array_equal(got, want)
            else:
                assert np.allclose(got, want, rtol=1e-5, atol=1e-4 * np.sqrt(max(m, n)))
