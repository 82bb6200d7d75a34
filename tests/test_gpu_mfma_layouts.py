"""The exported matrix-instruction layouts against the hardware and against the kernels.

kapy_matmul_layouts says which lane and register holds which element of the lhs, rhs and accumulator blocks of each
matrix instruction (the counterpart of getDefaultLayouts, lib/Support/LayoutUtils.cpp:123-149, whose layouts the
reference's lowering turns into register indices, MatmulOpToLLVM.cpp:94-123).  The kernels take their lane positions
from those layouts.  Here a tile is scattered into per-lane registers BY the exported layouts, multiplied by one
instruction through the wrapper the kernels use (kapy_mfma_probe), and the product gathered BY the exported accumulator
layout: it equals the checker's matmul only if the layouts describe what the hardware does.  Values are small
integers, so every sum is exact and the comparison is bit for bit."""
import ctypes as C

import numpy as np
import pytest

import kapy_hip as kh
import kapy_probe as kp
from gpu_util import dev_zeros, sync, to_dev, to_host

pytestmark = pytest.mark.gpu

WAYS = [(kh.MFMA_32X32X16_16B, kh.F16, kh.F16), (kh.MFMA_32X32X16_16B, kh.BF16, kh.BF16), (kh.MFMA_16X16X32_16B, kh.F16, kh.F16),
        (kh.MFMA_16X16X32_16B, kh.BF16, kh.BF16), (kh.MFMA_16X16X128_F8, kh.F8E4M3, kh.F8E4M3), (kh.MFMA_16X16X128_F8, kh.F8E4M3, kh.F8E5M2),
        (kh.MFMA_16X16X128_F8, kh.F8E5M2, kh.F8E4M3), (kh.MFMA_32X32X64_F8, kh.F8E4M3, kh.F8E4M3), (kh.MFMA_32X32X64_F8, kh.F8E5M2, kh.F8E4M3),
        (kh.MFMA_32X32X64_F8, kh.F8E5M2, kh.F8E5M2)]


def _small_ints(ko, rng, shape, dtype):
    """Integers in [-4, 4] as storage bits of `dtype` (exactly representable in every float type here)."""
    vals = rng.integers(-4, 5, size=shape).astype(np.float64)
    enc = {ko.F16: ko.lib().ko_f64_to_f16, ko.BF16: ko.lib().ko_f64_to_bf16, ko.F8E4M3: ko.lib().ko_f64_to_e4m3, ko.F8E5M2: ko.lib().ko_f64_to_e5m2}[dtype]
    bits = np.array([enc(float(v), ko.RN) for v in vals.reshape(-1)], dtype=ko.NP_STORAGE[dtype]).reshape(shape)
    return vals, bits


def _scatter(layout, shape, tile_bits):
    """registers[lane][iv] = tile[index of (lane, iv) under the layout] (the reference's map 2)."""
    L = kh.lib()
    space = kh.A2(0, 0)
    L.kapy_fragments_loops(C.byref(layout), kh.A2(*shape), kh.A2(0, 0), space)
    per_lane = space[0] * space[1]
    regs = np.zeros((64, per_lane), dtype=tile_bits.dtype)
    o = kh.A2(0, 0)
    for lane in range(64):
        for iv in range(per_lane):
            assert L.kapy_fragments_map(C.byref(layout), kh.A2(*shape), 2, kh.A2(lane, iv), o) == 0
            regs[lane, iv] = tile_bits[o[0], o[1]]
    return regs


def _gather(layout, shape, regs):
    """tile[i][j] = registers[(lane, iv) that owns (i, j) under the layout] (the reference's map 3)."""
    L = kh.lib()
    tile = np.zeros(shape, dtype=regs.dtype)
    o = kh.A2(0, 0)
    for i in range(shape[0]):
        for j in range(shape[1]):
            assert L.kapy_fragments_map(C.byref(layout), kh.A2(*shape), 3, kh.A2(i, j), o) == 0
            tile[i, j] = regs[o[0], o[1]]
    return tile


@pytest.mark.parametrize("exchanged", [0, 1])
@pytest.mark.parametrize("way,lhs_dt,rhs_dt", WAYS)
def test_exported_layouts_describe_the_matrix_instruction(ko, way, lhs_dt, rhs_dt, exchanged):
    (lhs_l, (m, n, k)), (rhs_l, _), (acc_l, _) = kh.matmul_layouts(way, 0), kh.matmul_layouts(way, 1), kh.matmul_layouts(way, 3 if exchanged else 2)
    rng = np.random.default_rng(way * 10 + exchanged)
    a_vals, a_bits = _small_ints(ko, rng, (m, k), lhs_dt)
    b_vals, b_bits = _small_ints(ko, rng, (k, n), rhs_dt)
    # the checker's kapy.matmul on the same bits
    bt = np.ascontiguousarray(b_bits.T)
    want = np.zeros((m, n), np.float32)
    assert ko.lib().ko_matmul(C.byref(ko.mk_global(a_bits, m, k, k, 1, lhs_dt)), C.byref(ko.mk_global(bt, k, n, 1, k, rhs_dt)), None,
                              C.byref(ko.mk_global(want, m, n, n, 1, ko.F32)), ko.RN) == 0
    assert np.array_equal(want, (a_vals @ b_vals).astype(np.float32))
    d_a, d_b = to_dev(_scatter(lhs_l, (m, k), a_bits)), to_dev(_scatter(rhs_l, (k, n), b_bits))
    d_acc = dev_zeros(64 * (m * n // 64), 4)
    kp.mfma_probe(way, lhs_dt, rhs_dt, exchanged, d_a.data_ptr(), d_b.data_ptr(), d_acc.data_ptr())
    sync()
    got = _gather(acc_l, (m, n), to_host(d_acc, np.float32, (64, m * n // 64)))
    assert np.array_equal(got, want)
    # ... and the other accumulator layout must NOT fit (the two differ: one is the transpose of the other)
    other = _gather(kh.matmul_layouts(way, 2 if exchanged else 3)[0], (m, n), to_host(d_acc, np.float32, (64, m * n // 64)))
    assert np.array_equal(other, want.T) and not np.array_equal(other, want)


def test_a_one_hot_element_lands_where_the_layouts_say(ko):
    """lhs = e_(i,kk), rhs = e_(kk,j): the single non-zero of the product sits in the (lane, register) the accumulator
    layout names for (i, j), for a few (i, j, kk) per instruction."""
    L = kh.lib()
    for way, dt in ((kh.MFMA_16X16X32_16B, kh.BF16), (kh.MFMA_32X32X16_16B, kh.F16)):
        (lhs_l, (m, n, k)), (rhs_l, _) = kh.matmul_layouts(way, 0), kh.matmul_layouts(way, 1)
        one = 0x3F80 if dt == kh.BF16 else 0x3C00
        for (i, j, kk) in ((0, 0, 0), (3, 9, 5), (m - 1, 2, k - 1), (7, n - 1, 8)):
            a, b = np.zeros((m, k), np.uint16), np.zeros((k, n), np.uint16)
            a[i, kk], b[kk, j] = one, one
            d_a, d_b, d_acc = to_dev(_scatter(lhs_l, (m, k), a)), to_dev(_scatter(rhs_l, (k, n), b)), dev_zeros(m * n, 4)
            for exchanged in (0, 1):
                kp.mfma_probe(way, dt, dt, exchanged, d_a.data_ptr(), d_b.data_ptr(), d_acc.data_ptr())
                sync()
                regs = to_host(d_acc, np.float32, (64, m * n // 64))
                o = kh.A2(0, 0)
                acc_l = kh.matmul_layouts(way, 3 if exchanged else 2)[0]
                assert L.kapy_fragments_map(C.byref(acc_l), kh.A2(m, n), 3, kh.A2(i, j), o) == 0
                assert regs[o[0], o[1]] == 1.0 and np.count_nonzero(regs) == 1


def test_probe_refuses_mismatched_operands():
    d = dev_zeros(64 * 32, 4)
    for way, a, b in ((kh.MFMA_16X16X32_16B, kh.F16, kh.BF16), (kh.MFMA_16X16X32_16B, kh.F8E4M3, kh.F8E4M3), (kh.MFMA_16X16X128_F8, kh.F16, kh.F16)):
        with pytest.raises(kh.KapyError) as e:
            kp.mfma_probe(way, a, b, 0, d.data_ptr(), d.data_ptr(), d.data_ptr())
        assert e.value.status == kh.ERR_VERIFY
    with pytest.raises(kh.KapyError) as e:
        kp.mfma_probe(kh.MMA_M16N8K16_F16, kh.F16, kh.F16, 0, d.data_ptr(), d.data_ptr(), d.data_ptr())
    assert e.value.status == kh.ERR_INVALID
