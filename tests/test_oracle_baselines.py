"""The timing baselines of the benchmark's cpu_baseline leg (oracle/kapy_baseline.cpp) against the checker:
a baseline that computed something else would make the reported CPU time meaningless."""
import ctypes as C

import numpy as np
import pytest


@pytest.mark.parametrize("M,N,K,dt,scaled", [(96, 96, 96, "BF16", False), (40, 72, 1100, "F16", False), (33, 64, 256, "F8E4M3", True)])
def test_gemm_baseline_agrees_with_checker(ko, M, N, K, dt, scaled):
    dtype = getattr(ko, dt)
    if dtype == ko.F8E4M3:
        a = (ko.fill_bits16(M * K, 0, 0) % 120).astype(np.uint8).reshape(M, K)
        bt = (ko.fill_bits16(N * K, 0, 1) % 120).astype(np.uint8).reshape(N, K)
    else:
        a = ko.fill_uniform(M * K, dtype, 0, 0).reshape(M, K)
        bt = ko.fill_uniform(N * K, dtype, 0, 1).reshape(N, K)
    o1, o2 = np.zeros((M, N), np.float32), np.zeros((M, N), np.float32)
    ga, gb = ko.mk_global(a, M, K, K, 1, dtype), ko.mk_global(bt, K, N, 1, K, dtype)
    secs = C.c_double(-1.0)
    if scaled:
        rs = (np.arange(M, dtype=np.float32) % 7 + 1) * 0.01
        cs = (np.arange(N, dtype=np.float32) % 5 + 1) * 0.02
        assert ko.lib().ko_matmul_scaled_f8(C.byref(ga), C.byref(gb), rs.ctypes.data, cs.ctypes.data, C.byref(ko.mk_global(o1, M, N, N, 1, ko.F32))) == 0
        assert ko.lib().ko_baseline_gemm(C.byref(ga), C.byref(gb), rs.ctypes.data, cs.ctypes.data, C.byref(ko.mk_global(o2, M, N, N, 1, ko.F32)), C.byref(secs)) == 0
    else:
        assert ko.lib().ko_matmul(C.byref(ga), C.byref(gb), None, C.byref(ko.mk_global(o1, M, N, N, 1, ko.F32)), ko.RN) == 0
        assert ko.lib().ko_baseline_gemm(C.byref(ga), C.byref(gb), None, None, C.byref(ko.mk_global(o2, M, N, N, 1, ko.F32)), C.byref(secs)) == 0
    assert secs.value >= 0.0
    assert np.linalg.norm(o1.astype(np.float64) - o2) / np.linalg.norm(o1) < 1e-5


def test_gelu_baseline_within_two_ulp_of_checker(ko):
    m, n = 24, 512
    x = ko.fill_normal(m * n, ko.F16, 0).reshape(m, n)
    x[0, :8] = np.array([0x0000, 0x8000, 0x4900, 0xC900, 0x0001, 0x8001, 0x7BFF, 0xFBFF], np.uint16)   # zeros, +-10, least subnormals, +-max
    bias = ko.fill_normal(n, ko.F16, 1)
    want, got = np.zeros((m, n), np.uint16), np.zeros((m, n), np.uint16)
    assert ko.elementwise(ko.gelu_program(), [ko.mk_global(x, m, n, n, 1, ko.F16), ko.mk_global(bias, 1, n, n, 1, ko.F16)],
                          ko.mk_global(want, m, n, n, 1, ko.F16)) == 0
    assert ko.lib().ko_baseline_gelu_f16(x.ctypes.data, bias.ctypes.data, 0.5, got.ctypes.data, m, n, n) == 0
    line = lambda v: np.where(v.astype(np.int32) & 0x8000, -(v.astype(np.int32) & 0x7FFF), v.astype(np.int32) & 0x7FFF)
    assert np.abs(line(got) - line(want)).max() <= 2


def test_transpose_and_permute_baselines_are_bit_exact(ko):
    m, n = 200, 136
    src = ko.fill_bits16(m * n, 0).reshape(m, n)
    want, got = np.zeros((n, m), np.uint16), np.zeros((n, m), np.uint16)
    assert ko.lib().ko_copy(C.byref(ko.mk_global(src, m, n, n, 1, ko.F16)), C.byref(ko.mk_global(want, n, m, m, 1, ko.F16)), 1, 0) == 0
    assert ko.lib().ko_baseline_transpose16(src.ctypes.data, got.ctypes.data, m, n) == 0
    assert np.array_equal(got, want) and np.array_equal(got, src.T)
    b, h, s, d = 2, 3, 10, 16
    src = ko.fill_bits16(b * h * s * d, 1)
    want, got = np.zeros(b * h * s * d, np.uint16), np.zeros(b * h * s * d, np.uint16)
    assert ko.lib().ko_copy_batched(C.byref(ko.mk_global(src, s, d, d, 1, ko.BF16)), C.byref(ko.mk_global(want, s, d, h * d, 1, ko.BF16)), 0, 0,
                                    b, h, h * s * d, s * d, s * h * d, d) == 0
    assert ko.lib().ko_baseline_permute_bhsd_bshd16(src.ctypes.data, got.ctypes.data, b, h, s, d) == 0
    assert np.array_equal(got, want)
    assert np.array_equal(got.reshape(b, s, h, d), src.reshape(b, h, s, d).transpose(0, 2, 1, 3))
