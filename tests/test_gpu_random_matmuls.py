"""Seeded random matmuls: random extents (multiples of the tiles and not), operand layouts (row- or column-major each),
16-bit operand type, result type, accumulator input, rounding mode, a fused tail; and random W8A8 shapes.  Relative
Frobenius error <= 1e-3 against the oracle (fp64 accumulate), and no element off by more than a few ulp of the largest."""
import ctypes as C

import numpy as np
import pytest

import kapy_hip as kh
from gpu_util import dev_zeros, dglobal, sync, to_dev, to_host

pytestmark = pytest.mark.gpu
NPS = {kh.F16: np.uint16, kh.BF16: np.uint16, kh.F32: np.float32}
vp = lambda x: x.ctypes.data_as(C.c_void_p)
EXTENTS = [1, 8, 16, 24, 64, 100, 128, 136, 200, 256, 264, 384, 520]


def _check(ko, got, want, dtype, what):
    g, w = ko.decode(got, dtype), ko.decode(want, dtype)
    assert np.all(np.isfinite(g)), what
    rel = np.linalg.norm(g - w) / max(np.linalg.norm(w), 1e-30)
    assert rel <= 1e-3, "%s: relative Frobenius error %g" % (what, rel)
    eps = {kh.F16: 2.0 ** -10, kh.BF16: 2.0 ** -7, kh.F32: 2.0 ** -12}[dtype]      # (f32 results: the accumulation order differs)
    assert np.abs(g - w).max() <= 4 * eps * max(np.abs(w).max(), 1e-30), what


@pytest.mark.parametrize("seed", range(60))
def test_random_matmul(ko, seed):
    rng = np.random.RandomState(3000 + seed)
    dt = [kh.F16, kh.BF16][rng.randint(2)]
    M, N, K = (EXTENTS[rng.randint(len(EXTENTS))] for _ in range(3))
    a_rm, b_rm = bool(rng.randint(2)), bool(rng.randint(2))
    out_dt = [dt, dt, kh.F32][rng.randint(3)]
    with_acc = rng.randint(5) == 0
    rmode = kh.RZ if rng.randint(6) == 0 else kh.RN
    fused = not with_acc and out_dt == dt and rmode == kh.RN and rng.randint(3) == 0
    a, b = ko.fill_normal(M * K, dt, seed, 0, 0.0, 0.5), ko.fill_normal(K * N, dt, seed, 1, 0.0, 0.5)
    a_str, b_str = ((K, 1) if a_rm else (1, M)), ((N, 1) if b_rm else (1, K))
    what = "seed %d: %dx%dx%d dtype %d A %s B %s -> dtype %d acc %s rmode %d fused %s" % (seed, M, N, K, dt, "row" if a_rm else "col", "row" if b_rm else "col",
                                                                                       out_dt, with_acc, rmode, fused)
    ga, gb = ko.mk_global(a, M, K, *a_str, dt), ko.mk_global(b, K, N, *b_str, dt)
    da, db = to_dev(a), to_dev(b)
    gda, gdb = dglobal(da, M, K, *a_str, dt), dglobal(db, K, N, *b_str, dt)
    dd = dev_zeros(M * N, kh.DTYPE_BYTES[out_dt])
    gdd = dglobal(dd, M, N, N, 1, out_dt)
    want = np.zeros(M * N, NPS[out_dt])
    if fused:
        bias = ko.fill_normal(N, dt, seed, 3)
        c32 = np.zeros(M * N, np.float32)
        assert ko.lib().ko_matmul(C.byref(ga), C.byref(gb), None, C.byref(ko.mk_global(c32, M, N, N, 1, kh.F32)), kh.RN) == 0, what
        L, ADD, MAX, ST, CAST, SPL = kh.EW_LD_GLOBAL, kh.EW_ADDF, kh.EW_MAXIMUMF, kh.EW_ST_GLOBAL, kh.EW_FPTOFP, kh.EW_SPLAT
        insts = [dict(op=L, dst=0, a=0), dict(op=L, dst=1, a=1), dict(op=CAST, dst=1, a=1, dtype=kh.F32), dict(op=ADD, dst=0, a=0, b=1),
                 dict(op=SPL, dst=2, dtype=kh.F32, imm=0.0), dict(op=MAX, dst=0, a=0, b=2), dict(op=CAST, dst=3, a=0, dtype=dt, rmode=kh.RN), dict(op=ST, a=3)]
        assert ko.elementwise(ko.program(insts), [ko.mk_global(c32.view(np.uint32), M, N, N, 1, kh.F32), ko.mk_global(bias, 1, N, N, 1, dt)],
                              ko.mk_global(want, M, N, N, 1, dt)) == 0, what
        dbias = to_dev(bias)
        kh.matmul_fused(gda, gdb, gdd, bias=dglobal(dbias, 1, N, N, 1, dt), act=kh.EW_MAXIMUMF, act_operand=0.0)
    else:
        go_acc = gd_acc = None
        if with_acc:
            acc = ko.fill_normal(M * N, kh.F32, seed, 2)
            dacc = to_dev(acc)
            go_acc, gd_acc = ko.mk_global(acc, M, N, N, 1, kh.F32), dglobal(dacc, M, N, N, 1, kh.F32)
        assert ko.lib().ko_matmul(C.byref(ga), C.byref(gb), C.byref(go_acc) if go_acc is not None else None, C.byref(ko.mk_global(want, M, N, N, 1, out_dt)), rmode) == 0, what
        kh.matmul(gda, gdb, gdd, acc=gd_acc, rmode=rmode)
    sync()
    _check(ko, to_host(dd, want.dtype), want, out_dt, what)


@pytest.mark.parametrize("seed", range(24))
def test_random_scaled_f8(ko, seed):
    rng = np.random.RandomState(5000 + seed)
    M = [1, 5, 16, 17, 33, 64, 100, 128, 200, 300][rng.randint(10)]
    N = [16, 48, 64, 136, 256, 520][rng.randint(6)]
    K = [128, 256, 384, 1024, 2048, 144][rng.randint(6)]
    a = ko.fill_normal(M * K, ko.F32, seed, 0).reshape(M, K)
    w = ko.fill_normal(N * K, ko.F32, seed, 1).reshape(N, K)
    aq, sa, wq, sb = np.zeros((M, K), np.uint8), np.zeros(M, np.float32), np.zeros((N, K), np.uint8), np.zeros(N, np.float32)
    ko.lib().ko_quantize_e4m3(vp(a), M, K, K, 1, 1, vp(aq), vp(sa))
    ko.lib().ko_quantize_e4m3(vp(w), N, K, K, 1, 1, vp(wq), vp(sb))
    want = np.zeros((M, N), np.uint16)
    assert ko.lib().ko_matmul_scaled_f8(C.byref(ko.mk_global(aq, M, K, K, 1, ko.F8E4M3)), C.byref(ko.mk_global(wq, K, N, 1, K, ko.F8E4M3)),
                                        vp(sa), vp(sb), C.byref(ko.mk_global(want, M, N, N, 1, ko.BF16))) == 0
    da, dw, dsa, dsb, dd = to_dev(aq), to_dev(wq), to_dev(sa), to_dev(sb), dev_zeros(M * N, 2)
    kh.matmul_scaled_f8(dglobal(da, M, K, K, 1, kh.F8E4M3), dglobal(dw, K, N, 1, K, kh.F8E4M3), dsa.data_ptr(), dsb.data_ptr(), dglobal(dd, M, N, N, 1, kh.BF16))
    sync()
    _check(ko, to_host(dd, np.uint16, (M, N)).ravel(), want.ravel(), kh.BF16, "seed %d: W8A8 %dx%dx%d" % (seed, M, N, K))
