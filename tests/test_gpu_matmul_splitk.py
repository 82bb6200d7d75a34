"""Split K: several workgroups share one output tile, each multiplying one part of K; their fp32 partial tiles meet in a
caller-provided workspace and the workgroup that arrives last sums them in split order.  Parity against the checker's
fp64-accumulated kapy.matmul (relative Frobenius error <= 1e-3, the tolerance the benchmark definition states), results
that do not depend on arrival order (two runs are bit-equal), counters left zero, and the refusals."""
import ctypes as C

import numpy as np
import pytest
import torch

import kapy_hip as kh
from gpu_util import dev_zeros, dglobal, sync, to_dev, to_host

pytestmark = pytest.mark.gpu
FROB_TOL = 1e-3
vp = lambda x: x.ctypes.data_as(C.c_void_p)


def _frob(ko, got, want, dtype):
    g, w = ko.decode(got, dtype), ko.decode(want, dtype)
    assert np.all(np.isfinite(g))
    return np.linalg.norm(g - w) / max(np.linalg.norm(w), 1e-30)


def _workspace(m, n):
    nbytes = kh.lib().kapy_matmul_workspace_bytes(m, n)
    assert nbytes >= 16384
    return torch.zeros(nbytes, dtype=torch.uint8, device="cuda")


def _operands(ko, dt, M, N, K, b_row_major, seed):
    a, b = ko.fill_uniform(M * K, dt, seed, 0), ko.fill_uniform(K * N, dt, seed, 1)
    b_str = (N, 1) if b_row_major else (1, K)
    want = np.zeros(M * N, np.uint16)
    assert ko.lib().ko_matmul(C.byref(ko.mk_global(a, M, K, K, 1, dt)), C.byref(ko.mk_global(b, K, N, *b_str, dt)), None,
                              C.byref(ko.mk_global(want, M, N, N, 1, dt)), ko.RN) == 0
    return a, b, b_str, want


@pytest.mark.parametrize("dt,M,N,K,b_row_major,tile,splits", [
    (kh.F16, 1024, 1024, 1024, True, (128, 128, 32), (2, 4, 8)),       # benchmark configuration 1 on the transposing-read kernel
    (kh.BF16, 256, 384, 2048, True, (128, 128, 64), (2, 4)),
    (kh.BF16, 200, 128, 512, True, (128, 128, 32), (2,)),              # a tile hangs over the last rows of the lhs
    (kh.BF16, 256, 384, 2048, False, (128, 128, 64), (2, 4, 8)),       # lhs row-major, rhs column-major: the 128 x 128 ring kernel
    (kh.F16, 200, 136, 1024, False, (128, 128, 64), (2, 4)),           # tiles hang over both edges
])
def test_split_k_matches_checker_and_is_deterministic(ko, dt, M, N, K, b_row_major, tile, splits):
    a, b, b_str, want = _operands(ko, dt, M, N, K, b_row_major, seed=11)
    da, db = to_dev(a), to_dev(b)
    ws = _workspace(M, N)
    ga, gb = dglobal(da, M, K, K, 1, dt), dglobal(db, K, N, *b_str, dt)
    stages = 0 if b_row_major else 25
    dd0 = dev_zeros(M * N, 2)
    kh.matmul(ga, gb, dglobal(dd0, M, N, N, 1, dt), tile=tile, stages=stages, split_k=1)
    sync()
    assert _frob(ko, to_host(dd0, np.uint16), want, dt) <= FROB_TOL
    for sp in splits:
        outs = []
        for rep in range(2):
            dd = dev_zeros(M * N, 2, fill=0x7E7E)
            kh.matmul(ga, gb, dglobal(dd, M, N, N, 1, dt), tile=tile, stages=stages, split_k=sp, workspace=ws)
            sync()
            outs.append(to_host(dd, np.uint16))
        assert _frob(ko, outs[0], want, dt) <= FROB_TOL, sp
        assert np.array_equal(outs[0], outs[1]), sp                      # fixed summation order: no run-to-run difference
        assert int(ws[:16384].max().item()) == 0, sp                     # the arrival counters are back to zero


def test_alternating_problems_never_see_the_other_problems_partial_sums(ko):
    """Two different operand sets of one shape take turns on ONE workspace: the partial sums of the call before lie exactly
    where this call's go, so a reader that was served a stale cache line would produce the other problem's numbers."""
    dt, M, N, K, tile = kh.F16, 512, 512, 2048, (128, 128, 32)
    sets = []
    for seed in (21, 22):
        a, b, b_str, want = _operands(ko, dt, M, N, K, True, seed=seed)
        sets.append((to_dev(a), to_dev(b), want))
    ws = _workspace(M, N)
    first = {}
    for rep in range(6):
        for k, (da, db, want) in enumerate(sets):
            dd = dev_zeros(M * N, 2, fill=0x7E7E)
            kh.matmul(dglobal(da, M, K, K, 1, dt), dglobal(db, K, N, N, 1, dt), dglobal(dd, M, N, N, 1, dt), tile=tile, split_k=8, workspace=ws)
            sync()
            got = to_host(dd, np.uint16)
            if rep == 0:
                assert _frob(ko, got, want, dt) <= FROB_TOL
                first[k] = got
            assert np.array_equal(got, first[k]), (rep, k)
    # the same back to back without a synchronisation in between (stream order alone keeps the calls apart)
    outs = [dev_zeros(M * N, 2) for _ in range(8)]
    for t, dd in enumerate(outs):
        da, db, _ = sets[t % 2]
        kh.matmul(dglobal(da, M, K, K, 1, dt), dglobal(db, K, N, N, 1, dt), dglobal(dd, M, N, N, 1, dt), tile=tile, split_k=8, workspace=ws)
    sync()
    for t, dd in enumerate(outs):
        assert np.array_equal(to_host(dd, np.uint16), first[t % 2]), t


def test_library_chooses_a_split_only_with_a_workspace(ko):
    """split_k = 0: with a workspace a result of 16 tiles and 64 K-tiles on 256 CUs is split four ways (parts of at least 16
    K-tiles; same bits as asking for 4), without one nothing changes (same bits as asking for 1)."""
    dt, M, N, K = kh.F16, 512, 512, 2048
    a, b, b_str, want = _operands(ko, dt, M, N, K, True, seed=0)
    da, db, ws = to_dev(a), to_dev(b), _workspace(M, N)
    ga, gb = dglobal(da, M, K, K, 1, dt), dglobal(db, K, N, *b_str, dt)
    res = {}
    for name, kw in (("auto_ws", dict(workspace=ws)), ("four", dict(split_k=4, workspace=ws)), ("auto", {}), ("one", dict(split_k=1, workspace=ws))):
        dd = dev_zeros(M * N, 2)
        kh.matmul(ga, gb, dglobal(dd, M, N, N, 1, dt), tile=(128, 128, 32), **kw)
        sync()
        res[name] = to_host(dd, np.uint16)
        assert _frob(ko, res[name], want, dt) <= FROB_TOL
    cus = C.c_int32()
    assert kh.lib().kapy_device_info(C.byref(cus), None, None, None, 0) == 0
    if cus.value == 256:
        assert np.array_equal(res["auto_ws"], res["four"]) and not np.array_equal(res["four"], res["one"])
    assert np.array_equal(res["auto"], res["one"])


@pytest.mark.parametrize("M,N,K", [(64, 512, 4096), (100, 384, 2048), (17, 256, 8192), (128, 8192, 8192)])
def test_w8a8_few_rows_split_k(ko, M, N, K):
    """W8A8 with few rows: with a workspace the tiled kernel splits K (the weight is read once, by tiles * split workgroups)."""
    a = ko.fill_normal(M * K, ko.F32, 5, 0).reshape(M, K)
    w = ko.fill_normal(N * K, ko.F32, 6, 0).reshape(N, K)
    aq, sa, wq, sb = np.zeros((M, K), np.uint8), np.zeros(M, np.float32), np.zeros((N, K), np.uint8), np.zeros(N, np.float32)
    ko.lib().ko_quantize_e4m3(vp(a), M, K, K, 1, 1, vp(aq), vp(sa))
    ko.lib().ko_quantize_e4m3(vp(w), N, K, K, 1, 1, vp(wq), vp(sb))
    want = np.zeros((M, N), np.uint16)
    assert ko.lib().ko_matmul_scaled_f8(C.byref(ko.mk_global(aq, M, K, K, 1, ko.F8E4M3)), C.byref(ko.mk_global(wq, K, N, 1, K, ko.F8E4M3)),
                                        vp(sa), vp(sb), C.byref(ko.mk_global(want, M, N, N, 1, ko.BF16))) == 0
    da, dw, dsa, dsb, ws = to_dev(aq), to_dev(wq), to_dev(sa), to_dev(sb), _workspace(M, N)
    ga, gw = dglobal(da, M, K, K, 1, kh.F8E4M3), dglobal(dw, K, N, 1, K, kh.F8E4M3)
    outs = []
    for kw in (dict(workspace=ws), dict(workspace=ws), dict(split_k=2, workspace=ws), {}):
        dd = dev_zeros(M * N, 2, fill=0x7E7E)
        kh.matmul_scaled_f8(ga, gw, dsa.data_ptr(), dsb.data_ptr(), dglobal(dd, M, N, N, 1, kh.BF16), **kw)
        sync()
        outs.append(to_host(dd, np.uint16, (M, N)))
        assert _frob(ko, outs[-1], want, kh.BF16) <= FROB_TOL
    assert np.array_equal(outs[0], outs[1])
    assert int(ws[:16384].max().item()) == 0


def test_split_k_refusals(ko):
    dt, M, N, K = kh.F16, 256, 256, 256
    d = dev_zeros(M * K, 2)
    g = dglobal(d, M, K, K, 1, dt)
    ws = _workspace(M, N)
    for kw, status in ((dict(split_k=3, workspace=ws), kh.ERR_INVALID), (dict(split_k=16, workspace=ws), kh.ERR_INVALID),
                       (dict(split_k=4), kh.ERR_INVALID),                                                 # no workspace
                       (dict(split_k=4, workspace=(ws.data_ptr(), 16384 + 4096)), kh.ERR_UNSUPPORTED),   # too small
                       (dict(split_k=8, workspace=ws), kh.ERR_UNSUPPORTED)):                              # K = 256 has no 8 parts of whole 64-wide tiles
        with pytest.raises(kh.KapyError) as e:
            kh.matmul(g, g, g, tile=(128, 128, 64), **kw)
        assert e.value.status == status, kw


def test_an_explicit_split_with_a_free_tile_choice_is_honoured(ko):
    """A problem large enough for the 256 x 256 tiles (which cannot split K): an explicit split_k moves the call to the
    128 x 128 tiles instead of being dropped; the result equals the unsplit call's within the GEMM bar, and a split the
    workspace cannot hold is refused, not ignored."""
    dt, M, N, K = kh.BF16, 4096, 4096, 512
    a, b = ko.fill_normal(M * K, dt, 41, 0, 0.0, 0.5), ko.fill_normal(N * K, dt, 42, 0, 0.0, 0.5)
    da, db = to_dev(a), to_dev(b)
    ga, gb = dglobal(da, M, K, K, 1, dt), dglobal(db, K, N, 1, K, dt)
    plain, split = dev_zeros(M * N, 2), dev_zeros(M * N, 2)
    kh.matmul(ga, gb, dglobal(plain, M, N, N, 1, dt))
    ws = _workspace(M, N)
    kh.matmul(ga, gb, dglobal(split, M, N, N, 1, dt), split_k=2, workspace=ws)
    sync()
    p, q = ko.decode(to_host(plain, np.uint16), dt), ko.decode(to_host(split, np.uint16), dt)
    assert np.linalg.norm(p - q) <= 2e-3 * np.linalg.norm(p) and not np.array_equal(to_host(split, np.uint16), np.zeros(M * N, np.uint16))
    assert not ws[:16384].any()                                        # the split ran: its counters were used and are back at zero
    with pytest.raises(kh.KapyError) as e:
        kh.matmul(ga, gb, dglobal(split, M, N, N, 1, dt), split_k=2, workspace=(ws.data_ptr(), 16384 + 4096))
    assert e.value.status == kh.ERR_UNSUPPORTED

