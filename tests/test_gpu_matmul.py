"""GPU parity for kapy.matmul: relative Frobenius error <= 1e-3 against the oracle's fp64-accumulated
result (the tolerance the benchmark definition states), closed forms bit-exact."""
import ctypes as C

import numpy as np
import pytest

import kapy_hip as kh
from gpu_util import dev_zeros, dglobal, sync, to_dev, to_host

pytestmark = pytest.mark.gpu
FROB_TOL = 1e-3


def _frob(ko, got, want, dtype):
    g, w = ko.decode(got, dtype), ko.decode(want, dtype)
    assert np.all(np.isfinite(g))
    return np.linalg.norm(g - w) / max(np.linalg.norm(w), 1e-30)


def _np_store(dtype):
    return {1: np.uint8, 2: np.uint16, 4: np.float32}[kh.DTYPE_BYTES[dtype]]


def _run(ko, dt, M, N, K, a_row_major=True, b_row_major=True, out_dtype=None, with_acc=None, d_col_major=False,
         seed=0, gen="uniform", rmode=kh.RN, tile=(0, 0, 0), stages=0, impl_way=0):
    out_dtype = dt if out_dtype is None else out_dtype
    fill = (lambda n, s: ko.fill_uniform(n, dt, seed, s)) if gen == "uniform" else (lambda n, s: ko.fill_normal(n, dt, seed, s, 0.0, 0.02))
    a, b = fill(M * K, 0), fill(K * N, 1)
    a_str = (K, 1) if a_row_major else (1, M)
    b_str = (N, 1) if b_row_major else (1, K)
    d_str = (1, M) if d_col_major else (N, 1)
    want = np.zeros(M * N, dtype=_np_store(out_dtype))
    acc = None
    da, db, dd = to_dev(a), to_dev(b), dev_zeros(M * N, kh.DTYPE_BYTES[out_dtype])
    go_acc = gd_acc = None
    if with_acc is not None:
        acc = ko.fill_normal(M * N, with_acc, seed, 2)
        dacc = to_dev(acc)
        go_acc, gd_acc = ko.mk_global(acc, M, N, N, 1, with_acc), dglobal(dacc, M, N, N, 1, with_acc)
    rc = ko.lib().ko_matmul(C.byref(ko.mk_global(a, M, K, *a_str, dt)), C.byref(ko.mk_global(b, K, N, *b_str, dt)),
                            C.byref(go_acc) if go_acc is not None else None, C.byref(ko.mk_global(want, M, N, *d_str, out_dtype)), rmode)
    assert rc == 0
    kh.matmul(dglobal(da, M, K, *a_str, dt), dglobal(db, K, N, *b_str, dt), dglobal(dd, M, N, *d_str, out_dtype), acc=gd_acc,
              rmode=rmode, tile=tile, stages=stages, impl_way=impl_way)
    sync()
    return to_host(dd, want.dtype), want


def test_config1_fp16_1024_row_major_128x128x32_tiles(ko):
    """benchmark configuration 1: fp16 GEMM 1024^3, row-major A and B, fp32 accumulate, fp16 out, uniform[-1,1) seed 0."""
    got, want = _run(ko, kh.F16, 1024, 1024, 1024, True, True, tile=(128, 128, 32))
    assert _frob(ko, got, want, kh.F16) <= FROB_TOL
    assert (got != want).mean() < 0.05    # fp32 vs fp64 accumulation flips few roundings


@pytest.mark.parametrize("tile_k,stages", [(64, 4), (64, 3), (32, 4)])
def test_nn_transposing_read_kernel_every_variant(ko, tile_k, stages):
    """Both operands row-major, extents multiples of 128 x 128 x tile_k: the kernel that stages the rhs as it lies in
    memory and transposes on the way out of LDS; K of 1, 2, 3, 7 and 16 tiles (prologue, ring wrap, fragment parity)."""
    for dt in (kh.BF16, kh.F16):
        for (M, N, K) in ((128, 128, tile_k), (128, 256, 2 * tile_k), (256, 128, 3 * tile_k), (128, 128, 7 * tile_k), (384, 256, 16 * tile_k),
                          (200, 128, 4 * tile_k), (1, 256, 2 * tile_k), (333, 128, 5 * tile_k)):   # the last three: a tile hangs over the last rows of the lhs
            got, want = _run(ko, dt, M, N, K, True, True, seed=7, tile=(128, 128, tile_k), stages=stages)
            assert _frob(ko, got, want, dt) <= FROB_TOL, (M, N, K)
    got32, want32 = _run(ko, kh.F16, 256, 256, 8 * tile_k, True, True, out_dtype=kh.F32, with_acc=kh.F32, seed=7, tile=(128, 128, tile_k), stages=stages)
    assert _frob(ko, got32, want32, kh.F32) <= 1e-5


def test_general_kernel_when_asked_for_one_stage(ko):
    """stages=1 selects the register-staged general kernel also for shapes the faster kernels would take."""
    got, want = _run(ko, kh.F16, 256, 256, 128, True, True, seed=9, tile=(128, 128, 32), stages=1)
    assert _frob(ko, got, want, kh.F16) <= FROB_TOL


@pytest.mark.parametrize("dt", [kh.F16, kh.BF16])
@pytest.mark.parametrize("a_rm,b_rm", [(True, True), (True, False), (False, True), (False, False)])
def test_all_operand_layouts_and_ragged_shapes(ko, dt, a_rm, b_rm):
    for (M, N, K) in ((128, 128, 64), (200, 136, 72), (16, 8, 16), (130, 257, 100)):
        got, want = _run(ko, dt, M, N, K, a_rm, b_rm, seed=3)
        assert _frob(ko, got, want, dt) <= FROB_TOL, (M, N, K)


MFMA16, MFMA32 = 17, 16   # KAPY_MFMA_16X16X32_16B, KAPY_MFMA_32X32X16_16B
TN_VARIANTS = [((256, 256, 64), 25, MFMA16), ((256, 256, 64), 2, MFMA16), ((256, 256, 64), 25, MFMA32), ((256, 256, 64), 2, MFMA32),
               ((256, 256, 32), 4, MFMA32), ((128, 128, 64), 25, MFMA16), ((128, 128, 64), 2, MFMA32), ((128, 128, 32), 4, MFMA32),
               ((128, 128, 64), 4, MFMA32), ((128, 64, 64), 4, MFMA32), ((64, 64, 128), 4, MFMA32)]


@pytest.mark.parametrize("tile,stages,impl_way", TN_VARIANTS)
def test_tn_roofline_kernel_every_variant(ko, tile, stages, impl_way):
    """lhs row-major, rhs column-major, extents multiples of the tile: the LDS-direct kernels, each compiled
    configuration forced through kapy_matmul_cfg, including K of 1, 2, 3 and many tiles (pipeline prologue / tail)."""
    bm, bn, bk = tile
    for dt in (kh.BF16, kh.F16):
        for (M, N, K) in ((bm, bn, bk), (bm, bn, 2 * bk), (bm, 2 * bn, 3 * bk), (2 * bm, bn, 4 * bk), (bm, bn, 7 * bk), (3 * bm, 2 * bn, 16 * bk)):
            got, want = _run(ko, dt, M, N, K, True, False, seed=5, tile=tile, stages=stages, impl_way=impl_way)
            assert _frob(ko, got, want, dt) <= FROB_TOL, (M, N, K)
    got32, want32 = _run(ko, kh.BF16, 2 * bm, 2 * bn, 8 * bk, True, False, out_dtype=kh.F32, seed=5, tile=tile, stages=stages, impl_way=impl_way)
    assert _frob(ko, got32, want32, kh.F32) <= 1e-5


@pytest.mark.parametrize("dt", [kh.BF16, kh.F16])
def test_few_tiles_take_smaller_tiles(ko, dt):
    """K-contiguous operands whose 64 x 64 (or 128 x 64) tiles number no more than the CUs: the four-stage builds on those tiles,
    with tiles that hang over the last rows and columns, K of one to many K-tiles, NaNs behind the operands."""
    for (M, N, K) in ((100, 520, 512), (192, 1024, 384), (256, 2048, 320), (130, 264, 192), (1, 64, 128), (64, 4096, 1024), (250, 72, 64)):
        a, b = ko.fill_normal(M * K, dt, 17, 0, 0.0, 0.5), ko.fill_normal(K * N, dt, 17, 1, 0.0, 0.5)
        want = np.zeros(M * N, np.uint16)
        assert ko.lib().ko_matmul(C.byref(ko.mk_global(a, M, K, K, 1, dt)), C.byref(ko.mk_global(b, K, N, 1, K, dt)), None,
                                  C.byref(ko.mk_global(want, M, N, N, 1, dt)), kh.RN) == 0
        poison = np.full(4096, 0x7e00 if dt == kh.F16 else 0x7fc0, np.uint16)
        da, db, dd = to_dev(np.concatenate([a, poison])), to_dev(np.concatenate([b, poison])), dev_zeros(M * N + 256, 2, fill=0x1234)
        kh.matmul(dglobal(da, M, K, K, 1, dt), dglobal(db, K, N, 1, K, dt), dglobal(dd, M, N, N, 1, dt))
        sync()
        got = to_host(dd, np.uint16)
        assert np.all(got[M * N:] == 0x1234), (M, N, K)
        assert _frob(ko, got[:M * N], want, dt) <= FROB_TOL, (M, N, K)


def test_tn_default_choice(ko):
    for (M, N, K) in ((256, 256, 64), (512, 768, 1024), (1024, 1024, 96), (384, 640, 160)):
        got, want = _run(ko, kh.BF16, M, N, K, True, False, seed=6)
        assert _frob(ko, got, want, kh.BF16) <= FROB_TOL, (M, N, K)


def test_closed_forms_identity_ones_rank1(ko):
    n = 256
    eye = np.eye(n, dtype=np.float16).view(np.uint16)
    b = ko.fill_uniform(n * n, kh.F16, 4)
    d_eye, d_b, d_out = to_dev(eye), to_dev(b), dev_zeros(n * n, 2)
    g = lambda t, s=(n, 1): dglobal(t, n, n, s[0], s[1], kh.F16)
    kh.matmul(g(d_eye), g(d_b), g(d_out))                           # staged kernel: I·B = B
    sync()
    assert np.array_equal(to_host(d_out, np.uint16), b)
    kh.matmul(g(d_eye), g(d_b, (1, n)), g(d_out))                   # TN kernel: I·(B^T as col-major) = B^T
    sync()
    assert np.array_equal(to_host(d_out, np.uint16, (n, n)), b.reshape(n, n).T)
    ones = np.ones(n * n, dtype=np.float16).view(np.uint16)
    d_ones = to_dev(ones)
    kh.matmul(g(d_ones), g(d_ones, (1, n)), g(d_out))
    sync()
    assert np.all(to_host(d_out, np.uint16).view(np.float16) == n)  # all-ones -> K
    u = (np.arange(n) % 7 + 1).astype(np.float16)
    a1 = np.outer(u, np.ones(n)).astype(np.float16).view(np.uint16)
    b1t = np.outer(u, np.ones(n)).astype(np.float16).view(np.uint16)  # column-major rhs: (k,n) at n*K+k -> rhs[k,n] = u[n]
    d32 = dev_zeros(n * n, 4)
    kh.matmul(g(to_dev(a1)), g(to_dev(b1t), (1, n)), dglobal(d32, n, n, n, 1, kh.F32))
    sync()
    assert np.array_equal(to_host(d32, np.float32, (n, n)), n * np.outer(u, u).astype(np.float32))


def test_accumulator_input_f32_out_and_column_major_result(ko):
    got, want = _run(ko, kh.BF16, 256, 256, 128, True, False, out_dtype=kh.F32, with_acc=kh.F32, seed=8)
    assert _frob(ko, got, want, kh.F32) <= 1e-5
    got, want = _run(ko, kh.F16, 192, 160, 64, True, True, out_dtype=kh.F16, with_acc=kh.F16, seed=8)
    assert _frob(ko, got, want, kh.F16) <= FROB_TOL
    got, want = _run(ko, kh.F16, 256, 256, 64, True, False, d_col_major=True, seed=9)
    assert _frob(ko, got, want, kh.F16) <= FROB_TOL
    got, want = _run(ko, kh.BF16, 128, 128, 256, True, False, rmode=kh.RZ, seed=9)
    assert _frob(ko, got, want, kh.BF16) <= 2e-3   # RZ against RZ oracle; accumulation order differs


@pytest.mark.parametrize("dt", [kh.F16, kh.BF16])
@pytest.mark.parametrize("a_rm,b_rm", [(True, True), (True, False), (False, True), (False, False)])
def test_column_major_result_is_the_transposed_problem(ko, dt, a_rm, b_rm):
    """A column-major result is computed as D^T = B^T . A^T with a row-major result: against the checker, and bit for bit the
    row-major result of the same call (every dot product sums the same products in the same order), with and without a
    column-major fp32 accumulator input, on whole tiles and on ragged extents, and an explicit tile turned with the problem."""
    for (M, N, K, tile) in ((256, 384, 128, (0, 0, 0)), (200, 136, 72, (0, 0, 0)), (130, 264, 104, (0, 0, 0)), (512, 256, 192, (128, 128, 64))):
        if tile != (0, 0, 0) and not (a_rm and not b_rm):
            continue   # (the explicit tile names the K-contiguous kernel)
        a, b = ko.fill_normal(M * K, dt, 13, 0, 0.0, 0.5), ko.fill_normal(K * N, dt, 13, 1, 0.0, 0.5)
        acc = ko.fill_normal(M * N, kh.F32, 13, 2, 0.0, 0.5)            # read as column-major [M x N] and as row-major [M x N] below
        a_str, b_str = ((K, 1) if a_rm else (1, M)), ((N, 1) if b_rm else (1, K))
        da, db, dacc = to_dev(a), to_dev(b), to_dev(acc)
        acc_t = np.ascontiguousarray(acc.reshape(N, M).T).ravel()      # the same accumulator values laid out row-major
        dacc_t = to_dev(acc_t)
        for with_acc in (False, True):
            out_dt = kh.F32 if with_acc else dt
            ob = kh.DTYPE_BYTES[out_dt]
            want = np.zeros(M * N, dtype=_np_store(out_dt))
            assert ko.lib().ko_matmul(C.byref(ko.mk_global(a, M, K, *a_str, dt)), C.byref(ko.mk_global(b, K, N, *b_str, dt)),
                                      C.byref(ko.mk_global(acc, M, N, 1, M, kh.F32)) if with_acc else None,
                                      C.byref(ko.mk_global(want, M, N, 1, M, out_dt)), kh.RN) == 0
            d_col, d_row = dev_zeros(M * N + 64, ob, fill=0x1234), dev_zeros(M * N, ob)
            kh.matmul(dglobal(da, M, K, *a_str, dt), dglobal(db, K, N, *b_str, dt), dglobal(d_col, M, N, 1, M, out_dt),
                      acc=dglobal(dacc, M, N, 1, M, kh.F32) if with_acc else None, tile=tile)
            kh.matmul(dglobal(da, M, K, *a_str, dt), dglobal(db, K, N, *b_str, dt), dglobal(d_row, M, N, N, 1, out_dt),
                      acc=dglobal(dacc_t, M, N, N, 1, kh.F32) if with_acc else None, tile=tile)
            sync()
            got = to_host(d_col, want.dtype)
            bits = np.uint32 if ob == 4 else np.uint16
            assert np.all(got[M * N:].view(bits) == 0x1234), (M, N, K)
            got = got[:M * N]
            assert _frob(ko, got, want, out_dt) <= (1e-5 if out_dt == kh.F32 else FROB_TOL), (M, N, K, with_acc)
            row = to_host(d_row, want.dtype).reshape(M, N)
            assert np.array_equal(got.reshape(N, M).T.view(bits), row.view(bits)), (M, N, K, with_acc)


def test_subview_operands(ko):
    """matmul on sv_global views of larger buffers (start offsets, same strides)."""
    M, N, K = 128, 128, 96
    big_a = ko.fill_uniform(256 * 256, kh.F16, 6, 0)
    big_b = ko.fill_uniform(256 * 256, kh.F16, 6, 1)
    want = np.zeros((M, N), dtype=np.uint16)
    va = ko.sv_global(ko.mk_global(big_a, 256, 256, 256, 1, ko.F16), 64, 64 + M, 32, 32 + K)
    vb = ko.sv_global(ko.mk_global(big_b, 256, 256, 256, 1, ko.F16), 16, 16 + K, 100, 100 + N)
    assert ko.lib().ko_matmul(C.byref(va), C.byref(vb), None, C.byref(ko.mk_global(want, M, N, N, 1, ko.F16)), ko.RN) == 0
    da, db, dd = to_dev(big_a), to_dev(big_b), dev_zeros(M * N, 2)
    kh.matmul(kh.sv_global(dglobal(da, 256, 256, 256, 1, kh.F16), 64, 64 + M, 32, 32 + K),
              kh.sv_global(dglobal(db, 256, 256, 256, 1, kh.F16), 16, 16 + K, 100, 100 + N), dglobal(dd, M, N, N, 1, kh.F16))
    sync()
    assert _frob(ko, to_host(dd, np.uint16), want.ravel(), kh.F16) <= FROB_TOL


def test_config4_bf16_8192_sampled_against_oracle(ko):
    """benchmark configuration 4: bf16 8192^3, A row-major, B column-major, normal(0,0.02) seeds 0/1, bf16 out.
    The GPU computes the whole product; the fp64 oracle recomputes 64x64 blocks spread over the
    result (every block row and column of the 256-tile grid is hit), and linearity in A covers the rest:
    (A + A)·B must equal 2·(A·B) exactly, element by element, in bf16."""
    n = 8192
    a = ko.fill_normal(n * n, ko.BF16, 0, 0, 0.0, 0.02)
    bt = ko.fill_normal(n * n, ko.BF16, 1, 0, 0.0, 0.02)      # column-major rhs: element (k, j) at j*n + k
    da, db, dd = to_dev(a), to_dev(bt), dev_zeros(n * n, 2)
    ga, gb, gd = dglobal(da, n, n, n, 1, kh.BF16), dglobal(db, n, n, 1, n, kh.BF16), dglobal(dd, n, n, n, 1, kh.BF16)
    kh.matmul(ga, gb, gd)
    sync()
    got = to_host(dd, np.uint16, (n, n))
    goa, gob = ko.mk_global(a, n, n, n, 1, ko.BF16), ko.mk_global(bt, n, n, 1, n, ko.BF16)
    num = den = 0.0
    blk = 64
    for t in range(32):
        r0, c0 = (t * 256 + (t * 37) % 192) % n, ((31 - t) * 256 + (t * 53) % 192) % n
        want = np.zeros((blk, blk), dtype=np.uint16)
        rc = ko.lib().ko_matmul(C.byref(ko.sv_global(goa, r0, r0 + blk, 0, n)), C.byref(ko.sv_global(gob, 0, n, c0, c0 + blk)), None,
                                C.byref(ko.mk_global(want, blk, blk, blk, 1, ko.BF16)), ko.RN)
        assert rc == 0
        g, w = ko.decode(got[r0:r0 + blk, c0:c0 + blk], ko.BF16), ko.decode(want, ko.BF16)
        num += ((g - w) ** 2).sum()
        den += (w ** 2).sum()
    assert np.sqrt(num / den) <= FROB_TOL
    # linearity: doubling A (exact in bf16) doubles every output bit-exactly (exponent + 1)
    import torch
    a2 = (torch.from_numpy(a.view(np.int16)).view(torch.bfloat16) * 2).view(torch.int16).numpy().view(np.uint16)
    da.copy_(torch.from_numpy(a2.view(np.int16)).cuda())
    dd2 = dev_zeros(n * n, 2)
    kh.matmul(ga, gb, dglobal(dd2, n, n, n, 1, kh.BF16))
    sync()
    got2 = to_host(dd2, np.uint16, (n, n))
    g1 = (got.astype(np.uint32) << 16).view(np.float32)
    g2 = (got2.astype(np.uint32) << 16).view(np.float32)
    assert np.array_equal(g2, 2 * g1)


@pytest.mark.parametrize("dt", [kh.BF16, kh.F16])
@pytest.mark.parametrize("M,N,K", [(300, 512, 256), (513, 264, 192), (1000, 1000, 128), (257, 255 + 1, 64), (130, 777 + 7, 320),
                                   (256, 256, 72), (300, 520, 200), (512, 256, 8), (640, 384, 1000)])   # the last four: a partial last K-tile
def test_extents_that_are_not_multiples_of_the_tile_stay_on_the_ring_kernel(ko, dt, M, N, K):
    """K-contiguous operands, K a multiple of 8 (whole 16-byte chunks), M and N anything: tiles hang over the last rows of
    the operands, whose loads the buffer descriptors bound, and over the end of K, where the lanes past it fetch zeros;
    nothing is written outside the result."""
    a, b = ko.fill_normal(M * K, dt, 7, 0, 0.0, 0.5), ko.fill_normal(K * N, dt, 7, 1, 0.0, 0.5)
    want = np.zeros(M * N, dtype=np.uint16)
    assert ko.lib().ko_matmul(C.byref(ko.mk_global(a, M, K, K, 1, dt)), C.byref(ko.mk_global(b, K, N, 1, K, dt)), None,
                              C.byref(ko.mk_global(want, M, N, N, 1, dt)), kh.RN) == 0
    pad = 4096
    da, db, dd = to_dev(a), to_dev(b), dev_zeros(M * N + pad, 2, fill=0x1234)
    kh.matmul(dglobal(da, M, K, K, 1, dt), dglobal(db, K, N, 1, K, dt), dglobal(dd, M, N, N, 1, dt))
    sync()
    got = to_host(dd, np.uint16)
    assert np.all(got[M * N:] == 0x1234)
    assert _frob(ko, got[:M * N], want, dt) <= FROB_TOL
    # the same through the ring variants asked for by name (both tile sizes take ragged extents)
    for tile in ((256, 256, 64), (128, 128, 64)):
        dd2 = dev_zeros(M * N, 2)
        kh.matmul(dglobal(da, M, K, K, 1, dt), dglobal(db, K, N, 1, K, dt), dglobal(dd2, M, N, N, 1, dt), tile=tile, stages=25)
        sync()
        assert _frob(ko, to_host(dd2, np.uint16), want, dt) <= FROB_TOL, tile


@pytest.mark.parametrize("M,N,K", [(300, 512, 256), (513, 264, 192), (257, 256, 72), (1000, 1000, 128), (130, 136, 64)])
def test_f32_result_takes_the_strip_epilogue_and_writes_nothing_outside(ko, M, N, K):
    """A row-major fp32 result (16-byte aligned rows, no accumulator input) is stored by the same strips through LDS as a
    16-bit one, 32 bytes per lane; tiles that hang over the result's last rows and columns must leave the words behind it
    alone, and a result window inside a wider buffer must leave the columns beside it alone."""
    dt = kh.BF16
    a, b = ko.fill_normal(M * K, dt, 11, 0, 0.0, 0.5), ko.fill_normal(K * N, dt, 11, 1, 0.0, 0.5)
    want = np.zeros(M * N, dtype=np.float32)
    assert ko.lib().ko_matmul(C.byref(ko.mk_global(a, M, K, K, 1, dt)), C.byref(ko.mk_global(b, K, N, 1, K, dt)), None,
                              C.byref(ko.mk_global(want, M, N, N, 1, kh.F32)), kh.RN) == 0
    da, db = to_dev(a), to_dev(b)
    for tile, stages in (((0, 0, 0), 0), ((256, 256, 64), 25), ((128, 128, 64), 25)):
        pitch = N + 16    # the result is a window of a wider buffer
        dd = dev_zeros(M * pitch + 64, 4, fill=0x12345678)
        kh.matmul(dglobal(da, M, K, K, 1, dt), dglobal(db, K, N, 1, K, dt), dglobal(dd, M, N, pitch, 1, kh.F32), tile=tile, stages=stages)
        sync()
        got = to_host(dd, np.uint32)
        assert np.all(got[M * pitch:] == 0x12345678), tile
        rows = got[:M * pitch].reshape(M, pitch)
        assert np.all(rows[:, N:] == 0x12345678), tile
        assert _frob(ko, np.ascontiguousarray(rows[:, :N]).view(np.float32).reshape(-1), want, kh.F32) <= 1e-5, tile


@pytest.mark.parametrize("acc_dt,out_dt", [(kh.F32, kh.F32), (kh.F32, kh.BF16), (kh.F16, kh.F16), (kh.F16, kh.F32)])
@pytest.mark.parametrize("M,N,K", [(512, 512, 256), (300, 264, 192)])
def test_accumulator_input_through_the_strip_epilogue(ko, acc_dt, out_dt, M, N, K):
    """result = lhs x rhs + acc with a row-major acc whose rows are 16-byte aligned: the strip epilogue fetches the lane's 8
    acc values a strip ahead and adds them in fp32 before the final rounding; ragged extents drop out in the descriptors."""
    dt = kh.F16 if out_dt == kh.F16 or acc_dt == kh.F16 else kh.BF16
    a, b = ko.fill_normal(M * K, dt, 13, 0, 0.0, 0.5), ko.fill_normal(K * N, dt, 13, 1, 0.0, 0.5)
    acc = ko.fill_normal(M * N, acc_dt, 13, 2)
    want = np.zeros(M * N, dtype=_np_store(out_dt))
    assert ko.lib().ko_matmul(C.byref(ko.mk_global(a, M, K, K, 1, dt)), C.byref(ko.mk_global(b, K, N, 1, K, dt)), C.byref(ko.mk_global(acc, M, N, N, 1, acc_dt)),
                              C.byref(ko.mk_global(want, M, N, N, 1, out_dt)), kh.RN) == 0
    da, db, dacc = to_dev(a), to_dev(b), to_dev(acc)
    for tile, stages in (((0, 0, 0), 0), ((256, 256, 64), 25), ((128, 128, 64), 25)):
        dd = dev_zeros(M * N + 64, kh.DTYPE_BYTES[out_dt], fill=0x1234)
        kh.matmul(dglobal(da, M, K, K, 1, dt), dglobal(db, K, N, 1, K, dt), dglobal(dd, M, N, N, 1, out_dt), acc=dglobal(dacc, M, N, N, 1, acc_dt),
                  tile=tile, stages=stages)
        sync()
        got = to_host(dd, want.dtype.type if out_dt != kh.F32 else np.float32)
        assert np.all(to_host(dd, np.uint16 if out_dt != kh.F32 else np.uint32)[M * N:] == 0x1234), tile
        assert _frob(ko, got[:M * N], want, out_dt) <= (1e-5 if out_dt == kh.F32 else FROB_TOL), tile


@pytest.mark.parametrize("dt", [kh.F16, kh.BF16])
@pytest.mark.parametrize("a_rm,b_rm", [(True, True), (False, True), (False, False)])
@pytest.mark.parametrize("tile_k,stages", [(64, 4), (64, 3), (32, 4)])
def test_transposing_read_kernel_takes_either_operand_transposed(ko, dt, a_rm, b_rm, tile_k, stages):
    """A column-major lhs and / or a row-major rhs is staged as it lies and read with the transposing read (row-major x
    row-major is the reference fixture's layout): every form and ring depth against the oracle, K of several tiles so
    that the unrolled ring wraps, a last partial round of the unroll, and a result the tiles cover exactly."""
    for (M, N, K) in ((256, 384, 64 * 9), (128, 128, 64 * 4), (384, 256, 64 * 5)):
        got, want = _run(ko, dt, M, N, K, a_rm, b_rm, seed=21, tile=(128, 128, tile_k), stages=stages)
        assert _frob(ko, got, want, dt) <= FROB_TOL, (M, N, K)


@pytest.mark.parametrize("dt", [kh.F16, kh.BF16])
@pytest.mark.parametrize("a_rm,b_rm", [(True, True), (False, True), (False, False)])
def test_transposing_read_kernel_with_columns_that_do_not_fill_the_last_tile(ko, dt, a_rm, b_rm):
    """N a multiple of 8 but not of the 128-wide tile: the rhs descriptor ends with the rhs, the columns beyond it reach no
    stored result.  Against the oracle, with guard words behind the result; M ragged too where the lhs is row-major."""
    for (M, N, K, tile_k) in ((256 if not a_rm else 200, 136, 64 * 5, 64), (128, 1000, 32 * 7, 32), (384 if not a_rm else 333, 8, 64 * 4, 64)):
        a, b = ko.fill_uniform(M * K, dt, 23, 0), ko.fill_uniform(K * N, dt, 23, 1)
        a_str, b_str = ((K, 1) if a_rm else (1, M)), ((N, 1) if b_rm else (1, K))
        want = np.zeros(M * N, dtype=np.uint16)
        assert ko.lib().ko_matmul(C.byref(ko.mk_global(a, M, K, *a_str, dt)), C.byref(ko.mk_global(b, K, N, *b_str, dt)), None,
                                  C.byref(ko.mk_global(want, M, N, N, 1, dt)), kh.RN) == 0
        da, db, dd = to_dev(a), to_dev(b), dev_zeros(M * N + 256, 2, fill=0x1234)
        kh.matmul(dglobal(da, M, K, *a_str, dt), dglobal(db, K, N, *b_str, dt), dglobal(dd, M, N, N, 1, dt), tile=(128, 128, tile_k))
        sync()
        got = to_host(dd, np.uint16)
        assert np.all(got[M * N:] == 0x1234), (M, N, K)
        assert _frob(ko, got[:M * N], want, dt) <= FROB_TOL, (M, N, K)


@pytest.mark.parametrize("dt", [kh.F16, kh.BF16])
@pytest.mark.parametrize("a_rm,b_rm", [(True, True), (False, True), (False, False)])
def test_transposing_read_kernel_with_a_partial_last_k_tile(ko, dt, a_rm, b_rm):
    """K a multiple of 8 that the K-tile does not divide: the pieces of the last tile beyond K arrive as zeros.  The operands
    are followed in memory by large finite values and NaNs (a next row, another tensor): none of it may reach a result."""
    for (M, N, K) in ((128, 256, 1000), (256, 128, 72), (128, 136, 8), (384 if not a_rm else 200, 128, 64 * 5 + 8), (128, 128, 32 * 3 + 24)):
        a, b = ko.fill_uniform(M * K, dt, 27, 0), ko.fill_uniform(K * N, dt, 27, 1)
        a_str, b_str = ((K, 1) if a_rm else (1, M)), ((N, 1) if b_rm else (1, K))
        want = np.zeros(M * N, dtype=np.uint16)
        assert ko.lib().ko_matmul(C.byref(ko.mk_global(a, M, K, *a_str, dt)), C.byref(ko.mk_global(b, K, N, *b_str, dt)), None,
                                  C.byref(ko.mk_global(want, M, N, N, 1, dt)), kh.RN) == 0
        poison = np.full(4096, 0x7e00 if dt == kh.F16 else 0x7fc0, np.uint16)       # NaNs behind each operand
        da, db, dd = to_dev(np.concatenate([a, poison])), to_dev(np.concatenate([b, poison])), dev_zeros(M * N + 256, 2, fill=0x1234)
        kh.matmul(dglobal(da, M, K, *a_str, dt), dglobal(db, K, N, *b_str, dt), dglobal(dd, M, N, N, 1, dt))
        sync()
        got = to_host(dd, np.uint16)
        assert np.all(got[M * N:] == 0x1234), (M, N, K)
        assert _frob(ko, got[:M * N], want, dt) <= FROB_TOL, (M, N, K)


@pytest.mark.parametrize("M,N", [(3072, 3072), (3001, 3016)])   # (the second: tiles that hang over the last rows and columns)
@pytest.mark.parametrize("dt,acc_dt,out_dt", [("BF16", None, "BF16"), ("F16", None, "F16"), ("BF16", "F32", "F32"), ("F16", "F16", "F16")])
def test_large_row_major_operands_on_256_wide_tiles(ko, monkeypatch, dt, acc_dt, out_dt, M, N):
    """Row-major x row-major with at least 0.55 tiles of 256 x 256 per CU: the 256-wide kernel that stages the rhs as it lies and
    transposes it on the way out of LDS.  Sampled blocks against the checker (spread over the tile: every wavefront's part and
    both column halves of the rhs image), nothing written past the result, and the bits of the 128-wide kernel's result where no
    accumulator order differs - both sum K in ascending slices of 32 from zero - i.e. everywhere."""
    dt, out_dt = getattr(ko, dt), getattr(ko, out_dt)
    acc_dt = getattr(ko, acc_dt) if acc_dt else None
    K = 192
    ob = 4 if out_dt == ko.F32 else 2
    a, b = ko.fill_normal(M * K, dt, 51, 0, 0.0, 0.5), ko.fill_normal(K * N, dt, 51, 1, 0.0, 0.5)
    acc = ko.fill_normal(M * N, acc_dt, 51, 2, 0.0, 0.5) if acc_dt is not None else None
    poison = np.full(8192, 0x7e00 if dt == ko.F16 else 0x7fc0, np.uint16)       # NaNs behind each operand
    da, db = to_dev(np.concatenate([a, poison])), to_dev(np.concatenate([b, poison]))
    dacc = to_dev(acc) if acc is not None else None
    ga, gb = dglobal(da, M, K, K, 1, dt), dglobal(db, K, N, N, 1, dt)
    gacc = dglobal(dacc, M, N, N, 1, acc_dt) if acc is not None else None
    outs = []
    for wide in ("1", "0"):
        # (the switch is read once per process: the narrow run comes from an explicit 128-wide tile)
        dd = dev_zeros(M * N + 64, ob, fill=0x1234)
        kh.matmul(ga, gb, dglobal(dd, M, N, N, 1, out_dt), acc=gacc, **({} if wide == "1" else dict(tile=(128, 128, 64))))
        sync()
        got = to_host(dd, _np_store(out_dt))
        assert np.all(got[M * N:].view(np.uint32 if ob == 4 else np.uint16) == 0x1234)
        outs.append(got[:M * N].reshape(M, N))
    assert np.array_equal(outs[0].view(np.uint32 if ob == 4 else np.uint16), outs[1].view(np.uint32 if ob == 4 else np.uint16))
    goa, gob = ko.mk_global(a, M, K, K, 1, dt), ko.mk_global(b, K, N, N, 1, dt)
    goacc = ko.mk_global(acc, M, N, N, 1, acc_dt) if acc is not None else None
    for t in range(8):
        r0, c0 = (t * 331 + 37 * (t % 4) * 16) % (M - 64), (t * 577 + 128 * (t % 2)) % (N - 64)
        if t == 7:
            r0, c0 = M - 64, N - 64   # (the corner of the last tile)
        want = np.zeros((64, 64), _np_store(out_dt))
        assert ko.lib().ko_matmul(C.byref(ko.sv_global(goa, r0, r0 + 64, 0, K)), C.byref(ko.sv_global(gob, 0, K, c0, c0 + 64)),
                                  C.byref(ko.sv_global(goacc, r0, r0 + 64, c0, c0 + 64)) if goacc is not None else None,
                                  C.byref(ko.mk_global(want, 64, 64, 64, 1, out_dt)), kh.RN) == 0
        assert _frob(ko, np.ascontiguousarray(outs[0][r0:r0 + 64, c0:c0 + 64]).ravel(), want.ravel(), out_dt) <= FROB_TOL



@pytest.mark.parametrize("dt", [kh.F16, kh.BF16])
@pytest.mark.parametrize("a_rm,b_rm", [(True, True), (False, True), (False, False)])
def test_large_problem_with_a_workspace_turns_the_operand_first(ko, dt, a_rm, b_rm):
    """A row-major rhs / column-major lhs of a large problem, with a workspace of kapy_matmul_turn_workspace_bytes: the operand is
    turned K-contiguous into the workspace and the K-contiguous kernel multiplies.  Same result as the in-place kernel within the
    GEMM tolerance (sampled blocks against the checker), the counters at the head of the workspace stay zero, and a workspace
    that is too small changes nothing."""
    import torch
    M, N, K = 6144, 6400, 1024
    a, b = ko.fill_normal(M * K, dt, 41, 0, 0.0, 0.5), ko.fill_normal(K * N, dt, 41, 1, 0.0, 0.5)
    a_str, b_str = ((K, 1) if a_rm else (1, M)), ((N, 1) if b_rm else (1, K))
    da, db = to_dev(a), to_dev(b)
    ga, gb = dglobal(da, M, K, *a_str, dt), dglobal(db, K, N, *b_str, dt)
    need = kh.lib().kapy_matmul_turn_workspace_bytes(C.byref(ga), C.byref(gb))
    assert need == 16384 + (0 if a_rm else M * K * 2) + (K * N * 2 if b_rm else 0)
    outs = []
    for ws_bytes in (0, 4096 + 16384, need):
        ws = torch.zeros(ws_bytes, dtype=torch.uint8, device="cuda") if ws_bytes else None
        dd = dev_zeros(M * N + 256, 2, fill=0x1234)
        kh.matmul(ga, gb, dglobal(dd, M, N, N, 1, dt), workspace=ws)
        sync()
        got = to_host(dd, np.uint16)
        assert np.all(got[M * N:] == 0x1234)
        if ws is not None:
            assert not ws[:16384].any()
        outs.append(got[:M * N].reshape(M, N))
    assert np.array_equal(outs[0], outs[1])                      # too small a workspace: the in-place kernel, as without one
    goa, gob = ko.mk_global(a, M, K, *a_str, dt), ko.mk_global(b, K, N, *b_str, dt)
    for t in range(6):
        r0, c0 = (t * 331) % (M - 64), (t * 577) % (N - 64)
        want = np.zeros((64, 64), np.uint16)
        assert ko.lib().ko_matmul(C.byref(ko.sv_global(goa, r0, r0 + 64, 0, K)), C.byref(ko.sv_global(gob, 0, K, c0, c0 + 64)), None,
                                  C.byref(ko.mk_global(want, 64, 64, 64, 1, dt)), kh.RN) == 0
        for got in (outs[0], outs[2]):
            assert _frob(ko, np.ascontiguousarray(got[r0:r0 + 64, c0:c0 + 64]).ravel(), want.ravel(), dt) <= FROB_TOL
