"""GPU parity for fp8 (OCP E4M3FN / E5M2) matmuls with fp32 row/column scales (benchmark configuration 5)."""
import ctypes as C

import numpy as np
import pytest

import kapy_hip as kh
from gpu_util import dev_zeros, dglobal, sync, to_dev, to_host

pytestmark = pytest.mark.gpu
FROB_TOL = 1e-3
vp = lambda x: x.ctypes.data_as(C.c_void_p)


def _quantised(ko, M, N, K, seed=0):
    a = ko.fill_normal(M * K, ko.F32, seed, 0).reshape(M, K)
    w = ko.fill_normal(N * K, ko.F32, seed + 1, 0).reshape(N, K)   # W stored K-contiguous per output column
    aq, sa = np.zeros((M, K), np.uint8), np.zeros(M, np.float32)
    wq, sb = np.zeros((N, K), np.uint8), np.zeros(N, np.float32)
    ko.lib().ko_quantize_e4m3(vp(a), M, K, K, 1, 1, vp(aq), vp(sa))
    ko.lib().ko_quantize_e4m3(vp(w), N, K, K, 1, 1, vp(wq), vp(sb))
    return aq, sa, wq, sb


def _frob(ko, got, want, dt=kh.BF16):
    g, w = ko.decode(got, dt), ko.decode(want, dt)
    assert np.all(np.isfinite(g))
    return np.linalg.norm(g - w) / np.linalg.norm(w)


@pytest.mark.parametrize("M,N,K", [(16, 64, 128), (16, 256, 1024), (5, 48, 256), (33, 100, 384), (64, 64, 512), (5, 40, 2048), (33, 100, 3072),
                                   (64, 64, 4096), (1, 16, 1024)])
def test_scaled_f8_small(ko, M, N, K):
    aq, sa, wq, sb = _quantised(ko, M, N, K)
    want = np.zeros((M, N), dtype=np.uint16)
    rc = ko.lib().ko_matmul_scaled_f8(C.byref(ko.mk_global(aq, M, K, K, 1, ko.F8E4M3)), C.byref(ko.mk_global(wq, K, N, 1, K, ko.F8E4M3)),
                                      vp(sa), vp(sb), C.byref(ko.mk_global(want, M, N, N, 1, ko.BF16)))
    assert rc == 0
    da, dw, dsa, dsb, dd = to_dev(aq), to_dev(wq), to_dev(sa), to_dev(sb), dev_zeros(M * N, 2)
    kh.matmul_scaled_f8(dglobal(da, M, K, K, 1, kh.F8E4M3), dglobal(dw, K, N, 1, K, kh.F8E4M3), dsa.data_ptr(), dsb.data_ptr(),
                        dglobal(dd, M, N, N, 1, kh.BF16))
    sync()
    assert _frob(ko, to_host(dd, np.uint16, (M, N)), want) <= FROB_TOL


@pytest.mark.parametrize("M,N,K", [(17, 64, 512), (32, 96, 1024), (33, 100, 1536), (48, 32, 512), (49, 40, 2048), (64, 256, 4096), (24, 1000, 512),
                                   (64, 8, 512), (65, 64, 512), (80, 96, 1024), (81, 40, 512), (100, 100, 1536), (112, 32, 512), (113, 72, 1024),
                                   (128, 256, 2048), (129, 64, 512), (160, 48, 1024)])
@pytest.mark.parametrize("formats", [(0, 0), (1, 0)])
def test_scaled_f8_block_streaming_kernel(ko, M, N, K, formats):
    """17 .. 160 rows with K a multiple of 512: 32 columns x 32 / 48 / ... / 128 rows per workgroup, beyond 128 rows blocks of
    64 (row and column blocks that hang over M and N included), both operand formats in the first slot."""
    fa = (ko.F8E4M3, ko.F8E5M2)[formats[0]]
    aq, sa, wq, sb = _quantised(ko, M, N, K, seed=7)
    if formats[0]:      # the same values re-encoded as e5m2
        aq = ko.fptofp(np.ascontiguousarray(ko.decode(aq, ko.F8E4M3).astype(np.float32)), ko.F32, ko.F8E5M2).reshape(M, K)
    want = np.zeros((M, N), dtype=np.uint16)
    assert ko.lib().ko_matmul_scaled_f8(C.byref(ko.mk_global(aq, M, K, K, 1, fa)), C.byref(ko.mk_global(wq, K, N, 1, K, ko.F8E4M3)),
                                        vp(sa), vp(sb), C.byref(ko.mk_global(want, M, N, N, 1, ko.BF16))) == 0
    da, dw, dsa, dsb, dd = to_dev(aq), to_dev(wq), to_dev(sa), to_dev(sb), dev_zeros(M * N + 64, 2, fill=0x1234)
    kh.matmul_scaled_f8(dglobal(da, M, K, K, 1, fa), dglobal(dw, K, N, 1, K, kh.F8E4M3), dsa.data_ptr(), dsb.data_ptr(),
                        dglobal(dd, M, N, N, 1, kh.BF16))
    sync()
    got = to_host(dd, np.uint16)
    assert np.all(got[M * N:] == 0x1234)                      # nothing written past the result
    assert _frob(ko, got[:M * N].reshape(M, N), want) <= FROB_TOL


@pytest.mark.parametrize("M,N,K", [(128, 128, 128), (128, 256, 384), (256, 256, 256), (384, 128, 512), (512, 768, 1024), (1024, 2560, 256),
                                   (300, 520, 256), (1000, 136, 384), (129, 1001, 128), (300, 520, 272), (256, 256, 144),   # tiles hang over the edges of M, N and K
                                   (161, 8192, 256), (192, 4096, 512), (320, 2056, 128), (500, 8192, 128)])   # at most one tile per CU: the four-stage build
def test_scaled_f8_tiled_kernel(ko, M, N, K):
    """Rows >= 128 and extents multiples of the tile: the LDS-direct MFMA kernel (128- and 256-wide tiles)."""
    aq, sa, wq, sb = _quantised(ko, M, N, K, seed=3)
    want = np.zeros((M, N), dtype=np.uint16)
    assert ko.lib().ko_matmul_scaled_f8(C.byref(ko.mk_global(aq, M, K, K, 1, ko.F8E4M3)), C.byref(ko.mk_global(wq, K, N, 1, K, ko.F8E4M3)),
                                        vp(sa), vp(sb), C.byref(ko.mk_global(want, M, N, N, 1, ko.BF16))) == 0
    da, dw, dsa, dsb, dd = to_dev(aq), to_dev(wq), to_dev(sa), to_dev(sb), dev_zeros(M * N, 2)
    kh.matmul_scaled_f8(dglobal(da, M, K, K, 1, kh.F8E4M3), dglobal(dw, K, N, 1, K, kh.F8E4M3), dsa.data_ptr(), dsb.data_ptr(),
                        dglobal(dd, M, N, N, 1, kh.BF16))
    sync()
    assert _frob(ko, to_host(dd, np.uint16, (M, N)), want) <= FROB_TOL


def test_f8_tiled_mixed_formats_f32_result(ko):
    """e4m3 x e5m2 and e5m2 x e4m3 through the tiled kernel, fp32 result, no scales: checks the operand format
    selectors of the matrix instruction on both sides."""
    M, N, K = 256, 128, 256
    rng = np.random.default_rng(1)
    e4 = rng.integers(0x20, 0x50, size=(M, K)).astype(np.uint8) | (rng.integers(0, 2, size=(M, K)).astype(np.uint8) << 7)
    e5 = rng.integers(0x30, 0x48, size=(N, K)).astype(np.uint8) | (rng.integers(0, 2, size=(N, K)).astype(np.uint8) << 7)
    for (a, adt, b, bdt, m, n) in ((e4, ko.F8E4M3, e5, ko.F8E5M2, M, N), (e5, ko.F8E5M2, e4, ko.F8E4M3, N, M)):
        want = np.zeros((m, n), dtype=np.float32)
        assert ko.lib().ko_matmul(C.byref(ko.mk_global(a, m, K, K, 1, adt)), C.byref(ko.mk_global(b, K, n, 1, K, bdt)), None,
                                  C.byref(ko.mk_global(want, m, n, n, 1, ko.F32)), ko.RN) == 0
        da, db, dd = to_dev(a), to_dev(b), dev_zeros(m * n, 4)
        kh.matmul(dglobal(da, m, K, K, 1, adt), dglobal(db, K, n, 1, K, bdt), dglobal(dd, m, n, n, 1, kh.F32))
        sync()
        got = to_host(dd, np.float32, (m, n))
        assert np.linalg.norm(got - want) / np.linalg.norm(want) <= 1e-4


def test_plain_f8_matmul_mixed_formats_and_fallback(ko):
    """kapy.matmul on f8 operands without scales: e4m3 x e5m2 mix (Kapy.cpp:484-487), f32 result; and an
    operand layout only the element-wise kernel serves (row-major rhs)."""
    M, N, K = 32, 48, 256
    rng = np.random.default_rng(0)
    a = rng.integers(0, 256, size=(M, K)).astype(np.uint8)
    a[(a & 0x7F) == 0x7F] = 0x30                      # no NaN patterns (e4m3fn)
    b = rng.integers(0, 256, size=(N, K)).astype(np.uint8)
    b[(b & 0x7C) == 0x7C] = 0x3C                      # no inf/NaN patterns (e5m2)
    want = np.zeros((M, N), dtype=np.float32)
    assert ko.lib().ko_matmul(C.byref(ko.mk_global(a, M, K, K, 1, ko.F8E4M3)), C.byref(ko.mk_global(b, K, N, 1, K, ko.F8E5M2)), None,
                              C.byref(ko.mk_global(want, M, N, N, 1, ko.F32)), ko.RN) == 0
    da, db, dd = to_dev(a), to_dev(b), dev_zeros(M * N, 4)
    kh.matmul(dglobal(da, M, K, K, 1, kh.F8E4M3), dglobal(db, K, N, 1, K, kh.F8E5M2), dglobal(dd, M, N, N, 1, kh.F32))
    sync()
    got = to_host(dd, np.float32, (M, N))
    # full-range random fp8 bytes span 2^-16..2^15: the matrix core aligns 128 products to one exponent before
    # adding, so the error is above fp32 round-off but far inside the GEMM tolerance
    assert np.linalg.norm(got - want) / np.linalg.norm(want) <= FROB_TOL
    # rhs row-major (N contiguous): naive kernel
    bk = np.ascontiguousarray(b.T)                     # [K, N] row-major, same logical matrix
    dbk = to_dev(bk)
    dd.zero_()
    kh.matmul(dglobal(da, M, K, K, 1, kh.F8E4M3), dglobal(dbk, K, N, N, 1, kh.F8E5M2), dglobal(dd, M, N, N, 1, kh.F32))
    sync()
    got2 = to_host(dd, np.float32, (M, N))
    assert np.linalg.norm(got2 - want) / np.linalg.norm(want) <= 1e-5   # element-wise kernel: plain fp32 FMAs


def test_config5_decode_shape_m16(ko):
    """benchmark configuration 5, M = 16: N = K = 8192, scales amax/448, bf16 out; full oracle check."""
    M, N, K = 16, 8192, 8192
    aq, sa, wq, sb = _quantised(ko, M, N, K)
    want = np.zeros((M, N), dtype=np.uint16)
    assert ko.lib().ko_matmul_scaled_f8(C.byref(ko.mk_global(aq, M, K, K, 1, ko.F8E4M3)), C.byref(ko.mk_global(wq, K, N, 1, K, ko.F8E4M3)),
                                        vp(sa), vp(sb), C.byref(ko.mk_global(want, M, N, N, 1, ko.BF16))) == 0
    da, dw, dsa, dsb, dd = to_dev(aq), to_dev(wq), to_dev(sa), to_dev(sb), dev_zeros(M * N, 2)
    kh.matmul_scaled_f8(dglobal(da, M, K, K, 1, kh.F8E4M3), dglobal(dw, K, N, 1, K, kh.F8E4M3), dsa.data_ptr(), dsb.data_ptr(),
                        dglobal(dd, M, N, N, 1, kh.BF16))
    sync()
    assert _frob(ko, to_host(dd, np.uint16, (M, N)), want) <= FROB_TOL


def test_config5_m4096_sampled(ko):
    """benchmark configuration 5, M = 4096: oracle on 64x64 blocks spread over the result."""
    M, N, K = 4096, 8192, 8192
    aq, sa, wq, sb = _quantised(ko, M, N, K)
    da, dw, dsa, dsb, dd = to_dev(aq), to_dev(wq), to_dev(sa), to_dev(sb), dev_zeros(M * N, 2)
    kh.matmul_scaled_f8(dglobal(da, M, K, K, 1, kh.F8E4M3), dglobal(dw, K, N, 1, K, kh.F8E4M3), dsa.data_ptr(), dsb.data_ptr(),
                        dglobal(dd, M, N, N, 1, kh.BF16))
    sync()
    got = to_host(dd, np.uint16, (M, N))
    goa, gow = ko.mk_global(aq, M, K, K, 1, ko.F8E4M3), ko.mk_global(wq, K, N, 1, K, ko.F8E4M3)
    num = den = 0.0
    blk = 64
    for t in range(16):
        r0, c0 = (t * 256 + 29 * t) % (M - blk), ((15 - t) * 512 + 71 * t) % (N - blk)
        want = np.zeros((blk, blk), dtype=np.uint16)
        rs, cs = np.ascontiguousarray(sa[r0:r0 + blk]), np.ascontiguousarray(sb[c0:c0 + blk])
        assert ko.lib().ko_matmul_scaled_f8(C.byref(ko.sv_global(goa, r0, r0 + blk, 0, K)), C.byref(ko.sv_global(gow, 0, K, c0, c0 + blk)),
                                            vp(rs), vp(cs), C.byref(ko.mk_global(want, blk, blk, blk, 1, ko.BF16))) == 0
        g, w = ko.decode(got[r0:r0 + blk, c0:c0 + blk], ko.BF16), ko.decode(want, ko.BF16)
        num += ((g - w) ** 2).sum()
        den += (w ** 2).sum()
    assert np.sqrt(num / den) <= FROB_TOL


@pytest.mark.parametrize("M,N,K", [(512, 512, 512), (768, 256, 1280), (300, 520, 256), (1000, 264, 384), (257, 1000, 128), (512, 256, 272), (256, 512, 144),
                                   (640, 384, 128 * 7)])   # ragged M and N, a partial last K-tile, K-tile counts around the ring's unroll of five
def test_scaled_f8_256_tiles_on_the_16x16x128_instruction(ko, M, N, K):
    """The 256 x 256 x 128 ring kernel (two passes per tile on v_mfma_scale_f32_16x16x128_f8f6f4), asked for by tile size on
    shapes the library would give to the 128-wide tiles: tiles that hang over every edge, and nothing written past the result."""
    aq, sa, wq, sb = _quantised(ko, M, N, K, seed=5)
    want = np.zeros((M, N), dtype=np.uint16)
    assert ko.lib().ko_matmul_scaled_f8(C.byref(ko.mk_global(aq, M, K, K, 1, ko.F8E4M3)), C.byref(ko.mk_global(wq, K, N, 1, K, ko.F8E4M3)),
                                        vp(sa), vp(sb), C.byref(ko.mk_global(want, M, N, N, 1, ko.BF16))) == 0
    da, dw, dsa, dsb, dd = to_dev(aq), to_dev(wq), to_dev(sa), to_dev(sb), dev_zeros(M * N + 4096, 2, fill=0x1234)
    kh.matmul_scaled_f8(dglobal(da, M, K, K, 1, kh.F8E4M3), dglobal(dw, K, N, 1, K, kh.F8E4M3), dsa.data_ptr(), dsb.data_ptr(),
                        dglobal(dd, M, N, N, 1, kh.BF16), tile=(256, 256, 128))
    sync()
    got = to_host(dd, np.uint16)
    assert np.all(got[M * N:] == 0x1234)
    assert _frob(ko, got[:M * N].reshape(M, N), want) <= FROB_TOL


def test_f8_256_tiles_mixed_formats_f32_result(ko):
    """e4m3 x e5m2 and e5m2 x e4m3 through the 256-wide tiles, fp32 result, no scales: the format selectors of the in-place
    matrix instruction on both sides."""
    M, N, K = 512, 256, 384
    rng = np.random.default_rng(2)
    e4 = rng.integers(0x20, 0x50, size=(M, K)).astype(np.uint8) | (rng.integers(0, 2, size=(M, K)).astype(np.uint8) << 7)
    e5 = rng.integers(0x30, 0x48, size=(N, K)).astype(np.uint8) | (rng.integers(0, 2, size=(N, K)).astype(np.uint8) << 7)
    for (a, adt, b, bdt, m, n) in ((e4, ko.F8E4M3, e5, ko.F8E5M2, M, N), (e5, ko.F8E5M2, e4, ko.F8E4M3, N, M), (e5, ko.F8E5M2, e5, ko.F8E5M2, N, N)):
        want = np.zeros((m, n), dtype=np.float32)
        assert ko.lib().ko_matmul(C.byref(ko.mk_global(a, m, K, K, 1, adt)), C.byref(ko.mk_global(b, K, n, 1, K, bdt)), None,
                                  C.byref(ko.mk_global(want, m, n, n, 1, ko.F32)), ko.RN) == 0
        da, db, dd = to_dev(a), to_dev(b), dev_zeros(m * n, 4)
        kh.matmul(dglobal(da, m, K, K, 1, adt), dglobal(db, K, n, 1, K, bdt), dglobal(dd, m, n, n, 1, kh.F32), tile=(256, 256, 128))
        sync()
        got = to_host(dd, np.float32, (m, n))
        assert np.linalg.norm(got - want) / np.linalg.norm(want) <= 1e-4


@pytest.mark.parametrize("M,N,K", [(16, 128, 144), (200, 256, 400), (64, 264, 656), (1000, 1000, 1040), (1, 128, 128 + 16), (300, 520, 8256)])
def test_scaled_f8_with_k_of_whole_16_byte_pieces_takes_the_tiled_kernel(ko, M, N, K):
    """K a multiple of 16 but not of 128, any number of rows: the tiled ring kernel with a partial last K-tile (the streaming
    kernels for few rows need whole 128-byte K steps).  Guard words behind the result."""
    aq, sa, wq, sb = _quantised(ko, M, N, K, seed=9)
    want = np.zeros((M, N), dtype=np.uint16)
    assert ko.lib().ko_matmul_scaled_f8(C.byref(ko.mk_global(aq, M, K, K, 1, ko.F8E4M3)), C.byref(ko.mk_global(wq, K, N, 1, K, ko.F8E4M3)),
                                        vp(sa), vp(sb), C.byref(ko.mk_global(want, M, N, N, 1, ko.BF16))) == 0
    da, dw, dsa, dsb, dd = to_dev(aq), to_dev(wq), to_dev(sa), to_dev(sb), dev_zeros(M * N + 4096, 2, fill=0x1234)
    kh.matmul_scaled_f8(dglobal(da, M, K, K, 1, kh.F8E4M3), dglobal(dw, K, N, 1, K, kh.F8E4M3), dsa.data_ptr(), dsb.data_ptr(),
                        dglobal(dd, M, N, N, 1, kh.BF16))
    sync()
    got = to_host(dd, np.uint16)
    assert np.all(got[M * N:] == 0x1234)
    assert _frob(ko, got[:M * N].reshape(M, N), want) <= FROB_TOL


@pytest.mark.parametrize("M,N,K", [(100, 200, 100), (64, 64, 8200), (130, 70, 24), (1, 4096, 40), (257, 129, 1000)])
def test_scaled_f8_with_rows_that_are_not_16_byte_aligned(ko, M, N, K):
    """K not a multiple of 16: no vector load reaches these rows; the tiled fp32 kernel for everything else.  Guard words."""
    aq, sa, wq, sb = _quantised(ko, M, N, K, seed=11)
    want = np.zeros((M, N), dtype=np.uint16)
    assert ko.lib().ko_matmul_scaled_f8(C.byref(ko.mk_global(aq, M, K, K, 1, ko.F8E4M3)), C.byref(ko.mk_global(wq, K, N, 1, K, ko.F8E4M3)),
                                        vp(sa), vp(sb), C.byref(ko.mk_global(want, M, N, N, 1, ko.BF16))) == 0
    da, dw, dsa, dsb, dd = to_dev(aq), to_dev(wq), to_dev(sa), to_dev(sb), dev_zeros(M * N + 4096, 2, fill=0x1234)
    kh.matmul_scaled_f8(dglobal(da, M, K, K, 1, kh.F8E4M3), dglobal(dw, K, N, 1, K, kh.F8E4M3), dsa.data_ptr(), dsb.data_ptr(),
                        dglobal(dd, M, N, N, 1, kh.BF16))
    sync()
    got = to_host(dd, np.uint16)
    assert np.all(got[M * N:] == 0x1234)
    assert _frob(ko, got[:M * N].reshape(M, N), want) <= FROB_TOL
