"""GPU parity for the layout moves (ld_global -> [transpose] -> st_global): bit-exact against the
oracle on small / ragged / strided cases and against closed forms at the benchmark sizes."""
import ctypes as C

import numpy as np
import pytest

import kapy_hip as kh
from gpu_util import dev_zeros, dglobal, sync, to_dev, to_host

pytestmark = pytest.mark.gpu

NP = {1: np.uint8, 2: np.uint16, 4: np.uint32}


def _rand(n, itemsize, seed):
    rng = np.random.default_rng(seed)
    return rng.integers(0, 2 ** (8 * itemsize), size=n, dtype=np.uint64).astype(NP[itemsize])


CASES = [
    # (dtype, src_shape(m,n), transpose, use swapped strides, view (s0,e0,s1,e1) or None)
    (kh.F16, (64, 64), True, False, None),
    (kh.F16, (128, 192), True, False, None),
    (kh.BF16, (37, 53), True, False, None),           # ragged: generic + edge tiles
    (kh.F16, (200, 136), True, False, None),          # interior tiles + ragged edges (136 % 8 == 0)
    (kh.F16, (128, 128), False, True, None),          # transpose expressed by swapped source strides
    (kh.F32, (96, 160), True, False, None),
    (kh.F8E4M3, (256, 384), True, False, None),
    (kh.I8, (130, 70), True, False, None),
    (kh.F16, (77, 129), False, False, None),          # plain ragged row copy
    (kh.F32, (64, 256), False, False, (3, 60, 8, 200)),  # sub-view copy
    (kh.F16, (256, 256), True, False, (64, 192, 32, 160)),
]


@pytest.mark.parametrize("dtype,shape,transpose,swapped,view", CASES)
def test_copy_matches_oracle(ko, dtype, shape, transpose, swapped, view):
    b = kh.DTYPE_BYTES[dtype]
    m, n = shape
    src = _rand(m * n, b, 7).reshape(m, n)
    if swapped:
        ssz, sst = (n, m), (1, n)
    else:
        ssz, sst = (m, n), (n, 1)
    logical = (ssz[1], ssz[0]) if transpose else ssz
    dm, dn = logical
    d_src = to_dev(src)
    want = np.full((dm, dn), 0x5A, dtype=NP[b]) if b == 1 else np.full((dm, dn), 0x5A5A, dtype=NP[b])
    d_dst = to_dev(want)
    gs_o, gd_o = ko.mk_global(src, ssz[0], ssz[1], sst[0], sst[1], dtype), ko.mk_global(want, dm, dn, dn, 1, dtype)
    gs_d, gd_d = dglobal(d_src, ssz[0], ssz[1], sst[0], sst[1], dtype), dglobal(d_dst, dm, dn, dn, 1, dtype)
    if view:
        s0, e0, s1, e1 = view
        vs = (s1, e1, s0, e0) if transpose else view
        gs_o, gs_d = ko.sv_global(gs_o, *vs), kh.sv_global(gs_d, *vs)
        gd_o, gd_d = ko.sv_global(gd_o, *view), kh.sv_global(gd_d, *view)
    assert ko.lib().ko_copy(C.byref(gs_o), C.byref(gd_o), int(transpose), 0) == 0
    kh.copy(gs_d, gd_d, transpose=transpose)
    sync()
    got = to_host(d_dst, NP[b], (dm, dn))
    assert np.array_equal(got, want)


@pytest.mark.parametrize("pad", [kh.PAD_ZERO, kh.PAD_QNAN, kh.PAD_PINF, kh.PAD_NINF])
def test_padding_for_out_of_bounds_source(ko, pad):
    """Destination larger than the source view: the excess reads as the padding pattern."""
    src = _rand(40 * 48, 2, 3).reshape(40, 48)
    want = np.zeros((64, 64), dtype=np.uint16)
    d_src, d_dst = to_dev(src), dev_zeros(64 * 64, 2, 0x1111)
    for tr in (False, True):
        ssz = (48, 40) if tr else (40, 48)
        so = ko.mk_global(src, 40, 48, 48, 1, ko.BF16)
        sd = dglobal(d_src, 40, 48, 48, 1, kh.BF16)
        assert ko.lib().ko_copy(C.byref(so), C.byref(ko.mk_global(want, 64, 64, 64, 1, ko.BF16)), int(tr), pad) == 0
        kh.copy(sd, dglobal(d_dst, 64, 64, 64, 1, kh.BF16), transpose=tr, padding=pad)
        sync()
        assert np.array_equal(to_host(d_dst, np.uint16, (64, 64)), want)
        assert want[ssz[0]:, :].min() == want[ssz[0]:, :].max() == {0: 0, 1: 0x7FC0, 2: 0x7F80, 3: 0xFF80}[pad]


def test_column_major_destination_and_no_contiguous_axis(ko):
    src = _rand(96 * 80, 2, 11).reshape(96, 80)
    d_src = to_dev(src)
    # destination column-major (stride0 == 1): same-axis copy in the transposed orientation
    want = np.zeros((80, 96), dtype=np.uint16)   # holds dst^T
    d_dst = dev_zeros(80 * 96, 2)
    ko.lib().ko_copy(C.byref(ko.mk_global(src, 96, 80, 80, 1, 0)), C.byref(ko.mk_global(want, 96, 80, 1, 96, 0)), 0, 0)
    kh.copy(dglobal(d_src, 96, 80, 80, 1, kh.F16), dglobal(d_dst, 96, 80, 1, 96, kh.F16))
    sync()
    assert np.array_equal(to_host(d_dst, np.uint16, (80, 96)), want) and np.array_equal(want, src.T)
    # every-other-element destination: no contiguous axis -> generic kernel
    want2 = np.zeros(96 * 80 * 2, dtype=np.uint16)
    d_dst2 = dev_zeros(96 * 80 * 2, 2)
    ko.lib().ko_copy(C.byref(ko.mk_global(src, 96, 80, 80, 1, 0)), C.byref(ko.mk_global(want2, 96, 80, 160, 2, 0)), 0, 0)
    kh.copy(dglobal(d_src, 96, 80, 80, 1, kh.F16), dglobal(d_dst2, 96, 80, 160, 2, kh.F16))
    sync()
    assert np.array_equal(to_host(d_dst2, np.uint16), want2)


def test_empty_views_are_no_ops():
    d = dev_zeros(64, 2, 0x7777)
    g = dglobal(d, 8, 8, 8, 1, kh.F16)
    kh.copy(kh.sv_global(g, 2, 2, 0, 8), kh.sv_global(g, 4, 4, 0, 8))
    kh.copy(g, kh.sv_global(g, 0, 8, 3, 3), transpose=True)
    sync()
    assert np.all(to_host(d, np.uint16) == 0x7777)


def test_bhsd_permute_small_matches_oracle(ko):
    b, h, s, d = 2, 3, 40, 64
    src = ko.fill_bits16(b * h * s * d, 1).reshape(b, h, s, d)
    want = np.zeros((b, s, h, d), dtype=np.uint16)
    ko.lib().ko_copy_batched(C.byref(ko.mk_global(src, s, d, d, 1, ko.BF16)), C.byref(ko.mk_global(want, s, d, h * d, 1, ko.BF16)),
                             0, 0, b, h, h * s * d, s * d, s * h * d, d)
    d_src, d_dst = to_dev(src), dev_zeros(b * s * h * d, 2)
    kh.copy_batched(dglobal(d_src, s, d, d, 1, kh.BF16), dglobal(d_dst, s, d, h * d, 1, kh.BF16),
                    (b, h, h * s * d, s * d, s * h * d, d))
    sync()
    got = to_host(d_dst, np.uint16, (b, s, h, d))
    assert np.array_equal(got, want) and np.array_equal(got, src.transpose(0, 2, 1, 3))


def test_config3a_transpose_8192_bit_exact(ko):
    """benchmark configuration 3a: fp16 8192x8192 (i,j)->(j,i), random 16-bit patterns from seed 0."""
    n = 8192
    src = ko.fill_bits16(n * n, 0).reshape(n, n)
    d_src, d_dst = to_dev(src), dev_zeros(n * n, 2)
    gs, gd = dglobal(d_src, n, n, n, 1, kh.F16), dglobal(d_dst, n, n, n, 1, kh.F16)
    kh.copy(gs, gd, transpose=True)
    sync()
    got = to_host(d_dst, np.uint16, (n, n))
    assert np.array_equal(got, src.T)                      # closed form: out[j,i] = in[i,j]
    assert int(np.bitwise_xor.reduce(got.ravel())) == int(np.bitwise_xor.reduce(src.ravel()))
    # oracle on a band of destination rows (sub-views of both sides)
    want = np.zeros((64, n), dtype=np.uint16)
    so = ko.sv_global(ko.mk_global(src, n, n, n, 1, ko.F16), 0, n, 4096, 4160)
    assert ko.lib().ko_copy(C.byref(so), C.byref(ko.mk_global(want, 64, n, n, 1, ko.F16)), 1, 0) == 0
    assert np.array_equal(got[4096:4160], want)
    # involution: transposing again restores the input bit for bit
    kh.copy(gd, gs, transpose=True)
    sync()
    assert np.array_equal(to_host(d_src, np.uint16, (n, n)), src)
    # the same move expressed with swapped source strides
    d_dst.zero_()
    kh.copy(dglobal(d_src, n, n, 1, n, kh.F16), gd)
    sync()
    assert np.array_equal(to_host(d_dst, np.uint16, (n, n)), src.T)


def test_config3b_permute_bhsd_bit_exact(ko):
    """benchmark configuration 3b: bf16 [8,32,2048,128] (b,h,s,d)->(b,s,h,d), random bits from seed 1."""
    b, h, s, d = 8, 32, 2048, 128
    src = ko.fill_bits16(b * h * s * d, 1).reshape(b, h, s, d)
    d_src, d_dst = to_dev(src), dev_zeros(b * h * s * d, 2)
    kh.copy_batched(dglobal(d_src, s, d, d, 1, kh.BF16), dglobal(d_dst, s, d, h * d, 1, kh.BF16),
                    (b, h, h * s * d, s * d, s * h * d, d))
    sync()
    got = to_host(d_dst, np.uint16, (b, s, h, d))
    assert np.array_equal(got, src.transpose(0, 2, 1, 3))
    # and back: (b,s,h,d) -> (b,h,s,d)
    d_back = dev_zeros(b * h * s * d, 2)
    kh.copy_batched(dglobal(d_dst, s, d, h * d, 1, kh.BF16), dglobal(d_back, s, d, d, 1, kh.BF16),
                    (b, h, s * h * d, d, h * s * d, s * d))
    sync()
    assert np.array_equal(to_host(d_back, np.uint16, (b, h, s, d)), src)


def test_cache_hints_do_not_change_results(ko):
    """EvictPriority and isVolatile of create_ld_global / create_st_global (python/src/ir.cc:1035-1049) choose between
    ordinary and non-temporal access; the bits moved are the same under every combination, transposed or not."""
    m, n = 256, 320
    src = ko.fill_bits16(m * n, 5).reshape(m, n)
    d_src = to_dev(src)
    for transpose in (False, True):
        want = src.T if transpose else src
        dm, dn = want.shape
        for cache, evict, vol in ((kh.CACHE_NONE, kh.EVICT_NORMAL, False), (kh.CACHE_NONE, kh.EVICT_FIRST, False), (kh.CACHE_NONE, kh.NO_ALLOCATE, False),
                                  (kh.CACHE_NONE, kh.EVICT_LAST, False), (kh.CACHE_NONE, kh.EVICT_UNCHANGED, False), (kh.CACHE_CS, kh.EVICT_LAST, False),
                                  (kh.CACHE_CS, kh.EVICT_FIRST, True), (kh.CACHE_CA, kh.EVICT_FIRST, False)):
            d_dst = dev_zeros(m * n, 2, fill=0x5A5A)
            kh.copy(dglobal(d_src, m, n, n, 1, kh.F16), dglobal(d_dst, dm, dn, dn, 1, kh.F16), transpose=transpose, cache=cache, evict=evict, volatile=vol)
            sync()
            assert np.array_equal(to_host(d_dst, np.uint16, (dm, dn)), want), (transpose, cache, evict, vol)


@pytest.mark.parametrize("rows,cols", [(4096, 8192), (8192, 4096), (6144, 5632)])
def test_transpose_with_256_tiles_on_windows_of_wider_buffers(ko, rows, cols):
    """Extents that 256 x 256 tiles divide, with enough tiles to fill the chip, take the large-tile form of the LDS transpose;
    source and destination are windows of wider buffers (pitches larger than the extents), and the words beside and behind
    the destination window must stay as they were."""
    sp, dp = cols + 64, rows + 128
    src = ko.fill_bits16(rows * sp, 3).reshape(rows, sp)
    d_src, d_dst = to_dev(src), dev_zeros(cols * dp + 256, 2, fill=0x5A5A)
    kh.copy(dglobal(d_src, rows, cols, sp, 1, kh.F16), dglobal(d_dst, cols, rows, dp, 1, kh.F16), transpose=True)
    sync()
    got = to_host(d_dst, np.uint16)
    assert np.all(got[cols * dp:] == 0x5A5A)
    win = got[:cols * dp].reshape(cols, dp)
    assert np.all(win[:, rows:] == 0x5A5A)
    assert np.array_equal(win[:, :rows], src[:, :cols].T)


@pytest.mark.parametrize("rows,cols", [(136, 200), (3000, 5000), (264, 392), (128, 136), (1032, 128), (8200, 8184)])
def test_transpose_whose_tiles_hang_over_the_edge_in_whole_blocks(ko, rows, cols):
    """Extents that are multiples of 8 but not of the tile: the tiles over the edge take the block path with the blocks beyond
    the edge left out.  Windows of wider buffers, guard words beside and behind the destination window."""
    sp, dp = cols + 8, rows + 24
    src = ko.fill_bits16(rows * sp, 5).reshape(rows, sp)
    d_src, d_dst = to_dev(src), dev_zeros(cols * dp + 256, 2, fill=0x5A5A)
    kh.copy(dglobal(d_src, rows, cols, sp, 1, kh.F16), dglobal(d_dst, cols, rows, dp, 1, kh.F16), transpose=True)
    sync()
    got = to_host(d_dst, np.uint16)
    assert np.all(got[cols * dp:] == 0x5A5A)
    win = got[:cols * dp].reshape(cols, dp)
    assert np.all(win[:, rows:] == 0x5A5A)
    assert np.array_equal(win[:, :rows], src[:, :cols].T)


@pytest.mark.parametrize("dtype", [kh.F16, kh.F32, kh.F8E4M3])
@pytest.mark.parametrize("rows,cols", [(301, 501), (17, 3), (3001, 5001), (2, 7)])
def test_dense_copy_with_odd_widths_moves_as_one_line(ko, dtype, rows, cols):
    """Two dense matrices of one shape are one line of rows * cols elements, whatever the width; guard words intact."""
    eb = kh.DTYPE_BYTES[dtype]
    np_t = {1: np.uint8, 2: np.uint16, 4: np.uint32}[eb]
    src = np.random.RandomState(rows * 7 + cols).randint(0, 2 ** (8 * eb - 1), size=rows * cols).astype(np_t)
    d_src, d_dst = to_dev(src), dev_zeros(rows * cols + 64, eb, fill=0x5A)
    kh.copy(dglobal(d_src, rows, cols, cols, 1, dtype), dglobal(d_dst, rows, cols, cols, 1, dtype))
    sync()
    got = to_host(d_dst, np_t)
    assert np.array_equal(got[:rows * cols], src) and np.all(got[rows * cols:] == got[-1]) and got[-1] != 0


@pytest.mark.parametrize("dtype", [kh.F16, kh.F32, kh.F8E4M3])
@pytest.mark.parametrize("rows,cols", [(301, 501), (17, 33), (3001, 5001), (64, 65), (1000, 16)])
def test_transpose_with_extents_no_vector_reaches(ko, dtype, rows, cols):
    """Extents that are not multiples of 8 (rows that are not 16-byte aligned): 64 x 64 tiles through LDS element by element.
    Windows of wider buffers, guard words beside and behind the destination window; against numpy's transpose."""
    eb = kh.DTYPE_BYTES[dtype]
    np_t = {1: np.uint8, 2: np.uint16, 4: np.uint32}[eb]
    sp, dp = cols + 3, rows + 5
    src = np.random.RandomState(rows * 11 + cols).randint(1, 2 ** (8 * eb - 1), size=rows * sp).astype(np_t).reshape(rows, sp)
    d_src, d_dst = to_dev(src), dev_zeros(cols * dp + 64, eb, fill=0x5A)
    kh.copy(dglobal(d_src, rows, cols, sp, 1, dtype), dglobal(d_dst, cols, rows, dp, 1, dtype), transpose=True)
    sync()
    got = to_host(d_dst, np_t)
    guard = got[-1]
    assert guard != 0 and np.all(got[cols * dp:] == guard)
    win = got[:cols * dp].reshape(cols, dp)
    assert np.all(win[:, rows:] == guard)
    assert np.array_equal(win[:, :rows], src[:, :cols].T)
