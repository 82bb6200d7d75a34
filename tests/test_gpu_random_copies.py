"""Seeded random layout moves (ld_global -> [transpose] -> st_global): random element size, extents, row pitches, windows
into larger buffers, row- or column-major source and destination, a destination larger than the source (padding), every
padding pattern.  Bit-exact against the oracle, and nothing outside the destination window may change."""
import ctypes as C

import numpy as np
import pytest

import kapy_hip as kh
from gpu_util import dglobal, sync, to_dev, to_host

pytestmark = pytest.mark.gpu
NP = {1: np.uint8, 2: np.uint16, 4: np.uint32}


def _view(rng, rows, cols, itemsize):
    """A rows x cols window: (buffer elements, offset, stride0, stride1), row- or column-major, with a pitch that may exceed the
    extent and may or may not keep 16-byte alignment."""
    col_major = rng.randint(3) == 0
    lead, other = (rows, cols) if col_major else (cols, rows)       # lead: extent along the contiguous axis
    pitch = lead + [0, 0, 8, 16 // itemsize, 3, 1][rng.randint(6)]
    offset = [0, 0, 16 // itemsize, 5][rng.randint(4)]
    count = offset + pitch * other + 8
    return count, offset, (1, pitch) if col_major else (pitch, 1)


@pytest.mark.parametrize("seed", range(80))
def test_random_copy(ko, seed):
    rng = np.random.RandomState(7000 + seed)
    dtype = [kh.F16, kh.BF16, kh.F32, kh.F8E4M3, kh.I8, kh.F16, kh.BF16][rng.randint(7)]
    b = kh.DTYPE_BYTES[dtype]
    m, n = [(64, 64), (128, 128), (256, 384), (37, 53), (200, 136), (8, 1000), (129, 257), (1, 77), (300, 16), (144, 72)][rng.randint(10)]
    transpose = bool(rng.randint(2))
    dm, dn = (n, m) if transpose else (m, n)
    grow = rng.randint(4) == 0                               # destination larger than the source: the excess is padding
    if grow:
        dm, dn = dm + [0, 3, 16][rng.randint(3)], dn + [0, 5, 8][rng.randint(3)]
    pad = [kh.PAD_ZERO, kh.PAD_QNAN, kh.PAD_PINF, kh.PAD_NINF][rng.randint(4)] if grow and dtype in (kh.F16, kh.BF16, kh.F32, kh.F8E4M3) else kh.PAD_ZERO
    s_count, s_off, s_str = _view(rng, m, n, b)
    d_count, d_off, d_str = _view(rng, dm, dn, b)
    src = rng.randint(0, 2 ** (8 * min(b, 4) - (1 if b == 4 else 0)), size=s_count).astype(NP[b])
    fill = 0x5A5A5A5A & (2 ** (8 * b) - 1)
    want = np.full(d_count, fill, NP[b])
    so = ko.mk_global(src[s_off:], m, n, s_str[0], s_str[1], dtype)
    do = ko.mk_global(want[d_off:], dm, dn, d_str[0], d_str[1], dtype)
    describe = "seed %d: dtype %d %dx%d %s-> %dx%d, src strides %s offset %d, dst strides %s offset %d, pad %d" % (
        seed, dtype, m, n, "transposed " if transpose else "", dm, dn, s_str, s_off, d_str, d_off, pad)
    assert ko.lib().ko_copy(C.byref(so), C.byref(do), int(transpose), pad) == 0, describe
    d_src, d_dst = to_dev(src), to_dev(np.full(d_count, fill, NP[b]))
    sd = dglobal(d_src, m, n, s_str[0], s_str[1], dtype, dynamic_offset=s_off)
    dd = dglobal(d_dst, dm, dn, d_str[0], d_str[1], dtype, dynamic_offset=d_off)
    kh.copy(sd, dd, transpose=transpose, padding=pad)
    sync()
    got = to_host(d_dst, NP[b])
    bad = np.flatnonzero(got != want)
    assert len(bad) == 0, "%s: %d elements differ, first at %d (got %#x want %#x)" % (describe, len(bad), bad[0], got[bad[0]], want[bad[0]])
