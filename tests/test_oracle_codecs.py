"""Pins the oracle's float codecs against independent implementations (numpy float16, torch CPU
casts) and against the constants the reference itself holds."""
import ctypes as C

import numpy as np
import pytest
import torch


def test_f16_decode_exhaustive(ko):
    bits = np.arange(65536, dtype=np.uint16)
    want = bits.view(np.float16).astype(np.float64)
    got = np.array([ko.lib().ko_f16_to_f64(int(b)) for b in bits])
    assert np.array_equal(np.isnan(want), np.isnan(got))
    m = ~np.isnan(want)
    assert np.array_equal(want[m], got[m])
    assert np.array_equal(np.signbit(want[m]), np.signbit(got[m]))


def _rand_f32(n, seed):
    rng = np.random.default_rng(seed)
    raw = rng.integers(0, 2**32, size=n, dtype=np.uint64).astype(np.uint32)
    return raw.view(np.float32)


def test_f16_encode_rn_vs_numpy(ko):
    x = np.concatenate([_rand_f32(200000, 1), np.float32(np.random.default_rng(2).normal(0, 1, 200000)),
                        np.float32(np.random.default_rng(3).normal(0, 1e-6, 50000))])
    # every midpoint between adjacent finite f16 values and its fp32 neighbours (tie handling)
    h = np.arange(0, 0x7C00, dtype=np.uint16).view(np.float16).astype(np.float64)
    mid = ((h[:-1] + h[1:]) / 2).astype(np.float32)
    x = np.concatenate([x, mid, np.nextafter(mid, np.float32(0)), np.nextafter(mid, np.float32(np.inf)), -mid,
                        np.float32([65504, 65519.99, 65520, 65536, 1e9, np.inf, -np.inf, 0.0, -0.0])])
    with np.errstate(over="ignore"):
        want = x.astype(np.float16).view(np.uint16)
    got = ko.fptofp(x, ko.F32, ko.F16, ko.RN)
    nan = np.isnan(x)
    assert np.array_equal(want[~nan], got[~nan])
    assert np.all(np.isnan(got[nan].view(np.float16)))


def test_f16_encode_rz(ko):
    x = np.concatenate([_rand_f32(100000, 5), np.float32(np.random.default_rng(6).normal(0, 10, 100000))])
    x = x[np.isfinite(x)]
    got = ko.fptofp(x, ko.F32, ko.F16, ko.RZ).view(np.float16).astype(np.float64)
    # RZ: largest-magnitude representable value not exceeding |x|; overflow clamps to max finite
    with np.errstate(over="ignore"):
        rn = x.astype(np.float16)
    rnv = rn.astype(np.float64)
    toward0 = np.nextafter(rn, np.float16(0)).astype(np.float64)
    want = np.where(np.abs(rnv) > np.abs(x.astype(np.float64)), toward0, rnv)
    want = np.where(np.isinf(want), np.sign(want) * 65504.0, want)
    assert np.array_equal(want, got)


def test_bf16_vs_torch(ko):
    x = np.concatenate([_rand_f32(300000, 7), np.float32(np.random.default_rng(8).normal(0, 0.02, 100000))])
    nan = np.isnan(x)
    want = torch.from_numpy(x).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    got = ko.fptofp(x, ko.F32, ko.BF16, ko.RN)
    assert np.array_equal(want[~nan], got[~nan])
    # decode: bf16 is the top half of an fp32
    bits = np.arange(65536, dtype=np.uint16)
    want_d = (bits.astype(np.uint32) << 16).view(np.float32).astype(np.float64)
    got_d = np.array([ko.lib().ko_bf16_to_f64(int(b)) for b in bits])
    m = ~np.isnan(want_d)
    assert np.array_equal(want_d[m], got_d[m]) and np.all(np.isnan(got_d[~m]))
    # RZ = truncation of the low 16 bits
    fin = x[np.isfinite(x)]
    assert np.array_equal(ko.fptofp(fin, ko.F32, ko.BF16, ko.RZ), (fin.view(np.uint32) >> 16).astype(np.uint16))


def test_e4m3fn_table_closed_form(ko):
    # OCP E4M3FN: bias 7, no infinities, NaN = S.1111.111, max finite 448, min subnormal 2^-9
    for b in range(256):
        s, e, m = b >> 7, (b >> 3) & 15, b & 7
        v = ko.lib().ko_e4m3_to_f64(b)
        if e == 15 and m == 7:
            assert np.isnan(v)
            continue
        want = (m / 8.0) * 2.0 ** -6 if e == 0 else (1 + m / 8.0) * 2.0 ** (e - 7)
        assert v == (-want if s else want)
    assert ko.lib().ko_e4m3_to_f64(0x7E) == 448.0 and ko.lib().ko_e4m3_to_f64(0x01) == 2.0 ** -9


def test_e4m3fn_encode_vs_torch_and_saturation(ko):
    # all 65536 fp16 inputs, as the reference's f16->e4m3 cast sees them
    h = np.arange(65536, dtype=np.uint16)
    x = h.view(np.float16).astype(np.float32)
    got = ko.fptofp(h, ko.F16, ko.F8E4M3, ko.RN)
    want = torch.from_numpy(x).to(torch.float8_e4m3fn).view(torch.uint8).numpy()
    inr = np.isfinite(x) & (np.abs(x) < 464.0)  # torch overflows to NaN instead of saturating
    assert np.array_equal(want[inr], got[inr])
    over = np.isfinite(x) & (np.abs(x) >= 464.0) | np.isinf(x)
    assert np.array_equal(got[over], np.where(np.signbit(x[over]), 0xFE, 0x7E).astype(np.uint8))
    assert np.all((got[np.isnan(x)] & 0x7F) == 0x7F)
    # fp32 midpoints between adjacent e4m3 values: ties-to-even
    vals = np.array([ko.lib().ko_e4m3_to_f64(b) for b in range(0x7F)])
    mids = ((vals[:-1] + vals[1:]) / 2).astype(np.float32)
    gm = ko.fptofp(mids, ko.F32, ko.F8E4M3, ko.RN)
    assert np.array_equal(gm, np.array([b if b % 2 == 0 else b + 1 for b in range(0x7E)], dtype=np.uint8))


def test_e5m2_vs_torch(ko):
    h = np.arange(65536, dtype=np.uint16)
    x = h.view(np.float16).astype(np.float32)
    got = ko.fptofp(h, ko.F16, ko.F8E5M2, ko.RN)
    want = torch.from_numpy(x).to(torch.float8_e5m2).view(torch.uint8).numpy()
    inr = np.isfinite(x) & (np.abs(x) < 61440.0)
    assert np.array_equal(want[inr], got[inr])
    over = (np.isfinite(x) & (np.abs(x) >= 61440.0)) | np.isinf(x)
    assert np.array_equal(got[over], np.where(np.signbit(x[over]), 0xFB, 0x7B).astype(np.uint8))  # satfinite
    # e5m2 is the top byte of an fp16: RZ = truncation (the reference's bit-trick path)
    fin = h[np.isfinite(x)]
    assert np.array_equal(ko.fptofp(fin, ko.F16, ko.F8E5M2, ko.RZ), (fin >> 8).astype(np.uint8))
    # decode
    for b in range(256):
        v = ko.lib().ko_e5m2_to_f64(b)
        w = float(np.array([b << 8], dtype=np.uint16).view(np.float16)[0])
        assert (np.isnan(v) and np.isnan(w)) or v == w


def test_padding_words_match_reference_constants(ko):
    # known answers held by the reference: lib/Conversion/KgpuToLLVM/ConvertUtils.cpp:267-334
    ref = {(ko.F32, ko.PAD_QNAN): 0x7FC00000, (ko.F32, ko.PAD_PINF): 0x7F800000, (ko.F32, ko.PAD_NINF): 0xFF800000,
           (ko.F16, ko.PAD_QNAN): 0x7E007E00, (ko.F16, ko.PAD_PINF): 0x7C007C00, (ko.F16, ko.PAD_NINF): 0xFC00FC00,
           (ko.BF16, ko.PAD_QNAN): 0x7FC07FC0, (ko.BF16, ko.PAD_PINF): 0x7F807F80, (ko.BF16, ko.PAD_NINF): 0xFF80FF80,
           (ko.F8E5M2, ko.PAD_QNAN): 0x7E7E7E7E, (ko.F8E5M2, ko.PAD_PINF): 0x7C7C7C7C,
           (ko.F8E5M2, ko.PAD_NINF): 0xFCFCFCFC}
    for (dt, pad), word in ref.items():
        assert ko.lib().ko_padding_word(dt, pad) == word
    for dt in (ko.F32, ko.F16, ko.BF16, ko.F8E4M3, ko.F8E5M2, ko.I32):
        assert ko.lib().ko_padding_word(dt, ko.PAD_ZERO) == 0
    # OCP e4m3fn has no infinities: documented deviation from ConvertUtils.cpp:309-318
    assert ko.lib().ko_padding_word(ko.F8E4M3, ko.PAD_QNAN) == 0x7F7F7F7F
    assert ko.lib().ko_padding_word(ko.F8E4M3, ko.PAD_PINF) == 0x7E7E7E7E


def test_fptofp_verifier_rules(ko):
    x = np.zeros(4, dtype=np.uint16)
    with pytest.raises(ValueError):
        ko.fptofp(x, ko.BF16, ko.F8E4M3, ko.RZ)      # Kapy.cpp:280-282
    with pytest.raises(ValueError):
        ko.fptofp(x.astype(np.uint8), ko.F8E4M3, ko.F8E5M2, ko.RN)  # Kapy.cpp:283-284
    with pytest.raises(ValueError):
        ko.fptofp(np.zeros(4, np.float32), ko.F32, ko.F16, 7)       # Kapy.cpp:273-274


def test_f32_to_f8_via_f16_route(ko):
    # ElementwiseOpToLLVM.cpp:577-594: pre-sm_90 / RZ casts go f32 -RZ-> f16 -> f8.  A value just above an
    # e4m3 midpoint by less than an f16 ulp shows the double rounding.
    x = np.float32([1.0625 + 2.0 ** -12])  # midpoint of 1.0 and 1.125 plus a bit f16 cannot hold
    assert ko.fptofp(x, ko.F32, ko.F8E4M3, ko.RN, via_f16=0)[0] == 0x39  # 1.125 (true RN)
    assert ko.fptofp(x, ko.F32, ko.F8E4M3, ko.RN, via_f16=1)[0] == 0x38  # 1.0 (tie after RZ to f16 -> even)


def test_generators_are_deterministic_and_sane(ko):
    a = ko.fill_uniform(1 << 16, ko.F32, 0, 0)
    b = ko.fill_uniform(1 << 16, ko.F32, 0, 0)
    c = ko.fill_uniform(1 << 16, ko.F32, 0, 1)
    assert np.array_equal(a, b) and not np.array_equal(a, c)
    assert a.min() >= -1.0 and a.max() < 1.0 and abs(a.mean()) < 0.02
    n = ko.fill_normal(1 << 18, ko.F32, 3, 0, 0.0, 0.02)
    assert abs(n.mean()) < 2e-4 and abs(n.std() - 0.02) < 2e-4
    bits = ko.fill_bits16(1 << 16, 9)
    assert len(np.unique(bits)) > 30000
    # splitmix64 known answer (first output of the published generator seeded with 0)
    assert ko.lib().ko_splitmix64(0) == 0xE220A8397B1DCDAF
