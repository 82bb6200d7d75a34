"""CPU-only checks of the product library: it loads, exports every symbol the header declares,
its host-side layout engine agrees with the oracle, and its verifiers reject what the
reference's verifiers reject.  No compute call is made here."""
import ctypes as C
import os
import re

import numpy as np
import pytest

import kapy_hip as kh

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_library_exports_every_declared_symbol():
    import kapy_probe as kp
    for header, module in (("kapy_hip.h", kh), ("kapy_probe.h", kp)):
        text = open(os.path.join(ROOT, "include", header)).read()
        declared = set(re.findall(r"\b(kapy_[a-z0-9_]+)\s*\(", text))
        assert declared == set(module.EXPORTS), header
        L = module.lib()
        for name in declared:
            assert hasattr(L, name), name
    assert kh.lib().kapy_version() >= 100
    # the measurement kernels are not part of the product library
    assert not any(hasattr(kh.lib(), name) for name in kp.EXPORTS)


def test_struct_layout_matches_header_and_oracle(ko):
    assert C.sizeof(kh.Global) == C.sizeof(ko.Global) == 40
    assert C.sizeof(kh.Fragments) == C.sizeof(ko.Fragments) == 24
    assert C.sizeof(kh.EwInst) == C.sizeof(ko.EwInst) == 32
    assert C.sizeof(kh.MatmulCfg) == 56 and C.sizeof(kh.Grid2) == 40 and C.sizeof(kh.CopyCfg) == 24 and C.sizeof(kh.Shared) == 48


def test_descriptors_match_oracle(ko):
    buf = np.zeros(4096, dtype=np.uint16)
    a = kh.mk_global(buf.ctypes.data, 16, 32, 32, 1, kh.F16, dynamic_offset=64)
    b = ko.mk_global(buf, 16, 32, 32, 1, ko.F16, dynamic_offset=64)
    s1, s2 = kh.sv_global(kh.sv_global(a, 2, 10, 4, 20), 1, 3, 2, 6), ko.sv_global(ko.sv_global(b, 2, 10, 4, 20), 1, 3, 2, 6)
    for f in ("ptr", "start0", "start1", "end0", "end1", "stride0", "stride1", "dtype"):
        assert getattr(s1, f) == getattr(s2, f), f
    with pytest.raises(kh.KapyError) as e:
        kh.mk_global(buf.ctypes.data, 4, 4, 4, 1, 99)
    assert e.value.status == kh.ERR_INVALID
    with pytest.raises(kh.KapyError):
        kh.mk_global(buf.ctypes.data, 4, 4, 4, 1, kh.F16, alignment=12)


LAYOUTS = [([8, 8], [1, 2], 0, 1), ([8, 8], [1, 8], 0, 1), ([32, 2], [1, 8], 1, 0), ([2, 32], [4, 1], 0, 1),
           ([64, 1], [1, 1], 1, 0), ([4, 16], [2, 2], 0, 1), ([16, 4], [8, 1], 1, 0)]


@pytest.mark.parametrize("shape", [(8, 8), (32, 16), (64, 64), (16, 128), (1, 64)])
def test_fragments_maps_agree_with_oracle(ko, shape):
    L, O = kh.lib(), ko.lib()
    for la, ll, mi, ma in LAYOUTS:
        f, g = kh.Fragments.make(la, ll, mi, ma), ko.Fragments.make(la, ll, mi, ma)
        w1, s1, w2, s2 = kh.A2(0, 0), kh.A2(0, 0), kh.A2(0, 0), kh.A2(0, 0)
        assert L.kapy_fragments_loops(C.byref(f), kh.A2(*shape), w1, s1) == 0
        O.ko_fragments_loops(C.byref(g), kh.A2(*shape), w2, s2)
        assert list(w1) == list(w2) and list(s1) == list(s2)
        n = s1[0] * s1[1]
        for lane in range(64):
            for iv in range(n):
                for opt in (1, 2):
                    o1, o2 = kh.A2(0, 0), kh.A2(0, 0)
                    L.kapy_fragments_map(C.byref(f), kh.A2(*shape), opt, kh.A2(lane, iv), o1)
                    O.ko_fragments_map12(C.byref(g), kh.A2(*shape), opt, lane, iv, o2)
                    assert list(o1) == list(o2)
        for i0 in range(0, shape[0], max(1, shape[0] // 8)):
            for i1 in range(shape[1]):
                o1 = kh.A2(0, 0)
                lane, iv = C.c_int64(), C.c_int64()
                L.kapy_fragments_map(C.byref(f), kh.A2(*shape), 3, kh.A2(i0, i1), o1)
                O.ko_fragments_map3(C.byref(g), kh.A2(*shape), i0, i1, C.byref(lane), C.byref(iv))
                assert (o1[0], o1[1]) == (lane.value, iv.value)
        t1, t2 = kh.Fragments(), ko.Fragments()
        L.kapy_fragments_transpose(C.byref(f), C.byref(t1))
        O.ko_fragments_transpose(C.byref(g), C.byref(t2))
        assert bytes(t1) == bytes(t2)
        L.kapy_fragments_exchange_axes(C.byref(f), C.byref(t1))
        O.ko_fragments_exchange_axes(C.byref(g), C.byref(t2))
        assert bytes(t1) == bytes(t2)


def test_layout_string_agrees_with_oracle(ko):
    for la, ll, mi, ma in LAYOUTS:
        for shape in ((8, 8), (16, 64), (64, 4), (128, 32)):
            f, g = kh.Fragments.make(la, ll, mi, ma), ko.Fragments.make(la, ll, mi, ma)
            n = ko.lib().ko_layout_string(C.byref(g), kh.A2(*shape), None, 0)
            buf = C.create_string_buffer(n + 1)
            ko.lib().ko_layout_string(C.byref(g), kh.A2(*shape), buf, n + 1)
            assert kh.layout_string(f, shape) == buf.value.decode()


def test_default_layout_simd_change_agree_with_oracle(ko):
    L, O = kh.lib(), ko.lib()
    for loops, shape, rm in (((1, 8), (64, 64), 1), ((1, 1), (1, 256), 1), ((8, 1), (64, 16), 0), ((1, 4), (8, 8), 1)):
        f, g = kh.Fragments(), ko.Fragments()
        assert L.kapy_fragments_default(kh.A2(*loops), kh.A2(*shape), rm, C.byref(f)) == 0
        O.ko_fragments_default(kh.A2(*loops), kh.A2(*shape), rm, 64, C.byref(g))
        assert bytes(f) == bytes(g)
    for args in ((128, 16, 256), (4, 16, 4096), (128, 16, 64), (128, 8, 1 << 20), (2, 16, 4096), (16, 32, 64)):
        assert L.kapy_access_simd_size(*args) == O.ko_access_simd_size(*args, 64)
    shape = (16, 32)
    s, d = kh.Fragments.make([8, 8], [1, 2], 0, 1), kh.Fragments.make([16, 4], [1, 8], 0, 1)
    so, do = ko.Fragments.make([8, 8], [1, 2], 0, 1), ko.Fragments.make([16, 4], [1, 8], 0, 1)
    for lane in range(64):
        for iv in range(8):
            a, b, c, e = C.c_int64(), C.c_int64(), C.c_int64(), C.c_int64()
            L.kapy_change_source(C.byref(s), C.byref(d), kh.A2(*shape), lane, iv, C.byref(a), C.byref(b))
            O.ko_change_source(C.byref(so), C.byref(do), kh.A2(*shape), lane, iv, C.byref(c), C.byref(e))
            assert (a.value, b.value) == (c.value, e.value)
    assert L.kapy_change_num_shuffles(C.byref(s), C.byref(d), kh.A2(*shape)) == \
        O.ko_change_num_shuffles(C.byref(so), C.byref(do), kh.A2(*shape), 64)
    assert L.kapy_fragments_default(kh.A2(1, 1), kh.A2(24, 8), 1, C.byref(kh.Fragments())) == kh.ERR_VERIFY  # OpTraits.cpp:43-58


def test_shared_memory_descriptors_follow_the_lowering(ko):
    """kapy.mk_shared / sv_shared as plain data (MkSharedOpToLLVM.cpp:49-70, SvSharedOpToLLVM.cpp:20-42): start 0 / end = shape,
    strides by orientation, sub-view bounds counted from the SOURCE view's start, addresses through the swizzle function."""
    L, O = kh.lib(), ko.lib()
    t = kh.Shared()
    assert L.kapy_mk_shared(C.byref(t), 16384, 64, 32, kh.F16, 1, 4, 4) == 0
    assert (t.offset, t.start0, t.start1, t.end0, t.end1, t.dtype) == (16384, 0, 0, 64, 32, kh.F16)
    assert (t.layout.stride0, t.layout.stride1, t.layout.bank_param, t.layout.line_param) == (32, 1, 4, 4)
    c = kh.Shared()
    assert L.kapy_mk_shared(C.byref(c), 0, 64, 32, kh.F16, 0, 0, 0) == 0
    assert (c.layout.stride0, c.layout.stride1, c.layout.bank_param, c.layout.line_param) == (1, 64, 4, 1)
    v, w = kh.Shared(), kh.Shared()
    assert L.kapy_sv_shared(C.byref(v), C.byref(t), 16, 48, 8, 24) == 0
    assert (v.start0, v.end0, v.start1, v.end1, v.offset) == (16, 48, 8, 24, 16384)
    assert L.kapy_sv_shared(C.byref(w), C.byref(v), 4, 8, 2, 6) == 0       # new end = old START + end, not old end
    assert (w.start0, w.end0, w.start1, w.end1) == (20, 24, 10, 14)
    for (i, j) in ((0, 0), (3, 5), (31, 15), (17, 0)):
        want = 16384 + O.ko_swizzle_offset(16 + i, 8 + j, 32, 1, 16, 4, 4, 64) * 2
        assert L.kapy_shared_address(C.byref(v), i, j) == want
    assert L.kapy_shared_address(C.byref(v), 32, 0) == kh.ERR_VERIFY and L.kapy_shared_address(C.byref(v), 0, 16) == kh.ERR_VERIFY
    assert L.kapy_shared_address(C.byref(v), -17, 0) == kh.ERR_VERIFY      # unsigned compare: a negative index is out of bounds
    # every element of an unswizzled and of a swizzled buffer has an address of its own inside the buffer
    for bp, lp in ((0, 0), (4, 8), (2, 16)):
        assert L.kapy_mk_shared(C.byref(t), 1024, 32, 64, kh.BF16, 1, bp, lp) == 0
        seen = {L.kapy_shared_address(C.byref(t), i, j) for i in range(32) for j in range(64)}
        assert len(seen) == 32 * 64 and min(seen) == 1024 and max(seen) == 1024 + 32 * 64 * 2 - 2
    assert L.kapy_mk_shared(C.byref(t), 0, 48, 32, kh.F16, 1, 0, 0) == kh.ERR_VERIFY            # OpTraits.cpp:43-58: powers of two
    assert L.kapy_mk_shared(C.byref(t), 100, 32, 32, kh.F16, 1, 0, 0) == kh.ERR_INVALID         # 128-byte aligned (AllocAnalysis)
    assert L.kapy_mk_shared(C.byref(t), 128 * 1024, 256, 128, kh.F16, 1, 0, 0) == kh.ERR_VERIFY  # beyond 160 KiB
    assert L.kapy_mk_shared(C.byref(t), 0, 32, 32, kh.F16, 1, 3, 1) == kh.ERR_INVALID
    assert L.kapy_sv_shared(C.byref(v), C.byref(t), 8, 4, 0, 4) == kh.ERR_INVALID


def test_copy_hints_are_validated():
    g = _g()
    for kw in (dict(cache=9), dict(evict=5), dict(evict=-1), dict(padding=4)):
        st, msg = _status(kh.copy, g, g, stream=NULL, **kw)
        assert st == kh.ERR_INVALID, kw
    st, msg = _status(kh.copy, g, g, evict=kh.NO_ALLOCATE, volatile=True, stream=NULL)
    assert st == kh.ERR_HIP       # accepted by the verifier; only the missing device stops it here


def test_swizzle_agrees_with_oracle_and_matmul_layout_is_searched(ko):
    L, O = kh.lib(), ko.lib()
    for bits, s0 in ((16, 64), (16, 32), (8, 128), (32, 32)):
        for bp, lp in ((4, 8), (4, 4), (2, 16), (1, 64), (4, 1)):
            sw = kh.Swizzling(s0, 1, bp, lp)
            for i0 in range(0, 64, 3):
                for i1 in range(0, s0, 5):
                    assert L.kapy_swizzle_offset(C.byref(sw), bits, i0, i1) == O.ko_swizzle_offset(i0, i1, s0, 1, bits, bp, lp, 64)
    # the reference's search, re-parameterised for 64 banks and lanes, agrees with the checker's restatement of it
    for tile_k in (32, 64):
        for way, want_mnk in ((kh.MFMA_16X16X32_16B, [16, 16, 32]), (kh.MFMA_32X32X16_16B, [32, 32, 16])):
            f, mnk = kh.Fragments(), (C.c_int32 * 3)()
            assert L.kapy_matmul_layouts(way, 0, C.byref(f), mnk) == 0 and list(mnk) == want_mnk
            shape = kh.A2(mnk[0], mnk[2])
            pairs = (C.c_int32 * 64)()
            n = L.kapy_swizzle_search(C.byref(f), shape, tile_k, 1, 16, 1024, pairs, 32)
            op = (C.c_int64 * 64)()
            g = ko.Fragments.make(*f.astuple())
            assert n == O.ko_swizzle_search(C.byref(g), shape, tile_k, 1, 16, 1024, 64, 64, op, 32) and n > 0
            assert [pairs[i] for i in range(2 * n)] == [op[i] for i in range(2 * n)]
            assert pairs[0] == 4 and (pairs[0], 1) not in {(pairs[2 * i], pairs[2 * i + 1]) for i in range(n)}  # unswizzled conflicts
            # ... and so does the search over the gfx950 read phases (triples with the key's rotation)
            triples, ot = (C.c_int32 * 300)(), (C.c_int64 * 300)()
            n = L.kapy_swizzle_search_gfx950(C.byref(f), shape, tile_k, 1, 16, 1024, triples, 100)
            assert n == O.ko_swizzle_search_gfx950(C.byref(g), shape, tile_k, 1, 16, 1024, ot, 100) and n > 0
            assert [triples[i] for i in range(3 * n)] == [ot[i] for i in range(3 * n)]
            if (way == kh.MFMA_16X16X32_16B) == (tile_k == 64):
                # the LDS layout the matmul uses is that search's first hit for the instruction its kernels of that depth are
                # built on (32-deep tiles: 32x32x16; 64-deep tiles: 16x16x32)
                sw = kh.Swizzling()
                assert L.kapy_matmul_lds_layout(kh.BF16, tile_k, C.byref(sw)) == 0
                assert (sw.stride0, sw.stride1, sw.bank_param, sw.line_param, sw.rotate) == (tile_k, 1) + tuple(triples[:3])
    # rotated keys through the offset function
    for lp, rot in ((8, 1), (16, 3)):
        sw = kh.Swizzling(128, 1, 4, lp, rot)
        assert all(L.kapy_swizzle_offset(C.byref(sw), 8, i0, i1) == O.ko_swizzle_offset_rotated(i0, i1, 128, 1, 8, 4, lp, rot)
                   for i0 in range(0, 40, 3) for i1 in range(0, 128, 5))


def test_mfma_layouts_are_consistent_fragments(ko):
    """lhs/rhs/acc layouts of each MFMA shape tile their operand exactly and agree on (m,n,k)."""
    L = kh.lib()
    for way, kpack in ((kh.MFMA_32X32X16_16B, 8), (kh.MFMA_16X16X32_16B, 8), (kh.MFMA_16X16X128_F8, 32), (kh.MFMA_32X32X64_F8, 32)):
        fr = [kh.Fragments() for _ in range(3)]
        mnk = (C.c_int32 * 3)()
        for which in range(3):
            assert L.kapy_matmul_layouts(way, which, C.byref(fr[which]), mnk) == 0
        m, n, k = list(mnk)
        shapes = [(m, k), (k, n), (m, n)]
        for which, shape in enumerate(shapes):
            seen = set()
            s = kh.A2(0, 0)
            L.kapy_fragments_loops(C.byref(fr[which]), kh.A2(*shape), kh.A2(0, 0), s)
            per_lane = s[0] * s[1]
            assert per_lane * 64 == shape[0] * shape[1]
            for lane in range(64):
                for iv in range(per_lane):
                    o = kh.A2(0, 0)
                    L.kapy_fragments_map(C.byref(fr[which]), kh.A2(*shape), 2, kh.A2(lane, iv), o)
                    seen.add((o[0], o[1]))
            assert len(seen) == shape[0] * shape[1]
        # a lane's lhs values are kpack consecutive k of one row, its rhs values kpack consecutive k of one column
        o0, o1 = kh.A2(0, 0), kh.A2(0, 0)
        L.kapy_fragments_map(C.byref(fr[0]), kh.A2(m, k), 2, kh.A2(5, 0), o0)
        L.kapy_fragments_map(C.byref(fr[0]), kh.A2(m, k), 2, kh.A2(5, kpack - 1), o1)
        assert o0[0] == o1[0] == 5 and o1[1] - o0[1] == kpack - 1
        # which = 3: the accumulator with the operands exchanged holds the transposed block, i.e. is the transposed layout
        ex, tr = kh.Fragments(), kh.Fragments()
        assert L.kapy_matmul_layouts(way, 3, C.byref(ex), None) == 0
        assert L.kapy_fragments_transpose(C.byref(fr[2]), C.byref(tr)) == 0 and bytes(ex) == bytes(tr)
        o2, o3 = kh.A2(0, 0), kh.A2(0, 0)
        for lane in (0, 17, 63):
            for iv in range(m * n // 64):
                L.kapy_fragments_map(C.byref(fr[2]), kh.A2(m, n), 2, kh.A2(lane, iv), o2)
                L.kapy_fragments_map(C.byref(ex), kh.A2(m, n), 2, kh.A2(lane, iv), o3)
                assert (o2[0], o2[1]) == (o3[1], o3[0])
    assert L.kapy_matmul_layouts(kh.MMA_M16N8K8_TF32, 0, C.byref(kh.Fragments()), None) == kh.ERR_UNSUPPORTED
    assert L.kapy_matmul_layouts(kh.MFMA_16X16X32_16B, 4, C.byref(kh.Fragments()), None) == kh.ERR_INVALID


def _g(dtype=kh.F16, m=16, n=16, s0=None, s1=1, buf=None):
    buf = buf if buf is not None else _g.buf
    return kh.mk_global(buf.ctypes.data, m, n, s0 if s0 is not None else n, s1, dtype)


_g.buf = np.zeros(1 << 16, dtype=np.uint8)


def _status(fn, *a, **k):
    try:
        fn(*a, **k)
    except kh.KapyError as e:
        return e.status, e.message
    return 0, ""


NULL = C.c_void_p(0)


def test_matmul_verifier_messages_follow_the_reference():
    # lib/Dialect/Kapy/IR/Kapy.cpp:451-487
    st, msg = _status(kh.matmul, _g(m=16, n=8), _g(m=16, n=16), _g(), stream=NULL)
    assert st == kh.ERR_VERIFY and "columns of lhs" in msg
    st, msg = _status(kh.matmul, _g(), _g(), _g(m=8, n=16), stream=NULL)
    assert st == kh.ERR_VERIFY and "rows of acc" in msg
    st, msg = _status(kh.matmul, _g(), _g(kh.F8E4M3), _g(), stream=NULL)
    assert st == kh.ERR_VERIFY and "same element bit width" in msg
    st, msg = _status(kh.matmul, _g(), _g(kh.BF16), _g(), stream=NULL)
    assert st == kh.ERR_VERIFY and "same element type unless" in msg
    st, msg = _status(kh.matmul, _g(kh.BF16), _g(kh.BF16), _g(kh.BF16), acc=_g(kh.F16), stream=NULL)
    assert st == kh.ERR_VERIFY and "f32 element type when operands are bf16" in msg
    st, msg = _status(kh.matmul, _g(), _g(), _g(), acc=_g(kh.BF16), stream=NULL)
    assert st == kh.ERR_VERIFY and "f16 or f32" in msg
    st, msg = _status(kh.matmul, _g(), _g(), _g(), impl_way=kh.MMA_M16N8K16_F8, stream=NULL)
    assert st == kh.ERR_VERIFY and "f8E4M3 or f8E5M2" in msg
    st, msg = _status(kh.matmul, _g(kh.F32), _g(kh.F32), _g(kh.F32), impl_way=kh.MMA_M16N8K8_TF32, stream=NULL)
    assert st == kh.ERR_UNSUPPORTED and "tf32" in msg
    st, msg = _status(kh.matmul, _g(), _g(), _g(), impl_way=77, stream=NULL)
    assert st == kh.ERR_INVALID


def test_elementwise_and_copy_verifiers():
    x = _g()
    ld_st = [dict(op=kh.EW_LD_GLOBAL, dst=0, a=0), dict(op=kh.EW_ST_GLOBAL, a=0)]
    st, msg = _status(kh.elementwise, kh.program(ld_st), [_g(m=16, n=8)], x, stream=NULL)
    assert st == kh.ERR_VERIFY and "broadcast" in msg                                   # Kapy.cpp:686-698
    st, msg = _status(kh.elementwise, kh.program(ld_st), [_g(kh.BF16)], x, stream=NULL)
    assert st == kh.ERR_VERIFY and "same element type" in msg                           # st_global operands
    down = [dict(op=kh.EW_LD_GLOBAL, dst=0, a=0), dict(op=kh.EW_FPTOFP, dst=1, a=0, dtype=kh.F16, rmode=5),
            dict(op=kh.EW_ST_GLOBAL, a=1)]
    st, msg = _status(kh.elementwise, kh.program(down), [_g(kh.F32)], x, stream=NULL)
    assert st == kh.ERR_VERIFY and "rounding mode is required" in msg                   # Kapy.cpp:273-274
    bf8 = [dict(op=kh.EW_LD_GLOBAL, dst=0, a=0), dict(op=kh.EW_FPTOFP, dst=1, a=0, dtype=kh.F8E4M3, rmode=kh.RZ),
           dict(op=kh.EW_ST_GLOBAL, a=1)]
    st, msg = _status(kh.elementwise, kh.program(bf8), [_g(kh.BF16)], _g(kh.F8E4M3), stream=NULL)
    assert st == kh.ERR_VERIFY and "bf16 to f8" in msg                                  # Kapy.cpp:280-282
    f8f8 = [dict(op=kh.EW_LD_GLOBAL, dst=0, a=0), dict(op=kh.EW_FPTOFP, dst=1, a=0, dtype=kh.F8E5M2, rmode=kh.RN),
            dict(op=kh.EW_ST_GLOBAL, a=1)]
    st, msg = _status(kh.elementwise, kh.program(f8f8), [_g(kh.F8E4M3)], _g(kh.F8E5M2), stream=NULL)
    assert st == kh.ERR_VERIFY and "f8 to f8" in msg                                    # Kapy.cpp:283-284
    mixed = [dict(op=kh.EW_LD_GLOBAL, dst=0, a=0), dict(op=kh.EW_SPLAT, dst=1, dtype=kh.F32, imm=1.0),
             dict(op=kh.EW_ADDF, dst=2, a=0, b=1), dict(op=kh.EW_ST_GLOBAL, a=2)]
    st, msg = _status(kh.elementwise, kh.program(mixed), [x], x, stream=NULL)
    assert st == kh.ERR_VERIFY
    st, msg = _status(kh.elementwise, kh.program(ld_st[:1]), [x], x, stream=NULL)
    assert st == kh.ERR_INVALID and "st_global" in msg
    st, msg = _status(kh.copy, _g(kh.F16), _g(kh.F32), stream=NULL)
    assert st == kh.ERR_VERIFY and "element width" in msg
    st, msg = _status(kh.copy, _g(kh.I16), _g(kh.I16), padding=kh.PAD_QNAN, stream=NULL)
    assert st == kh.ERR_VERIFY
    st, msg = _status(kh.reduce, _g(kh.F32), _g(kh.F32, m=16, n=2), 1, stream=NULL)
    assert st == kh.ERR_VERIFY and "number of elements in result" in msg


def test_device_entry_points_fail_loudly_without_a_gpu():
    """No CPU fallback: with valid arguments and no usable device the call must fail, not compute."""
    import torch
    if torch.cuda.is_available():
        pytest.skip("a GPU is present")
    x = _g()
    st, msg = _status(kh.copy, x, x, stream=NULL)
    assert st == kh.ERR_HIP and "no CPU fallback" in msg
    st, msg = _status(kh.matmul, _g(), _g(), _g(), stream=NULL)
    assert st == kh.ERR_HIP
    st, msg = _status(kh.elementwise, kh.gelu_program(), [x, _g(m=1, n=16)], x, stream=NULL)
    assert st == kh.ERR_HIP
