"""Pins the oracle's layout math: fragments maps against the diagrams the reference holds
(include/kapy/Dialect/Kgpu/IR/Attrs.td:28-78) and against structural invariants; the swizzle against
its closed form and a brute-force bank replay."""
import ctypes as C
import itertools

import numpy as np
import pytest


def A2(a, b):
    return (C.c_int64 * 2)(a, b)


def map12(ko, f, shape, option, lane, iv):
    out = A2(0, 0)
    ko.lib().ko_fragments_map12(C.byref(f), A2(*shape), option, lane, iv, out)
    return out[0], out[1]


def map3(ko, f, shape, i0, i1):
    lane, iv = C.c_int64(), C.c_int64()
    ko.lib().ko_fragments_map3(C.byref(f), A2(*shape), i0, i1, C.byref(lane), C.byref(iv))
    return lane.value, iv.value


def loops(ko, f, shape):
    w, s = A2(0, 0), A2(0, 0)
    ko.lib().ko_fragments_loops(C.byref(f), A2(*shape), w, s)
    return (w[0], w[1]), (s[0], s[1])


def test_attrs_td_diagram_8x4_lanes(ko):
    # #kgpu.fragments<[8,4],[1,2],(0,1)> on 8x8: row r holds lanes 4r..4r+3, each lane two adjacent columns
    f = ko.Fragments.make([8, 4], [1, 2], 0, 1)
    want = np.array([[4 * r + c // 2 for c in range(8)] for r in range(8)])
    got = np.array([[map3(ko, f, (8, 8), r, c)[0] for c in range(8)] for r in range(8)])
    assert np.array_equal(want, got)
    for lane in range(32):
        for iv in range(2):
            assert map12(ko, f, (8, 8), 2, lane, iv) == (lane // 4, 2 * (lane % 4) + iv)


def test_attrs_td_element_to_lane_example(ko):
    # 8-lane layout [[0,0,1,1],[2,2,3,3],[4,4,5,5],[6,6,7,7]] applied to a 2x8 tensor (Attrs.td:55-78):
    # A..H / I..P -> lanes {0,4},{0,4},{1,5},{1,5},{0,4},... ; {2,6},{2,6},{3,7},...
    f = ko.Fragments.make([4, 2], [1, 2], 0, 1)
    shape = (2, 8)
    _, space = loops(ko, f, shape)
    owners = {}
    for lane in range(8):
        for iv in range(space[0] * space[1]):
            owners.setdefault(map12(ko, f, shape, 1, lane, iv), set()).add(lane)
    want_row0 = [{0, 4}, {0, 4}, {1, 5}, {1, 5}, {0, 4}, {0, 4}, {1, 5}, {1, 5}]
    want_row1 = [{2, 6}, {2, 6}, {3, 7}, {3, 7}, {2, 6}, {2, 6}, {3, 7}, {3, 7}]
    assert [owners[(0, j)] for j in range(8)] == want_row0
    assert [owners[(1, j)] for j in range(8)] == want_row1


LAYOUTS = []
for a0 in (1, 2, 4, 8, 16, 32, 64):
    for l0, l1 in ((1, 1), (1, 2), (2, 1), (1, 8), (8, 1), (2, 4), (4, 4)):
        for major in (0, 1):
            LAYOUTS.append((a0, 64 // a0, l0, l1, major))


@pytest.mark.parametrize("shape", [(1, 64), (8, 8), (16, 64), (64, 16), (64, 64), (128, 32)])
def test_fragments_invariants(ko, shape):
    for a0, a1, l0, l1, major in LAYOUTS:
        f = ko.Fragments.make([a0, a1], [l0, l1], 1 - major, major)
        (w0, w1), (s0, s1) = loops(ko, f, shape)
        assert (w0, w1) == (max(shape[0] // (a0 * l0), 1), max(shape[1] // (a1 * l1), 1))
        n = s0 * s1
        exact = a0 * l0 <= shape[0] and a1 * l1 <= shape[1]
        seen = set()
        for lane in range(64):
            for iv in range(n):
                idx = map12(ko, f, shape, 1, lane, iv)
                assert 0 <= idx[0] < shape[0] and 0 <= idx[1] < shape[1]
                seen.add(idx)
                if exact:  # map3 inverts map2 when the layout tiles the shape without replication
                    assert map3(ko, f, shape, *map12(ko, f, shape, 2, lane, iv)) == (lane, iv)
        assert len(seen) == shape[0] * shape[1]  # every element owned by at least one (lane, iv)
        if exact:
            assert 64 * n == shape[0] * shape[1]
        # transpose(): involution, and commutes with swapping the indices
        t, tt = ko.Fragments(), ko.Fragments()
        ko.lib().ko_fragments_transpose(C.byref(f), C.byref(t))
        ko.lib().ko_fragments_transpose(C.byref(t), C.byref(tt))
        assert bytes(tt) == bytes(f)
        for lane, iv in ((0, 0), (5, n - 1), (63, n // 2)):
            i0, i1 = map12(ko, f, shape, 1, lane, iv)
            assert map12(ko, t, (shape[1], shape[0]), 1, lane, iv) == (i1, i0)


def test_default_layout_and_simd_rule(ko):
    # getFragmentsLayout (LayoutUtils.cpp:92-104) evaluated by hand for warp 32 and wave 64
    f = ko.Fragments()
    ko.lib().ko_fragments_default(A2(1, 8), A2(64, 64), 1, 32, C.byref(f))
    assert (list(f.lane_array), list(f.lane_loops), f.minor_axis, f.major_axis) == ([4, 8], [1, 8], 0, 1)
    ko.lib().ko_fragments_default(A2(1, 8), A2(64, 64), 1, 64, C.byref(f))
    assert list(f.lane_array) == [8, 8]
    ko.lib().ko_fragments_default(A2(1, 1), A2(1, 256), 1, 32, C.byref(f))
    assert list(f.lane_array) == [1, 32]
    ko.lib().ko_fragments_default(A2(8, 1), A2(64, 16), 0, 64, C.byref(f))
    assert (list(f.lane_array), f.major_axis) == ([8, 8], 0)
    # CoalesceAccess.cpp:18-27 by hand: f16, 128-B aligned, 1x256 tile on a 32-lane warp -> 8 elements
    assert ko.lib().ko_access_simd_size(128, 16, 256, 32) == 8
    assert ko.lib().ko_access_simd_size(4, 16, 4096, 32) == 2     # 4-byte alignment caps at one word
    assert ko.lib().ko_access_simd_size(128, 16, 64, 32) == 2     # tiny tile: numel/32 = 2
    assert ko.lib().ko_access_simd_size(128, 8, 1 << 20, 64) == 16
    assert ko.lib().ko_access_simd_size(2, 16, 4096, 32) == 2     # floor at one 32-bit word


def test_change_is_a_data_preserving_relayout(ko):
    shape = (16, 32)
    src = ko.Fragments.make([8, 8], [1, 2], 0, 1)
    dst = ko.Fragments.make([16, 4], [1, 8], 0, 1)
    (_, ss), (_, sd) = loops(ko, src, shape), loops(ko, dst, shape)
    ns, nd = ss[0] * ss[1], sd[0] * sd[1]
    tile = np.arange(shape[0] * shape[1], dtype=np.uint32).reshape(shape) * 7 + 3
    lanes_src = np.zeros((64, ns), dtype=np.uint32)
    for lane in range(64):
        for iv in range(ns):
            lanes_src[lane, iv] = tile[map12(ko, src, shape, 2, lane, iv)]
    lanes_dst = np.zeros((64, nd), dtype=np.uint32)
    ko.lib().ko_change_tile(lanes_src.ctypes.data_as(C.c_void_p), C.byref(src), C.byref(dst), A2(*shape), 4, 64,
                            lanes_dst.ctypes.data_as(C.c_void_p))
    for lane in range(64):
        for iv in range(nd):
            assert lanes_dst[lane, iv] == tile[map12(ko, dst, shape, 2, lane, iv)]
    # identical layouts need no shuffles; an in-register transpose relabel needs none either
    assert ko.lib().ko_change_num_shuffles(C.byref(src), C.byref(src), A2(*shape), 64) == 0
    assert ko.lib().ko_change_num_shuffles(C.byref(src), C.byref(dst), A2(*shape), 64) > 0


def swz(ko, i0, i1, s0, s1, bits, bp, lp, banks):
    return ko.lib().ko_swizzle_offset(i0, i1, s0, s1, bits, bp, lp, banks)


@pytest.mark.parametrize("banks", [32, 64])
def test_swizzle_is_a_bijection_and_keeps_lines(ko, banks):
    rows, cols, bits = 32, 64, 16
    line_elems = banks * 32 // bits
    for bp in (1, 2, 4):
        lp = 1
        while lp <= banks // bp:
            offs = np.array([[swz(ko, i, j, cols, 1, bits, bp, lp, banks) for j in range(cols)] for i in range(rows)])
            assert sorted(offs.ravel().tolist()) == list(range(rows * cols))
            lin = np.arange(rows * cols).reshape(rows, cols)
            assert np.array_equal(offs // line_elems, lin // line_elems)  # never leaves its line
            if lp == 1:
                assert np.array_equal(offs, lin)
            lp *= 2


def test_swizzle_4_8_is_the_textbook_128B_xor(ko):
    # 32 banks, f16, 64-element (128-B) rows: 16-byte chunk index ^= row % 8  (CpAsyncOpToLLVM.cpp:124-139)
    for i in range(16):
        for j in range(64):
            chunk, within = j // 8, j % 8
            want = i * 64 + ((chunk ^ (i % 8)) * 8 + within)
            assert swz(ko, i, j, 64, 1, 16, 4, 8, 32) == want


def _replay_conflicts(ko, f, shape, s0, s1, bits, bp, lp, banks, lanes_per_phase):
    """Brute-force replay: worst number of distinct lines hitting one bank within a phase."""
    worst = 0
    bytes_ = bits // 8
    vec = f.lane_loops[1] if s1 == 1 else f.lane_loops[0]
    for p0 in range(0, 64, lanes_per_phase):
        bank_lines = {}
        for lane in range(p0, p0 + lanes_per_phase):
            i0, i1 = map12(ko, f, shape, 1, lane, 0)
            for e in range(vec):
                a0, a1 = (i0, i1 + e) if s1 == 1 else (i0 + e, i1)
                off = swz(ko, a0, a1, s0, s1, bits, bp, lp, banks) * bytes_
                bank_lines.setdefault((off // 4) % banks, set()).add(off // (banks * 4))
        worst = max(worst, max(len(v) for v in bank_lines.values()))
    return worst


def test_swizzle_search_matches_bruteforce_replay_64_banks(ko):
    # MFMA 32x32x16 bf16 operand read: lane l reads 8 consecutive K elements (16 B) of row l%32, K-group l/32
    f = ko.Fragments.make([32, 2], [1, 8], 1, 0)
    shape, bits = (32, 64), 16
    pairs = (C.c_int64 * 64)()
    n = ko.lib().ko_swizzle_search(C.byref(f), A2(*shape), 64, 1, bits, 16, 64, 64, pairs, 32)
    found = {(pairs[2 * k], pairs[2 * k + 1]) for k in range(n)}
    assert (4, 8) in found and (4, 16) in found and (4, 1) not in found and (4, 4) not in found
    for bp, lp in itertools.product((4,), (1, 2, 4, 8, 16)):
        ok = _replay_conflicts(ko, f, shape, 64, 1, bits, bp, lp, 64, 64 // bp) == 1
        assert ok == ((bp, lp) in found)


def _layout_string(ko, f, shape):
    n = ko.lib().ko_layout_string(C.byref(f), A2(*shape), None, 0)
    buf = C.create_string_buffer(n + 1)
    ko.lib().ko_layout_string(C.byref(f), A2(*shape), buf, n + 1)
    return buf.value.decode()


def test_layout_string_of_the_attrs_td_example(ko):
    """What bin/kapy-layout.cpp prints (getLayoutString, Kgpu.cpp:293-353) for the documented example
    #kgpu.fragments<[8,4],[1,2],(0,1)> on an 8x8 tensor: row r = lanes 4r..4r+3, two loop ivs each, ids
    right-aligned to the widest lane id (31 -> width 2) and iv (1 -> width 1)."""
    f = ko.Fragments.make([8, 4], [1, 2], 0, 1)
    text = _layout_string(ko, f, (8, 8))
    rows = text.split("\n")
    assert len(rows) == 8
    assert rows[0] == "[[ T0:0,  T0:1,  T1:0,  T1:1,  T2:0,  T2:1,  T3:0,  T3:1],"
    assert rows[3] == " [T12:0, T12:1, T13:0, T13:1, T14:0, T14:1, T15:0, T15:1],"
    assert rows[7] == " [T28:0, T28:1, T29:0, T29:1, T30:0, T30:1, T31:0, T31:1]]"


def test_layout_string_prints_one_block_per_replication_round(ko):
    """A layout larger than the tensor owns every element several times (Attrs.td:55-78): the 8-lane example
    [[0,0,1,1],[2,2,3,3],...] x 4 rows on a 2x4 tensor replicates twice along rows."""
    f = ko.Fragments.make([4, 2], [1, 2], 0, 1)
    text = _layout_string(ko, f, (2, 4))
    blocks = text.split("\n\n")
    assert len(blocks) == 2
    assert blocks[0] == "[[T0:0, T0:1, T1:0, T1:1],\n [T2:0, T2:1, T3:0, T3:1]]"
    assert blocks[1] == "[[T4:0, T4:1, T5:0, T5:1],\n [T6:0, T6:1, T7:0, T7:1]]"


# ---- the gfx950 read phases ------------------------------------------------------------------------------------------
GFX950_PHASES_128 = [[0, 1, 2, 3, 12, 13, 14, 15, 20, 21, 22, 23, 24, 25, 26, 27], [4, 5, 6, 7, 8, 9, 10, 11, 16, 17, 18, 19, 28, 29, 30, 31]]
GFX950_PHASES_128 += [[l + 32 for l in ph] for ph in GFX950_PHASES_128]


def _rot(key, width, r):
    return ((key << r) | (key >> (width - r))) & ((1 << width) - 1) if width and r % width else key


def _replay_gfx950(rows_of_lane, chunks_of_lane, row_bytes, lp, rot):
    """A 16-byte read replayed by hand on byte addresses: lane -> (row, list of 16-byte chunks, one instruction each); a row is
    row_bytes long, chunk c of the row at byte row * row_bytes + 16 * c, its position within the 256-byte line XOR-ed with the
    rotated key.  True when no phase of no instruction asks one bank group (16 bytes = 4 banks) for two lines."""
    width = lp.bit_length() - 1
    for inst in range(len(chunks_of_lane(0))):
        for phase in GFX950_PHASES_128:
            seen = {}
            for lane in phase:
                byte = rows_of_lane(lane) * row_bytes + 16 * chunks_of_lane(lane)[inst]
                line, pos = byte // 256, (byte % 256) // 16
                pos ^= _rot(line % lp, width, rot)
                if seen.setdefault(pos, line) != line:
                    return False
    return True


def test_gfx950_model_says_what_the_counters_said(ko):
    """The two measurements the model was built on, as fixtures: the 16x16x128 operand reads (row lane % 16, chunks 2 * (lane / 16)
    and + 1 of a 128-byte row) with the plain key (4, 8) conflict on the device (SQ_LDS_BANK_CONFLICT on half of the LDS's
    active cycles) and are free of conflicts with the key rotated by one bit (counter zero).  The reference's first-lanes
    model passes both."""
    f = ko.Fragments.make([16, 4], [1, 32], 1, 0)
    shape = A2(16, 128)
    conflict_free = lambda bp, lp, rot: ko.lib().ko_no_bank_conflict_gfx950(C.byref(f), shape, 128, 1, 8, bp, lp, rot, 1024)
    assert conflict_free(4, 8, 0) == 0
    assert conflict_free(4, 8, 1) == 1
    assert ko.lib().ko_no_bank_conflict(C.byref(f), shape, 128, 1, 8, 4, 8, 1024, 64, 64) == 1
    triples = (C.c_int64 * 96)()
    n = ko.lib().ko_swizzle_search_gfx950(C.byref(f), shape, 128, 1, 8, 1024, triples, 32)
    assert n > 0 and tuple(triples[:3]) == (4, 8, 1)


@pytest.mark.parametrize("name,lane_array,kpack_bytes,rows,row_bytes", [
    ("16x16x32 16-bit, K-tile 32", [16, 4], 16, 16, 64), ("16x16x32 16-bit, K-tile 64", [16, 4], 16, 16, 128),
    ("32x32x16 16-bit, K-tile 32", [32, 2], 16, 32, 64), ("32x32x16 16-bit, K-tile 64", [32, 2], 16, 32, 128),
    ("16x16x128 fp8", [16, 4], 32, 16, 128), ("32x32x64 fp8", [32, 2], 32, 32, 128)])
def test_gfx950_search_matches_a_replay_on_byte_addresses(ko, name, lane_array, kpack_bytes, rows, row_bytes):
    """Every 16-byte candidate of the search for the operand reads of the four matrix instructions against the replay above,
    which knows nothing of fragments: lane l reads row l % rows, bytes kpack_bytes * (l / rows) .. of it."""
    f = ko.Fragments.make(lane_array, [1, kpack_bytes], 1, 0)
    k_bytes = kpack_bytes * lane_array[1]
    triples = (C.c_int64 * 300)()
    n = ko.lib().ko_swizzle_search_gfx950(C.byref(f), A2(rows, k_bytes), row_bytes, 1, 8, 1024, triples, 100)
    found = {tuple(triples[3 * i:3 * i + 3]) for i in range(n)}
    rows_of = lambda lane: lane % rows
    chunks_of = lambda lane: [(kpack_bytes * (lane // rows)) // 16 + i for i in range(kpack_bytes // 16)]
    for lp in (1, 2, 4, 8, 16):
        for rot in range(max(1, lp.bit_length() - 1)):
            assert _replay_gfx950(rows_of, chunks_of, row_bytes, lp, rot) == ((4, lp, rot) in found), (name, lp, rot)
    assert any(t[0] == 4 for t in found)


def test_rotated_offsets_are_a_bijection_that_keeps_lines(ko):
    rows, cols = 32, 128
    for lp, rot in ((8, 1), (8, 2), (16, 3), (4, 1)):
        offs = np.array([[ko.lib().ko_swizzle_offset_rotated(i, j, cols, 1, 8, 4, lp, rot) for j in range(cols)] for i in range(rows)])
        assert sorted(offs.ravel().tolist()) == list(range(rows * cols))
        lin = np.arange(rows * cols).reshape(rows, cols)
        assert np.array_equal(offs // 256, lin // 256) and np.array_equal(offs % 16, lin % 16)
    # rotate 0 is the reference's map
    assert all(ko.lib().ko_swizzle_offset_rotated(i, j, cols, 1, 8, 4, 8, 0) == ko.lib().ko_swizzle_offset(i, j, cols, 1, 8, 4, 8, 64)
               for i in range(rows) for j in range(0, cols, 7))
