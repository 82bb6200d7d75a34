"""The oracle and the library's host entry points against tests/golden/reference_held_vectors.json: the known
answers the reference's own files hold for this path (Attrs.td layout examples, generateInitConstant padding
words) and the OCP fp8 value tables.  The fixture is data written by tests/golden/make_golden.py."""
import ctypes as C
import json
import math
import os

import kapy_hip as kh

GOLD = json.load(open(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "reference_held_vectors.json")))


def _frag(mod, d):
    return mod.Fragments.make(d["lane_array"], d["lane_loops"], d["minor_axis"], d["major_axis"])


def test_attrs_td_owner_lanes_oracle_and_library(ko):
    g = GOLD["attrs_td"]
    shape = g["tensor_shape"]
    fo, fk = _frag(ko, g["layout"]), _frag(kh, g["layout"])
    for i in range(shape[0]):
        for j in range(shape[1]):
            lane, iv = C.c_int64(), C.c_int64()
            ko.lib().ko_fragments_map3(C.byref(fo), kh.A2(*shape), i, j, C.byref(lane), C.byref(iv))
            assert lane.value == g["owner_lane_of_element"][i][j]
            out = kh.A2(0, 0)
            assert kh.lib().kapy_fragments_map(C.byref(fk), kh.A2(*shape), 3, kh.A2(i, j), out) == 0
            assert out[0] == g["owner_lane_of_element"][i][j] and out[1] == j % 2
    # the lane grid itself: lane (r, c) of the 8x4 array is 4r + c, i.e. element (r, 2c) belongs to it
    for r in range(8):
        for c in range(4):
            assert g["owner_lane_of_element"][r][2 * c] == g["lane_grid"][r][c]


def test_attrs_td_broadcast_example_oracle_and_library(ko):
    g = GOLD["attrs_td"]["broadcast_example"]
    shape = g["tensor_shape"]
    fo, fk = _frag(ko, g["layout"]), _frag(kh, g["layout"])
    space = kh.A2(0, 0)
    warp = kh.A2(0, 0)
    ko.lib().ko_fragments_loops(C.byref(fo), kh.A2(*shape), warp, space)
    for mod_name in ("oracle", "library"):
        owners = {}
        for lane in range(8):
            for iv in range(space[0] * space[1]):
                idx = kh.A2(0, 0)
                if mod_name == "oracle":
                    ko.lib().ko_fragments_map12(C.byref(fo), kh.A2(*shape), 1, lane, iv, idx)
                else:
                    assert kh.lib().kapy_fragments_map(C.byref(fk), kh.A2(*shape), 1, kh.A2(lane, iv), idx) == 0
                owners.setdefault((idx[0], idx[1]), set()).add(lane)
        for i in range(shape[0]):
            for j in range(shape[1]):
                assert owners[(i, j)] == set(g["owners"][i][j]), (mod_name, i, j)


def test_padding_words(ko):
    dt = {"f32": ko.F32, "f16": ko.F16, "bf16": ko.BF16, "f8e5m2": ko.F8E5M2}
    pad = {"ZERO": ko.PAD_ZERO, "QNAN": ko.PAD_QNAN, "PINF": ko.PAD_PINF, "NINF": ko.PAD_NINF}
    for tname, words in GOLD["padding_words"].items():
        for pname, word in words.items():
            assert ko.lib().ko_padding_word(dt[tname], pad[pname]) == word, (tname, pname)


def test_ocp_fp8_tables(ko):
    for b, want in enumerate(GOLD["ocp_e4m3fn_decode"]):
        got = ko.lib().ko_e4m3_to_f64(b)
        assert math.isnan(got) if want is None else got == want, b
    for b, want in enumerate(GOLD["ocp_e5m2_decode"]):
        got = ko.lib().ko_e5m2_to_f64(b)
        if want is None:
            assert math.isnan(got)
        elif isinstance(want, str):
            assert got == float(want)
        else:
            assert got == want, b
