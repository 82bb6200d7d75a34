#!/usr/bin/env python3
"""Writes reference_held_vectors.json: the known answers that the reference's own files hold for the hot path,
transcribed as data (never as source text), plus the two OCP fp8 decode tables from their published closed form.

Provenance of each block:
  attrs_td            include/kapy/Dialect/Kgpu/IR/Attrs.td:28-78 - the documented #kgpu.fragments<[8,4],[1,2],(0,1)>
                      lane grid and its per-lane loop expansion on an 8x8 tensor, and the 8-lane broadcast example
                      (layout [[0,0,1,1],[2,2,3,3],[4,4,5,5],[6,6,7,7]] on a 2x8 tensor, element -> owning lanes).
  padding_words       lib/Conversion/KgpuToLLVM/ConvertUtils.cpp:267-334 - generateInitConstant: the 32-bit word that
                      pre-fills an out-of-bounds ld_global lane, per element type and PaddingOption.  The e4m3 entries
                      of the reference assume an IEEE-style e4m3 with infinities; the build uses OCP E4M3FN, so they are
                      listed under "padding_words_e4m3_reference" for the record and not asserted.
  ocp_e4m3fn / e5m2   OCP 8-bit Floating Point Specification (OFP8) rev 1.0, section 5: value tables by closed form.
Run: python tests/golden/make_golden.py   (deterministic; rewrites the JSON next to this file)."""
import json
import math
import os


def e4m3fn(b):
    s, e, m = b >> 7, (b >> 3) & 15, b & 7
    if e == 15 and m == 7:
        return None  # NaN (no infinities in E4M3FN)
    v = math.ldexp(m / 8.0, -6) if e == 0 else math.ldexp(1 + m / 8.0, e - 7)
    return -v if s else v


def e5m2(b):
    s, e, m = b >> 7, (b >> 2) & 31, b & 3
    if e == 31:
        return None if m else ("-inf" if s else "inf")
    v = math.ldexp(m / 4.0, -14) if e == 0 else math.ldexp(1 + m / 4.0, e - 15)
    return -v if s else v


doc = {
    "attrs_td": {
        "layout": {"lane_array": [8, 4], "lane_loops": [1, 2], "minor_axis": 0, "major_axis": 1},
        "lane_grid": [[4 * r + c for c in range(4)] for r in range(8)],
        "tensor_shape": [8, 8],
        "owner_lane_of_element": [[4 * r + c // 2 for c in range(8)] for r in range(8)],
        "broadcast_example": {
            "layout": {"lane_array": [4, 2], "lane_loops": [1, 2], "minor_axis": 0, "major_axis": 1},
            "tensor_shape": [2, 8],
            "owners": [[[0, 4], [0, 4], [1, 5], [1, 5], [0, 4], [0, 4], [1, 5], [1, 5]],
                       [[2, 6], [2, 6], [3, 7], [3, 7], [2, 6], [2, 6], [3, 7], [3, 7]]],
        },
    },
    "padding_words": {
        "f32": {"ZERO": 0, "QNAN": 0x7FC00000, "PINF": 0x7F800000, "NINF": 0xFF800000},
        "f16": {"ZERO": 0, "QNAN": 0x7E007E00, "PINF": 0x7C007C00, "NINF": 0xFC00FC00},
        "bf16": {"ZERO": 0, "QNAN": 0x7FC07FC0, "PINF": 0x7F807F80, "NINF": 0xFF80FF80},
        "f8e5m2": {"ZERO": 0, "QNAN": 0x7E7E7E7E, "PINF": 0x7C7C7C7C, "NINF": 0xFCFCFCFC},
    },
    "padding_words_e4m3_reference": {"QNAN": 0x7C7C7C7C, "PINF": 0x78787878, "NINF": 0xF8F8F8F8},
    "ocp_e4m3fn_decode": [e4m3fn(b) for b in range(256)],
    "ocp_e5m2_decode": [e5m2(b) for b in range(256)],
}
with open(os.path.join(os.path.dirname(os.path.abspath(__file__)), "reference_held_vectors.json"), "w") as f:
    json.dump(doc, f, indent=1)
    f.write("\n")
