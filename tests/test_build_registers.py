"""The built library's kernels keep their values in registers.

A kernel that starts to spill still passes every parity test - it only gets slower, and its scratch traffic shows up as
HBM bytes nobody asked for - so the code objects inside libkapy_hip.so are read back here: every kernel's metadata note
must say 0 spilled registers and 0 bytes of private segment.  Exempt, by name:
  * the row machines (row_kernel): their 1024-lane builds are held to 128 registers and index a private array by design;
  * the tiled matmul's builds off the fast path - the element-store epilogue (it calls an out-of-line store routine, which
    needs a stack) and the build for a partial last K-tile (its lane masks cost the registers the main loop has to spare);
  * the tick-reading build of the matrix-instruction probe (one register saved around its timer reads).
"""
import os
import re
import shutil
import struct
import subprocess

import pytest

HERE = os.path.dirname(os.path.abspath(__file__))
LIB = os.path.join(os.path.dirname(HERE), "kapy-lang_amd", "lib", "libkapy_hip.so")
PROBE_LIB = os.path.join(os.path.dirname(HERE), "kapy-lang_amd", "lib", "libkapy_probe.so")
LLVM = "/opt/rocm/llvm/bin"


def _code_objects(tmp_path, library=LIB, tag="p"):
    fat = str(tmp_path / (tag + "fat.bin"))
    subprocess.run([os.path.join(LLVM, "llvm-objcopy"), "--dump-section", ".hip_fatbin=" + fat, library, str(tmp_path / (tag + "copy.so"))], check=True)
    blob = open(fat, "rb").read()
    magic, pos, out = b"__CLANG_OFFLOAD_BUNDLE__", 0, []
    while True:
        at = blob.find(magic, pos)
        if at < 0:
            return out
        (count,) = struct.unpack_from("<Q", blob, at + len(magic))
        p = at + len(magic) + 8
        for _ in range(count):
            offset, size, id_len = struct.unpack_from("<QQQ", blob, p)
            p += 24
            target = blob[p:p + id_len].decode()
            p += id_len
            if "gfx950" in target and size:
                path = str(tmp_path / ("%sco_%d.elf" % (tag, len(out))))
                open(path, "wb").write(blob[at + offset:at + offset + size])
                out.append(path)
        pos = at + len(magic)


@pytest.mark.skipif(not os.path.exists(LIB), reason="library not built")
@pytest.mark.skipif(not all(os.path.exists(os.path.join(LLVM, t)) for t in ("llvm-objcopy", "llvm-readelf")) or not shutil.which("c++filt"), reason="binary tools not found")
def test_no_kernel_spills(tmp_path):
    objects = _code_objects(tmp_path)
    assert objects, "no gfx950 code object found in the library"
    if os.path.exists(PROBE_LIB):
        objects += _code_objects(tmp_path, PROBE_LIB, "q")
    seen, bad = 0, []
    for path in objects:
        notes = subprocess.run([os.path.join(LLVM, "llvm-readelf"), "--notes", path], check=True, capture_output=True, text=True).stdout
        for kernel in notes.split("- .agpr_count:")[1:]:
            field = lambda key: re.search(r"\." + key + r":\s*(\S+)", kernel).group(1)
            name = subprocess.run(["c++filt", field("name")], capture_output=True, text=True).stdout.strip()
            seen += 1
            if "row_kernel<" in name or re.search(r"mfma_loop_kernel<.*, true>", name):
                continue
            m = re.search(r"tn_kernel<.*, (true|false), (true|false), (true|false)>", name)
            if m and (m.group(1) == "false" or m.group(2) == "true"):  # element-store epilogue / partial last K-tile
                continue
            if re.search(r"nn_kernel<[^,]+, \d+, \d+, false,", name) or "staged_kernel<" in name:    # element-store epilogue (staged_kernel holds both)
                continue
            if int(field("vgpr_spill_count")) or int(field("sgpr_spill_count")) > 64 or int(field("private_segment_fixed_size")):
                bad.append("%s: %s VGPRs spilled, %s SGPRs spilled, %s bytes of private segment" %
                           (name[:140], field("vgpr_spill_count"), field("sgpr_spill_count"), field("private_segment_fixed_size")))
    assert seen > 100, "only %d kernels found" % seen
    assert not bad, "\n".join(bad)
