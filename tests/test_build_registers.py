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
            if "nn_kernel<" in name or "nn256_kernel<" in name:
                # no register of any build may be spilled: a transposing read's result is pending until the kernel's own wait, and a
                # spill (or a fragment buffer kept in scratch memory) would store it before it has arrived.  The builds with the
                # element-store epilogue call that store out of line, which takes a private segment and nothing else.
                packed = re.search(r"nn_kernel<[^,]+, \d+, \d+, true,", name) is not None or "nn256_kernel<" in name
                if int(field("vgpr_spill_count")) or int(field("sgpr_spill_count")) > 64 or int(field("private_segment_fixed_size")) > (0 if packed else 256):
                    bad.append("%s: %s VGPRs spilled, %s SGPRs spilled, %s bytes of private segment" %
                               (name[:140], field("vgpr_spill_count"), field("sgpr_spill_count"), field("private_segment_fixed_size")))
                continue
            if "staged_kernel<" in name:    # element-store epilogue
                continue
            if int(field("vgpr_spill_count")) or int(field("sgpr_spill_count")) > 64 or int(field("private_segment_fixed_size")):
                bad.append("%s: %s VGPRs spilled, %s SGPRs spilled, %s bytes of private segment" %
                           (name[:140], field("vgpr_spill_count"), field("sgpr_spill_count"), field("private_segment_fixed_size")))
    assert seen > 100, "only %d kernels found" % seen
    assert not bad, "\n".join(bad)


def _registers(text):
    """Vector registers named in an operand string: v7, v[4:7]."""
    regs = set()
    for lo, hi in re.findall(r"\bv\[(\d+):(\d+)\]", text):
        regs.update(range(int(lo), int(hi) + 1))
    regs.update(int(r) for r in re.findall(r"\bv(\d+)\b", text))
    return regs


@pytest.mark.skipif(not os.path.exists(LIB), reason="library not built")
@pytest.mark.skipif(not all(os.path.exists(os.path.join(LLVM, t)) for t in ("llvm-objcopy", "llvm-objdump")), reason="binary tools not found")
def test_no_instruction_touches_a_pending_transposing_read(tmp_path):
    """The kernels issue ds_read_b64_tr_b16 as opaque assembly and wait for the results themselves (s_waitcnt lgkmcnt(0)); the compiler
    does not know that the destination registers are pending in between.  In the library's own machine code, between such a read
    and the next wait for LDS results no instruction may name a destination register of the read - not a copy, not a store to
    scratch memory, not an overwrite - on the straight path and along every forward branch (the pending set travels with a branch
    to its label)."""
    seen_reads, bad = 0, []
    for path in _code_objects(tmp_path):
        text = subprocess.run([os.path.join(LLVM, "llvm-objdump"), "-d", "--symbolize-operands", "--no-show-raw-insn", path], check=True, capture_output=True, text=True).stdout
        if "ds_read_b64_tr_b16" not in text:
            continue
        kernel, pending, at_label = "?", set(), {}
        for line in text.split("\n"):
            m = re.match(r"^[0-9a-f]+ <(.+)>:$", line)
            if m:
                if re.fullmatch(r"L\d+", m.group(1)):
                    pending |= at_label.pop(m.group(1), set())
                else:
                    kernel, pending, at_label = m.group(1), set(), {}
                continue
            inst = line.split("//")[0].strip()
            if not inst:
                continue
            op, _, operands = inst.partition(" ")
            if op == "ds_read_b64_tr_b16":
                seen_reads += 1
                dst, _, rest = operands.partition(",")
                if _registers(rest) & pending:
                    bad.append("%s: %s addresses through a pending register" % (kernel[:100], inst))
                pending |= _registers(dst)
                continue
            if op == "s_waitcnt" and ("lgkmcnt(0)" in operands or re.fullmatch(r"(0x)?0+", operands.strip())):
                pending = set()
                continue
            if op.startswith("s_cbranch") or op == "s_branch":
                target = operands.strip()
                if pending and re.fullmatch(r"L\d+", target):
                    at_label[target] = at_label.get(target, set()) | pending
                if op == "s_branch":
                    pending = set()
                continue
            if op in ("s_endpgm", "s_setpc_b64", "s_swappc_b64") and pending:
                bad.append("%s: %s with reads pending" % (kernel[:100], op))
                pending = set()
                continue
            if pending and _registers(operands) & pending:
                bad.append("%s: '%s' names v%s while a transposing read into it is pending" % (kernel[:100], inst, sorted(_registers(operands) & pending)))
    assert seen_reads > 1000, "only %d transposing reads found: is the disassembly what this test expects?" % seen_reads
    assert not bad, "\n".join(bad[:20]) + "\n(%d in all)" % len(bad)
