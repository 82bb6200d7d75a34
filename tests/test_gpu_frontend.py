"""GPU parity of the textual front-end: programs with the structure of the reference's three Kapy fixtures
(test/Conversion/KapyToKgpu/{elementwise_add,reduce_sum,matmul}.mlir) run end to end through kapy_run_mlir
and are compared with the oracle's elementwise, reduce and matmul on the same inputs."""
import ctypes as C

import numpy as np
import pytest

import kapy_hip as kh
import kapy_programs as kp
from gpu_util import dev_zeros, sync, to_dev, to_host, ulp_diff_f16

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("op,ew,rows_per_warp,cols,warps,programs", [
    ("arith.addf", "EW_ADDF", 4, 128, 4, 3),      # the fixture's x + y
    ("arith.mulf", "EW_MULF", 2, 256, 2, 2),
    ("arith.subf", "EW_SUBF", 8, 64, 1, 5),
])
def test_binary_program_is_bit_exact(ko, op, ew, rows_per_warp, cols, warps, programs):
    rows = rows_per_warp * warps * programs
    x = ko.fill_normal(rows * cols, ko.F16, 11)
    y = ko.fill_normal(rows * cols, ko.F16, 12)
    want = np.zeros(rows * cols, np.uint16)
    prog = ko.program([dict(op=ko.EW_LD_GLOBAL, dst=0, a=0), dict(op=ko.EW_LD_GLOBAL, dst=1, a=1),
                       dict(op=getattr(ko, ew), dst=2, a=0, b=1), dict(op=ko.EW_ST_GLOBAL, a=2)])
    g = lambda a: ko.mk_global(a, rows, cols, cols, 1, ko.F16)
    assert ko.elementwise(prog, [g(x), g(y)], g(want)) == 0
    dx, dy, dout = to_dev(x), to_dev(y), dev_zeros(rows * cols, 2, fill=0x7e00)
    kh.run_mlir(kp.binary_program(op, rows_per_warp, cols, warps), [dx, dy, dout, rows], [programs])
    sync()
    assert np.array_equal(to_host(dout, np.uint16), want)


@pytest.mark.parametrize("comb,kind,rows_per_warp,cols,warps,programs", [
    ("arith.addf", 0, 2, 256, 2, 4),               # the fixture's row sum
    ("arith.maximumf", 1, 4, 512, 1, 3),
])
def test_reduce_program_matches_oracle(ko, comb, kind, rows_per_warp, cols, warps, programs):
    rows = rows_per_warp * warps * programs
    x = ko.fill_normal(rows * cols, ko.F16, 21)
    want = np.zeros(rows, np.uint16)
    assert ko.lib().ko_reduce(C.byref(ko.mk_global(x, rows, cols, cols, 1, ko.F16)), C.byref(ko.mk_global(want, rows, 1, 1, rows, ko.F16)),
                              1, kind) == 0
    dx, dout = to_dev(x), dev_zeros(rows, 2, fill=0x7e00)
    kh.run_mlir(kp.reduce_program(comb, rows_per_warp, cols, warps), [dx, dout, rows], [programs])
    sync()
    got = to_host(dout, np.uint16)
    # a sum is accumulated in fp32 in an order of the kernel's own: at most 1 ulp of f16 from the oracle; a max is exact
    assert ulp_diff_f16(got, want).max() <= (1 if kind == 0 else 0)


def _chunked_reference(a, b, bk, acc_dtype):
    """The program's arithmetic: per K step an fp32-accumulated product added to the carried accumulator,
    which is rounded to acc_dtype after every step."""
    acc = np.zeros((a.shape[0], b.shape[1]), acc_dtype)
    for k0 in range(0, a.shape[1], bk):
        acc = (acc.astype(np.float64) + a[:, k0:k0 + bk].astype(np.float64) @ b[k0:k0 + bk].astype(np.float64)).astype(acc_dtype)
    return acc


@pytest.mark.parametrize("bm,bn,bk,way,acc,M,N,K", [
    (64, 64, 16, "mma_m16n8k8_f16", "f16", 256, 128, 128),     # the fixture's tiling: 128x128 per program, f16 accumulator
    (64, 64, 32, "mma_m16n8k16_f16", "f32", 128, 256, 96),
    (32, 64, 32, "mma_m16n8k16_f16", "f32", 64, 128, 32),      # one K step: the loop body never runs
])
def test_matmul_program_matches_oracle(ko, bm, bn, bk, way, acc, M, N, K):
    a = ko.fill_normal(M * K, ko.F16, 31, std=0.5)
    b = ko.fill_normal(K * N, ko.F16, 32, std=0.5)
    da, db = to_dev(a), to_dev(b)
    acc_np, acc_bytes = (np.float16, 2) if acc == "f16" else (np.float32, 4)
    dc = dev_zeros(M * N, acc_bytes, fill=-1)
    grid = (M // (2 * bm)) * (N // (2 * bn))
    kh.run_mlir(kp.matmul_program(bm, bn, bk, way, acc), [da, db, dc, M, N, K], [grid])
    sync()
    got = to_host(dc, acc_np, (M, N)).astype(np.float64)
    af, bf = a.view(np.float16).reshape(M, K), b.view(np.float16).reshape(K, N)
    # against the oracle's whole-K matmul (fp64 reference rounded once)
    want = np.zeros(M * N, np.uint16 if acc == "f16" else np.float32)
    ga, gb = ko.mk_global(a, M, K, K, 1, ko.F16), ko.mk_global(b, K, N, N, 1, ko.F16)
    assert ko.lib().ko_matmul(C.byref(ga), C.byref(gb), None, C.byref(ko.mk_global(want, M, N, N, 1, ko.F16 if acc == "f16" else ko.F32)),
                              ko.RN) == 0
    ref = want.view(acc_np).reshape(M, N).astype(np.float64)
    rel = np.linalg.norm(got - ref) / np.linalg.norm(ref)
    assert rel <= (2e-3 if acc == "f16" else 1e-5), rel    # an f16 accumulator rounds after every K step
    # against the program's own arithmetic (accumulator rounded per step): only fp32 summation order differs
    step = _chunked_reference(af, bf, bk, acc_np).astype(np.float64)
    rel = np.linalg.norm(got - step) / np.linalg.norm(step)
    assert rel <= (3e-4 if acc == "f16" else 1e-6), rel


@pytest.mark.parametrize("cols", [256, 100])
@pytest.mark.parametrize("fuse", ["1", "0"])
def test_softmax_program_in_kapy_ops_matches_the_oracle_program(ko, monkeypatch, cols, fuse):
    """Fused (the default), the ten ops between the load and the store are the oracle's softmax program itself: both reduces
    are instructions of one row program.  A width that is no multiple of 8 is outside the row programs, so there the reduces run
    as kapy_reduce and the arithmetic between them as three programs; KAPY_MLIR_FUSE=0 runs every op by itself."""
    monkeypatch.setenv("KAPY_MLIR_FUSE", fuse)
    rows_per_warp, warps, programs = 2, 2, 3
    rows = rows_per_warp * warps * programs
    x = ko.fill_normal(rows * cols, ko.F16, 51, std=3.0)
    want = np.zeros(rows * cols, np.uint16)
    g = lambda a: ko.mk_global(a, rows, cols, cols, 1, ko.F16)
    assert ko.elementwise(ko.program(kh.softmax_insts(kh.F16)), [g(x)], g(want)) == 0
    dx, dout = to_dev(x), dev_zeros(rows * cols, 2, fill=0x7e00)
    kh.run_mlir(kp.softmax_program(rows_per_warp, cols, warps), [dx, dout, rows], [programs])
    sync()
    assert ulp_diff_f16(to_host(dout, np.uint16), want).max() <= 2     # in f32, one rounding to f16 at the end


@pytest.mark.parametrize("fuse", ["1", "0"])
def test_causal_masked_softmax_program_with_integer_tensor_ops(ko, monkeypatch, fuse):
    """kapy.arange, an integer splat, arith.addi, arith.cmpi and arith.select on tensors in front of the softmax chain: fused, one
    row program with integer registers (compiled on its first use); KAPY_MLIR_FUSE=0 runs every op by itself, the i32 and i1
    tensors going through memory."""
    monkeypatch.setenv("KAPY_MLIR_FUSE", fuse)
    rows_per_warp, cols, warps, programs = 2, 64, 2, 4
    rows = rows_per_warp * warps * programs
    x = ko.fill_normal(rows * cols, ko.F16, 55, std=3.0)
    dx, dout = to_dev(x), dev_zeros(rows * cols, 2, fill=0x7e00)
    kh.run_mlir(kp.causal_softmax_program(rows_per_warp, cols, warps), [dx, dout, rows], [programs])
    sync()
    got = ko.decode(to_host(dout, np.uint16, (rows, cols)), ko.F16)
    xf = ko.decode(x.reshape(rows, cols), ko.F16)
    ref = np.where(np.tril(np.ones((rows, cols), bool)), xf, -np.inf)
    ref = np.exp(ref - ref.max(axis=1, keepdims=True))
    ref /= ref.sum(axis=1, keepdims=True)
    assert not np.triu(got, 1).any() and np.abs(got - ref).max() <= 2.0 ** -10


def _gated_insts():
    L, CAST, ST = kh.EW_LD_GLOBAL, kh.EW_FPTOFP, kh.EW_ST_GLOBAL
    return [dict(op=L, dst=0, a=0), dict(op=CAST, dst=0, a=0, dtype=kh.F32), dict(op=L, dst=1, a=1), dict(op=CAST, dst=1, a=1, dtype=kh.F32),
            dict(op=kh.EW_NEGF, dst=2, a=0), dict(op=kh.EW_EXP, dst=2, a=2), dict(op=kh.EW_SPLAT, dst=3, dtype=kh.F32, imm=1.0),
            dict(op=kh.EW_ADDF, dst=2, a=2, b=3), dict(op=kh.EW_DIVF, dst=2, a=0, b=2), dict(op=kh.EW_MULF, dst=2, a=2, b=1),
            dict(op=L, dst=4, a=2), dict(op=kh.EW_MULF, dst=2, a=2, b=4), dict(op=CAST, dst=5, a=2, dtype=kh.F16, rmode=kh.RN),
            dict(op=ST, a=5)]


def test_chain_of_elementwise_ops_runs_as_one_program(ko, monkeypatch):
    """silu(x) * y * gate[row]: eleven elementwise ops between the loads and the store.  The front-end defers them and the store
    runs them as one program; with KAPY_MLIR_FUSE=0 every op is a call of its own.  Both equal the oracle's run of the same
    program to the bar of the elementwise tests, and each other bit for bit (the same instructions on the same values)."""
    rows_per_warp, cols, warps, programs = 4, 256, 2, 3
    rows = rows_per_warp * warps * programs
    x, y = ko.fill_normal(rows * cols, ko.F16, 61, std=2.0), ko.fill_normal(rows * cols, ko.F16, 62)
    gate = np.linspace(0.25, 2.0, rows).astype(np.float32)
    want = np.zeros(rows * cols, np.uint16)
    g = lambda a: ko.mk_global(a, rows, cols, cols, 1, ko.F16)
    assert ko.elementwise(ko.program(_gated_insts()), [g(x), g(y), ko.mk_global(gate, rows, 1, 1, 1, ko.F32)], g(want)) == 0
    dx, dy, dg = to_dev(x), to_dev(y), to_dev(gate)
    text = kp.gated_program(rows_per_warp, cols, warps)
    results = []
    for fuse in ("1", "0"):
        monkeypatch.setenv("KAPY_MLIR_FUSE", fuse)
        dout = dev_zeros(rows * cols, 2, fill=0x7e00)
        kh.run_mlir(text, [dx, dy, dg, dout, rows], [programs])
        sync()
        results.append(to_host(dout, np.uint16))
        assert ulp_diff_f16(results[-1], want).max() <= 2
    assert np.array_equal(results[0], results[1])


@pytest.mark.parametrize("fuse", ["1", "0"])
def test_a_store_into_memory_that_deferred_loads_read(ko, monkeypatch, fuse):
    """Loads join the deferred chain, so the program that needs a loaded value reads the caller's memory itself, later than the
    load stands in the text.  A store into that memory in between must not change what the load saw."""
    monkeypatch.setenv("KAPY_MLIR_FUSE", fuse)
    rows_per_warp, cols, warps, programs = 4, 128, 2, 2
    rows = rows_per_warp * warps * programs
    x, y = ko.fill_normal(rows * cols, ko.F16, 71), ko.fill_normal(rows * cols, ko.F16, 72)
    dx, dy, dout = to_dev(x), to_dev(y), dev_zeros(rows * cols, 2, fill=0x7e00)
    kh.run_mlir(kp.aliasing_program(rows_per_warp, cols, warps), [dx, dy, dout, rows], [programs])
    sync()
    xf, yf = x.view(np.float16), y.view(np.float16)
    assert np.array_equal(to_host(dout, np.float16), (xf + yf) * xf)          # numpy rounds each f16 op once, as the program does
    assert np.array_equal(to_host(dx, np.float16), yf + yf)
    assert np.array_equal(to_host(dy, np.float16), yf)


def test_deferred_values_carried_by_a_loop(ko, monkeypatch):
    """An scf.for whose body is a chain ending in the carried accumulator: the yield computes it once per iteration (one
    program: load, cast, tanh, scale, add), the splat defined before the loop stays deferred across all of them.  Fused and
    op-by-op runs agree bit for bit; both follow a numpy restatement with fp32 accumulation in the program's order."""
    rows_per_warp, bc, warps, programs, blocks = 4, 64, 2, 2, 5
    rows, cols = rows_per_warp * warps * programs, bc * blocks
    x = ko.fill_normal(rows * cols, ko.F16, 81)
    dx = to_dev(x)
    results = []
    for fuse in ("1", "0"):
        monkeypatch.setenv("KAPY_MLIR_FUSE", fuse)
        dout = dev_zeros(rows * bc, 2, fill=0x7e00)
        kh.run_mlir(kp.block_sum_program(rows_per_warp, bc, warps), [dx, dout, rows, cols], [programs])
        sync()
        results.append(to_host(dout, np.float16, (rows, bc)))
    assert np.array_equal(results[0].view(np.uint16), results[1].view(np.uint16))
    acc = np.full((rows, bc), 0.25, np.float32)
    xf = x.view(np.float16).reshape(rows, cols).astype(np.float64)
    for j in range(blocks):
        acc = acc + (np.tanh(xf[:, j * bc:(j + 1) * bc]).astype(np.float32) * np.float32(0.5))
    assert np.abs(results[0].astype(np.float64) - acc).max() <= 2e-3


def test_fused_chain_is_one_kernel(ko):
    """With KAPY_EW_AUTO_SPECIALIZE=1 (read once per process, so in a process of its own) every program outside the hand-written
    kernels is compiled when first seen: the chain of eleven ops leaves exactly one compiled kernel behind, launched ONCE for all
    program instances and warps (their tiles join into one view; KAPY_MLIR_BATCH=0: once per instance and warp)."""
    import os
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    code = r'''
import sys
sys.path[:0] = [%r, %r, %r]
import numpy as np, torch, kapy_hip as kh, ko, kapy_programs as kp
from gpu_util import dev_zeros, sync, to_dev, to_host
rows_per_warp, cols, warps, programs = 4, 256, 2, 3
rows = rows_per_warp * warps * programs
x, y = ko.fill_normal(rows * cols, ko.F16, 61, std=2.0), ko.fill_normal(rows * cols, ko.F16, 62)
gate = np.linspace(0.25, 2.0, rows).astype(np.float32)
dx, dy, dg, dout = to_dev(x), to_dev(y), to_dev(gate), dev_zeros(rows * cols, 2, fill=0x7e00)
kh.run_mlir(kp.gated_program(rows_per_warp, cols, warps), [dx, dy, dg, dout, rows], [programs]); sync()
assert kh.elementwise_specialize_stats() == (1, 1), kh.elementwise_specialize_stats()
import os
os.environ["KAPY_MLIR_BATCH"] = "0"
d2 = dev_zeros(rows * cols, 2, fill=0x7e00)
kh.run_mlir(kp.gated_program(rows_per_warp, cols, warps), [dx, dy, dg, d2, rows], [programs]); sync()
assert kh.elementwise_specialize_stats() == (1, 1 + programs * warps), kh.elementwise_specialize_stats()
assert np.array_equal(to_host(d2, np.uint16), to_host(dout, np.uint16))
xf, yf = x.view(np.float16).astype(np.float64).reshape(rows, cols), y.view(np.float16).astype(np.float64).reshape(rows, cols)
ref = xf / (1 + np.exp(-xf)) * yf * gate[:, None].astype(np.float64)
got = to_host(dout, np.float16, (rows, cols)).astype(np.float64)
assert np.all(np.abs(got - ref) <= 2e-3 * np.abs(ref) + 1e-6), np.abs(got - ref).max()
print("fused ok")
''' % (os.path.join(root, "kapy-lang_amd", "python"), os.path.join(root, "oracle"), os.path.join(root, "tests"))
    env = dict(os.environ, KAPY_EW_AUTO_SPECIALIZE="1")
    env.pop("KAPY_MLIR_FUSE", None)
    out = subprocess.run([sys.executable, "-c", code], env=env, capture_output=True, text=True, timeout=110)
    assert out.returncode == 0 and "fused ok" in out.stdout, out.stdout + out.stderr


def test_transpose_splat_program_is_bit_exact(ko):
    m, n, tile = 96, 64, 32
    x = ko.fill_normal(m * n, ko.F16, 52)
    dx, dout = to_dev(x), dev_zeros(m * n, 2, fill=0x7e00)
    kh.run_mlir(kp.scaled_transpose_program(tile, 0.5), [dx, dout, m, n], [m // tile, n // tile])
    sync()
    want = (x.view(np.float16).reshape(m, n).T * np.float16(0.5)).astype(np.float16)
    assert np.array_equal(to_host(dout, np.float16, (n, m)), want)


def test_buffers_that_share_planned_memory_do_not_disturb_each_other(ko):
    x = ko.fill_normal(64 * 64, ko.F16, 41)
    d = to_dev(x)
    kh.run_mlir(kp.phases_program(), [d], [1])
    sync()
    assert np.array_equal(to_host(d, np.float16), x.view(np.float16) * np.float16(2))


def test_errors_name_the_line_and_leave_the_device_usable(ko):
    rows, cols = 16, 128
    x = to_dev(ko.fill_normal(rows * cols, ko.F16, 1))
    out = dev_zeros(rows * cols, 2)
    text = kp.binary_program()
    with pytest.raises(kh.KapyError) as e:                 # grid of 2 programs needs 32 rows: the sub-view leaves its parent
        kh.run_mlir(text, [x, x, out, rows], [2])
    assert "sub-view leaves its parent" in e.value.message and "kapy.sv_global" in e.value.message
    with pytest.raises(kh.KapyError) as e:                 # rows argument larger than the allocation
        kh.run_mlir(text, [x, x, out, 4 * rows], [1])
    assert "reaches beyond" in e.value.message
    kh.run_mlir(text, [x, x, out, rows], [1])
    sync()
    assert np.array_equal(to_host(out, np.float16), to_host(x, np.float16) * 2)


@pytest.mark.parametrize("rows_per_warp,cols,warps,programs", [(16, 64, 4, 3), (8, 128, 2, 5), (4, 64, 8, 1)])
def test_warps_exchange_through_shared_memory(ko, rows_per_warp, cols, warps, programs):
    """Warp w reads what warp (w + 1) % warps stored before the barrier: right only if the warps run in step."""
    rows = rows_per_warp * warps * programs
    x = ko.fill_normal(rows * cols, ko.F16, 61).view(np.float16).reshape(programs, warps, rows_per_warp, cols)
    want = np.roll(x, -1, axis=1) * np.float16(2)
    dx, dout = to_dev(x.view(np.uint16).ravel()), dev_zeros(rows * cols, 2, fill=0x7e00)
    kh.run_mlir(kp.exchange_program(rows_per_warp, cols, warps), [dx, dout, rows], [programs])
    sync()
    assert np.array_equal(to_host(dout, np.uint16), want.view(np.uint16).ravel())


@pytest.mark.parametrize("rows_per_warp,cols,warps,steps,programs", [(8, 64, 4, 3, 2), (16, 64, 2, 5, 3)])
def test_warps_exchange_inside_a_loop(ko, rows_per_warp, cols, warps, steps, programs):
    """The exchange repeated in an scf.for that carries the tile: the loop itself has to advance all warps together."""
    rows = rows_per_warp * warps * programs
    x = ko.fill_normal(rows * cols, ko.F16, 62).view(np.float16).reshape(programs, warps, rows_per_warp, cols)
    want = x
    for _ in range(steps):
        want = np.roll(want + np.float16(1), -1, axis=1)
    dx, dout = to_dev(x.view(np.uint16).ravel()), dev_zeros(rows * cols, 2, fill=0x7e00)
    kh.run_mlir(kp.exchange_loop_program(rows_per_warp, cols, warps, steps), [dx, dout, rows], [programs])
    sync()
    assert np.array_equal(to_host(dout, np.uint16), want.view(np.uint16).ravel())


@pytest.mark.parametrize("rows,cols_per_warp", [(64, 64), (40, 24)])
@pytest.mark.parametrize("fuse", ["1", "0"])
def test_column_softmax_program_matches_the_oracle_program(ko, monkeypatch, rows, cols_per_warp, fuse):
    """Reduces along axis 0: fused (the default) the ops between the load and the store are one program on the column machine with
    both reduces as instructions; KAPY_MLIR_FUSE=0 runs every op by itself, the reduces as kapy_reduce along axis 0."""
    monkeypatch.setenv("KAPY_MLIR_FUSE", fuse)
    warps, programs = 2, 3
    cols = cols_per_warp * warps * programs
    x = ko.fill_normal(rows * cols, ko.F16, 71, std=3.0)
    want = np.zeros(rows * cols, np.uint16)
    g = lambda a: ko.mk_global(a, rows, cols, cols, 1, ko.F16)
    insts = [dict(i, b=0) if i["op"] in (kh.EW_REDUCE_SUM, kh.EW_REDUCE_MAX) else i for i in kh.softmax_insts(kh.F16)]
    assert ko.elementwise(ko.program(insts), [g(x)], g(want)) == 0
    dx, dout = to_dev(x), dev_zeros(rows * cols, 2, fill=0x7e00)
    kh.run_mlir(kp.column_softmax_program(rows, cols_per_warp, warps), [dx, dout, cols], [programs])
    sync()
    assert ulp_diff_f16(to_host(dout, np.uint16), want).max() <= 2     # in f32, one rounding to f16 at the end


def test_the_instances_of_a_grid_run_as_one_call_where_their_tiles_join(ko, monkeypatch):
    """The fixture-shaped programs over a grid: all programs and warps in step, and every kapy.st_global whose chains have one form
    and whose views tile a rectangle runs as ONE call over the union (counted by kapy_run_mlir_stats).  Results are bit for bit
    those of running one instance at a time (KAPY_MLIR_BATCH=0), which the tests above compare with the oracle."""
    def both(run, out_words, merged_stores):
        outs = []
        for batch in ("1", "0"):
            monkeypatch.setenv("KAPY_MLIR_BATCH", batch)
            dout = dev_zeros(out_words, 2, fill=0x7e00)
            before = kh.run_mlir_stats()
            run(dout)
            sync()
            assert kh.run_mlir_stats() - before == (merged_stores if batch == "1" else 0), batch
            outs.append(to_host(dout, np.uint16))
        assert np.array_equal(outs[0], outs[1])
        return outs[0]

    # x + y: 6 programs x 2 warps x [4 x 256] tiles stacked along the rows -> one elementwise call over [48 x 256]
    rows_per_warp, cols, warps, programs = 4, 256, 2, 6
    rows = rows_per_warp * warps * programs
    x, y = ko.fill_normal(rows * cols, ko.F16, 11), ko.fill_normal(rows * cols, ko.F16, 12)
    dx, dy = to_dev(x), to_dev(y)
    got = both(lambda d: kh.run_mlir(kp.binary_program("arith.addf", rows_per_warp, cols, warps), [dx, dy, d, rows], [programs]), rows * cols, 1)
    want = np.zeros(rows * cols, np.uint16)
    prog = ko.program([dict(op=ko.EW_LD_GLOBAL, dst=0, a=0), dict(op=ko.EW_LD_GLOBAL, dst=1, a=1), dict(op=ko.EW_ADDF, dst=2, a=0, b=1), dict(op=ko.EW_ST_GLOBAL, a=2)])
    g = lambda a: ko.mk_global(a, rows, cols, cols, 1, ko.F16)
    assert ko.elementwise(prog, [g(x), g(y)], g(want)) == 0
    assert np.array_equal(got, want)
    # the row sum of the fixture: the reduce of all instances as one kapy_reduce, its store as one copy
    rows_per_warp, cols, warps, programs = 2, 256, 2, 8
    rows = rows_per_warp * warps * programs
    x = ko.fill_normal(rows * cols, ko.F16, 21)
    dx = to_dev(x)
    both(lambda d: kh.run_mlir(kp.reduce_program("arith.addf", rows_per_warp, cols, warps), [dx, d, rows], [programs]), rows, 1)
    # softmax (two reduces along the rows inside the chain): one row program over all rows of the grid
    rows_per_warp, cols, warps, programs = 2, 256, 2, 5
    rows = rows_per_warp * warps * programs
    x = ko.fill_normal(rows * cols, ko.F16, 31)
    dx = to_dev(x)
    both(lambda d: kh.run_mlir(kp.softmax_program(rows_per_warp, cols, warps), [dx, d, rows], [programs]), rows * cols, 1)
    # a causal mask (kapy.arange: values depend on where the tile lies): never merged
    both(lambda d: kh.run_mlir(kp.causal_softmax_program(rows_per_warp, cols, warps), [dx, d, rows], [programs]), rows * cols, 0)


def test_a_repeated_call_replays_the_device_calls_of_the_first(ko, monkeypatch):
    """A second kapy_run_mlir with the same text, grid and argument values makes the device calls the first one made, without
    parsing or interpreting again (counted by kapy_run_mlir_plan_stats), on whatever the buffers hold by then; anything else
    in the key (here an i32 argument, then the grid) is a run of its own, and KAPY_MLIR_PLAN=0 turns the cache off."""
    rows_per_warp, cols, warps, programs = 4, 256, 2, 6
    rows = rows_per_warp * warps * programs
    text = kp.binary_program("arith.addf", rows_per_warp, cols, warps)
    prog = ko.program([dict(op=ko.EW_LD_GLOBAL, dst=0, a=0), dict(op=ko.EW_LD_GLOBAL, dst=1, a=1), dict(op=ko.EW_ADDF, dst=2, a=0, b=1), dict(op=ko.EW_ST_GLOBAL, a=2)])
    g = lambda a: ko.mk_global(a, rows, cols, cols, 1, ko.F16)

    def want_of(x, y):
        want = np.zeros(rows * cols, np.uint16)
        assert ko.elementwise(prog, [g(x), g(y)], g(want)) == 0
        return want
    x1, y1 = ko.fill_normal(rows * cols, ko.F16, 11), ko.fill_normal(rows * cols, ko.F16, 12)
    x2, y2 = ko.fill_normal(rows * cols, ko.F16, 13), ko.fill_normal(rows * cols, ko.F16, 14)
    dx, dy, dout = to_dev(x1), to_dev(y1), dev_zeros(rows * cols, 2, fill=0x7e00)
    plans0, replays0, _ = kh.run_mlir_plan_stats()
    kh.run_mlir(text, [dx, dy, dout, rows], [programs])
    sync()
    assert kh.run_mlir_plan_stats()[:2] == (plans0 + 1, replays0)
    assert np.array_equal(to_host(dout, np.uint16), want_of(x1, y1))
    # other contents in the same buffers: the kept calls, the new sums
    dx.copy_(to_dev(x2)); dy.copy_(to_dev(y2)); dout.fill_(0x7e00)
    merged0 = kh.run_mlir_stats()
    kh.run_mlir(text, [dx, dy, dout, rows], [programs])
    sync()
    assert kh.run_mlir_plan_stats()[:2] == (plans0 + 1, replays0 + 1)
    assert kh.run_mlir_stats() - merged0 == 1     # (the statistics of the kept run count again)
    assert np.array_equal(to_host(dout, np.uint16), want_of(x2, y2))
    # fewer rows (an i32 argument) and fewer programs: runs of their own
    dout.fill_(0x7e00)
    fewer = rows - rows_per_warp * warps
    kh.run_mlir(text, [dx, dy, dout, fewer], [programs - 1])
    sync()
    assert kh.run_mlir_plan_stats()[:2] == (plans0 + 2, replays0 + 1)
    got = to_host(dout, np.uint16)
    assert np.array_equal(got[:fewer * cols], want_of(x2, y2)[:fewer * cols]) and np.all(got[fewer * cols:] == 0x7e00)
    # the cache off: nothing kept, nothing replayed, the same result
    monkeypatch.setenv("KAPY_MLIR_PLAN", "0")
    dout.fill_(0x7e00)
    kh.run_mlir(text, [dx, dy, dout, rows], [programs])
    sync()
    assert kh.run_mlir_plan_stats()[:2] == (plans0 + 2, replays0 + 1)
    assert np.array_equal(to_host(dout, np.uint16), want_of(x2, y2))
    monkeypatch.delenv("KAPY_MLIR_PLAN")


@pytest.mark.parametrize("bm,bn,bk,way,acc,dtype,M,N,K", [
    (64, 64, 16, "mma_m16n8k8_f16", "f16", "f16", 256, 256, 128),    # the fixture's tiling; K steps of half an instruction's 32
    (64, 64, 32, "mma_m16n8k16_f16", "f32", "f16", 128, 256, 96),
    (32, 64, 64, "mma_m16n8k16_f16", "f32", "bf16", 128, 128, 192),  # two instructions per step
    (32, 32, 32, "mma_m16n8k16_f16", "f16", "f16", 64, 128, 32),     # one K step: the loop body never runs
])
def test_a_kept_run_makes_the_copies_and_products_of_all_instances_in_one_launch_each(ko, monkeypatch, bm, bn, bk, way, acc, dtype, M, N, K):
    """A program with a loop, shared-memory buffers and kapy.matmul makes one call per instance, warp and op when it is
    interpreted (hundreds to thousands a run).  In the kept run the same copy or product of all instances in flight is one
    launch over a table of their addresses: the replay gives the bits of the first run, which made the calls one by one
    (and is compared with the oracle by test_matmul_program_matches_oracle), with and without the tables."""
    kd = ko.F16 if dtype == "f16" else ko.BF16
    a, b = ko.fill_normal(M * K, kd, 31, 0, 0.0, 0.5), ko.fill_normal(K * N, kd, 32, 0, 0.0, 0.5)
    acc_bytes = 2 if acc == "f16" else 4
    grid = [(M // (2 * bm)) * (N // (2 * bn))]
    mm = kp.matmul_program(bm, bn, bk, way, acc, dtype)
    outs = {}
    for tables in ("1", "0"):
        monkeypatch.setenv("KAPY_MLIR_PLAN_BATCH", tables)
        da, db, dc = to_dev(a), to_dev(b), dev_zeros(M * N, acc_bytes, fill=0x7e00)
        kh.run_mlir(mm, [da, db, dc, M, N, K], grid)
        sync()
        first = to_host(dc, np.uint8).copy()
        dc.fill_(0x7e00)
        _, replays0, tables0 = kh.run_mlir_plan_stats()
        kh.run_mlir(mm, [da, db, dc, M, N, K], grid)
        sync()
        _, replays1, tables1 = kh.run_mlir_plan_stats()
        assert replays1 == replays0 + 1
        steps = K // bk
        # per K step at most: two copies into shared memory, two out of it and a product, each for all instances at once
        # (fewer where calls of one shape from neighbouring ops join one table, a few more where a group splits); the store of
        # the result is one more
        if tables == "1":
            assert 3 * steps <= tables1 - tables0 <= 6 * steps + 2, (tables1 - tables0, steps)
        else:
            assert tables1 == tables0
        got = to_host(dc, np.uint8)
        assert np.array_equal(got, first)
        outs[tables] = got
    assert np.array_equal(outs["1"], outs["0"])


@pytest.mark.parametrize("fuse", ["1", "0"])
@pytest.mark.parametrize("family", ["exchange", "exchange_narrow", "exchange_loop", "phases", "aliasing", "block_sum", "transpose", "softmax", "column_softmax",
                                    "causal_softmax", "gated", "reduce"])
def test_a_replayed_run_has_the_bits_of_the_interpreted_run(ko, monkeypatch, family, fuse):
    """Every program family of this file twice on the same buffers (inputs and results restored in between): the second call
    is served from the kept run - calls regrouped, copies of all instances in one launch where they are independent - and
    must leave what the interpreted first call left; a third pair does the same with the tables switched off.  The programs
    that exchange tiles through shared memory, overwrite what earlier loads read or update a buffer in place are the ones a
    wrong dependence test would break.  KAPY_MLIR_FUSE=0 runs every op as a call of its own (many more copies)."""
    monkeypatch.setenv("KAPY_MLIR_FUSE", fuse)
    f16 = lambda n, seed: ko.fill_normal(n, ko.F16, seed)
    if family in ("exchange", "exchange_narrow"):
        rpw, cols, warps, programs = (16, 64, 4, 3) if family == "exchange" else (8, 40, 2, 3)   # (rows of 80 bytes: no 16-byte pieces)
        rows = rpw * warps * programs
        bufs = [f16(rows * cols, 61), np.full(rows * cols, 0x7e00, np.uint16)]
        text, args, grid, outs = kp.exchange_program(rpw, cols, warps), lambda d: [d[0], d[1], rows], [programs], [1]
    elif family == "exchange_loop":
        rpw, cols, warps, steps, programs = 8, 64, 4, 3, 2
        rows = rpw * warps * programs
        bufs = [f16(rows * cols, 62), np.full(rows * cols, 0x7e00, np.uint16)]
        text, args, grid, outs = kp.exchange_loop_program(rpw, cols, warps, steps), lambda d: [d[0], d[1], rows], [programs], [1]
    elif family == "phases":
        bufs = [f16(64 * 64, 41)]
        text, args, grid, outs = kp.phases_program(), lambda d: [d[0]], [1], [0]
    elif family == "aliasing":
        rpw, cols, warps, programs = 4, 128, 2, 3
        rows = rpw * warps * programs
        bufs = [f16(rows * cols, 71), f16(rows * cols, 72), np.full(rows * cols, 0x7e00, np.uint16)]
        text, args, grid, outs = kp.aliasing_program(rpw, cols, warps), lambda d: [d[0], d[1], d[2], rows], [programs], [0, 2]
    elif family == "block_sum":
        rpw, bc, warps, programs, cols = 4, 64, 2, 3, 256
        rows = rpw * warps * programs
        bufs = [f16(rows * cols, 81), np.full(rows * bc, 0x7e00, np.uint16)]
        text, args, grid, outs = kp.block_sum_program(rpw, bc, warps), lambda d: [d[0], d[1], rows, cols], [programs], [1]
    elif family == "transpose":
        m, n, tile = 96, 64, 32
        bufs = [f16(m * n, 52), np.full(m * n, 0x7e00, np.uint16)]
        text, args, grid, outs = kp.scaled_transpose_program(tile, 0.5), lambda d: [d[0], d[1], m, n], [m // tile, n // tile], [1]
    elif family == "column_softmax":
        rows, cpw, warps, programs = 64, 64, 2, 3
        cols = cpw * warps * programs
        bufs = [f16(rows * cols, 91), np.full(rows * cols, 0x7e00, np.uint16)]
        text, args, grid, outs = kp.column_softmax_program(rows, cpw, warps), lambda d: [d[0], d[1], cols], [programs], [1]
    elif family == "gated":
        rpw, cols, warps, programs = 4, 256, 2, 3
        rows = rpw * warps * programs
        bufs = [f16(rows * cols, 1), f16(rows * cols, 2), f16(rows * cols, 3), np.full(rows * cols, 0x7e00, np.uint16)]
        text, args, grid, outs = kp.gated_program(rpw, cols, warps), lambda d: [d[0], d[1], d[2], d[3], rows], [programs], [3]
    elif family == "reduce":
        rpw, cols, warps, programs = 2, 256, 2, 8
        rows = rpw * warps * programs
        bufs = [f16(rows * cols, 21), np.full(rows, 0x7e00, np.uint16)]
        text, args, grid, outs = kp.reduce_program("arith.addf", rpw, cols, warps), lambda d: [d[0], d[1], rows], [programs], [1]
    else:
        rpw, cols, warps, programs = 2, 256, 2, 5
        rows = rpw * warps * programs
        bufs = [f16(rows * cols, 31), np.full(rows * cols, 0x7e00, np.uint16)]
        gen = kp.softmax_program if family == "softmax" else kp.causal_softmax_program
        text, args, grid, outs = gen(rpw, cols, warps), lambda d: [d[0], d[1], rows], [programs], [1]
    dev = [to_dev(b) for b in bufs]

    def run():
        for d, b in zip(dev, bufs):
            d.copy_(to_dev(b))
        kh.run_mlir(text, args(dev), grid)
        sync()
        return [to_host(dev[k], np.uint16).copy() for k in outs]
    results = []
    for tables in ("1", "0"):
        monkeypatch.setenv("KAPY_MLIR_PLAN_BATCH", tables)
        plans0, replays0, _ = kh.run_mlir_plan_stats()
        results.append(run())
        assert kh.run_mlir_plan_stats()[:2] == (plans0 + 1, replays0)
        results.append(run())
        assert kh.run_mlir_plan_stats()[:2] == (plans0 + 1, replays0 + 1)
    for r in results[1:]:
        assert all(np.array_equal(x, y) for x, y in zip(r, results[0]))
