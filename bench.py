#!/usr/bin/env python3
"""Benchmark of the kapy hot path on one MI355X.

`python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload NAME] [--no-others] [--skip NAMES] [--no-cpu]`

A step is one pass of the hot path over one batch of synthetic input, inputs resident in HBM.
The headline workload (the configuration the headline metric is quoted on) is the fused elementwise
y = GELU_tanh(x*0.5 + bias) on fp16 8192x8192; the JSON line also carries every other benchmark
configuration under "other_workloads", each with its own roofline.  One JSON line on stdout.

Inputs are the ones each configuration states, generated on the host by the seeded counter-based generators of
the CPU checker (fp64, rounded once to the storage type) and uploaded: the GPU and the checker see the same bytes.
Before a workload is timed, one launch on the timed buffers is compared with the checker (sampled rows / blocks for
the large shapes, the tolerance of the configuration): a workload that fails is not timed and is reported as failed.

Timing: K launches bracketed by torch.cuda.synchronize() give ms_per_step / value; HIP events
recorded on the stream the kernels are launched on (torch's current stream, whose handle is
passed to the C ABI) give the per-launch duration used for roofline.achieved.  Memory-bound
workloads rotate over buffer sets larger than the 256 MB Infinity Cache so the rate is HBM's.

cpu_baseline: the same workload (or a stated slice of it) through the host implementations written for speed in
oracle/kapy_baseline.cpp, over all the host threads this process may use, in the same run.
"""
import argparse
import ctypes as C
import json
import os
import re
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.join(ROOT, "kapy-lang_amd", "python"))
sys.path.insert(0, os.path.join(ROOT, "oracle"))

HBM_PEAK_GBS = 8000.0
MFMA_PEAK_TFLOPS = {"bf16": 2500.0, "f16": 2500.0, "f8": 5000.0}
FROB_TOL = 1e-3        # GEMMs: relative Frobenius error against the fp64-accumulated checker
ULP_TOL = 2            # elementwise: units in the last place of the 16-bit result
CPU_SECONDS = 2.0      # wall time each cpu_baseline leg repeats its workload for

PREWARM_S = 0.25  # untimed launches before the W warm-up steps: the GPU clock needs ~0.2 s of load to settle


class CheckFailed(Exception):
    pass


def _events(fn, steps, warmup):
    """Run fn(i) untimed until the clock has settled, then warmup + steps times;
    return (wall ms per step, event ms per launch)."""
    import gc
    import torch
    gc.collect()   # (now, not between the warm-up and the timed steps: the device clock falls within a fraction of a second of idling)
    t0, i = time.perf_counter(), 0
    while time.perf_counter() - t0 < PREWARM_S:
        fn(i)
        i += 1
        if i % 8 == 0:
            torch.cuda.synchronize()
    for i in range(warmup):
        fn(i)
    torch.cuda.synchronize()
    # The launches are queued back to back between events; an event every fifth of the way, and the per-launch figure is the
    # median of the fifths: a pause of the launching thread inside the timed region (the collector, a worker pool of a CPU leg
    # winding down) once put a millisecond of idle queue into a 20-launch average of a 13 us kernel.  The wall clock is over all
    # steps, pauses included.
    parts = 5 if steps >= 10 else 1
    marks = [torch.cuda.Event(enable_timing=True) for _ in range(parts + 1)]
    at = [steps * k // parts for k in range(parts + 1)]
    gc.disable()
    try:
        t0 = time.perf_counter()
        marks[0].record()
        k = 1
        for i in range(steps):
            fn(i)
            if i + 1 == at[k]:
                marks[k].record()
                k += 1
        torch.cuda.synchronize()
        wall_ms = (time.perf_counter() - t0) * 1e3 / steps
    finally:
        gc.enable()
    per_launch = sorted(marks[k].elapsed_time(marks[k + 1]) / (at[k + 1] - at[k]) for k in range(parts))
    return wall_ms, per_launch[parts // 2]


# HBM bytes per launch from rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE (two runs), each scaled by what the same counter reads
# for the rows copy of 2 x 128 MiB (workload "copy").  The figures are read from the tracked summary of those runs (its
# lines "traffic_bytes <workload> <bytes>"), which `bench.py --pmc-summary` writes from the profiler's output.
TRAFFIC_SUMMARY = os.path.join(ROOT, "profiles", "bench_all_workloads.hbm_traffic_pmc.txt")


def _read_traffic(path=TRAFFIC_SUMMARY):
    out = {}
    try:
        for l in open(path):
            f = l.split()
            if len(f) == 3 and f[0] == "traffic_bytes":
                out[f[1]] = int(f[2])
    except OSError:
        pass
    return out


MEASURED_TRAFFIC = _read_traffic()


def _roof_hbm(bytes_per_launch, ev_ms, key=None):
    a = bytes_per_launch / (ev_ms * 1e-3) / 1e9
    return {"bound": "hbm", "achieved": round(a, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": round(a / HBM_PEAK_GBS, 4),
            "traffic": MEASURED_TRAFFIC.get(key)}


def _roof_mfma(flops, ev_ms, kind, key=None):
    a = flops / (ev_ms * 1e-3) / 1e12
    p = MFMA_PEAK_TFLOPS[kind]
    return {"bound": "mfma", "achieved": round(a, 1), "peak": p, "unit": "TFLOP/s", "frac": round(a / p, 4), "traffic": MEASURED_TRAFFIC.get(key)}


# ---------------------------------------------------------------- seeded inputs (host-generated, cached on the device)
_host_cache, _dev_cache = {}, {}


def _host(kind, n, dtype, seed, stream=0, **kw):
    """A seeded host array from the checker's generators; kept, because several workloads share the large ones."""
    import ko
    key = (kind, n, dtype, seed, stream, tuple(sorted(kw.items())))
    if key not in _host_cache:
        if kind == "normal":
            _host_cache[key] = ko.fill_normal(n, dtype, seed, stream, kw.get("mean", 0.0), kw.get("std", 1.0))
        elif kind == "uniform":
            _host_cache[key] = ko.fill_uniform(n, dtype, seed, stream, kw.get("lo", -1.0), kw.get("hi", 1.0))
        else:
            _host_cache[key] = ko.fill_bits16(n, seed, stream)
    return _host_cache[key]


def _dev(kind, n, dtype, seed, stream=0, **kw):
    import numpy as np
    import torch
    key = (kind, n, dtype, seed, stream, tuple(sorted(kw.items())))
    if key not in _dev_cache:
        a = _host(kind, n, dtype, seed, stream, **kw)
        _dev_cache[key] = torch.from_numpy(a.view({1: np.uint8, 2: np.int16, 4: np.int32}[a.itemsize])).cuda()
    return _dev_cache[key]


def _upload(a):
    import numpy as np
    import torch
    a = np.ascontiguousarray(a)
    return torch.from_numpy(a.view({1: np.uint8, 2: np.int16, 4: np.int32}[a.itemsize]).reshape(-1)).cuda()


def _download(t, np_dtype, shape):
    return t.cpu().numpy().view(np_dtype).reshape(shape)


def _line16(v):
    """16-bit float patterns on the monotone integer line (for ulp distances)."""
    import numpy as np
    v = v.astype(np.int32)
    return np.where(v & 0x8000, -(v & 0x7FFF), v & 0x7FFF)


def _sample_rows(n, count):
    step = n // count
    return [(k * step + (7 * k) % step) % n for k in range(count)]


def _cpu_repeat(fn, work_per_call, unit_scale, unit, sample):
    """Time fn() repeatedly for about CPU_SECONDS (after one warm-up call)."""
    import ko
    fn()
    reps, t0 = 0, time.perf_counter()
    while True:
        fn()
        reps += 1
        dt = time.perf_counter() - t0
        if dt > CPU_SECONDS:
            break
    return {"value": round(work_per_call * reps / dt / unit_scale, 3), "unit": unit, "cores": ko.lib().ko_num_threads(), "kind": "port",
            "sample": "%s; %d repetitions in %.1f s" % (sample, reps, dt)}


# ---------------------------------------------------------------- memory-bound workloads
def bench_gelu(kh, steps, warmup, cpu):
    """C2: x fp16 8192x8192 normal(0,1) seed 0, bias fp16 [8192] normal(0,1) seed 1 broadcast along rows, scale 0.5."""
    import numpy as np
    import torch
    import ko
    n, sets = 8192, 4
    xs = [_dev("normal", n * n, ko.F16, 0, k) for k in range(sets)]       # set 0 is the configuration's x; the others rotate past the cache
    ys = [torch.empty(n * n, device="cuda", dtype=torch.int16) for _ in range(sets)]
    bias = _dev("normal", n, ko.F16, 1)
    prog = kh.gelu_program(kh.F16, 0.5)
    gx = [kh.mk_global(x.data_ptr(), n, n, n, 1, kh.F16) for x in xs]
    gy = [kh.mk_global(y.data_ptr(), n, n, n, 1, kh.F16) for y in ys]
    gb = kh.mk_global(bias.data_ptr(), 1, n, n, 1, kh.F16)
    # gate: 32 rows of the result against the checker
    kh.elementwise(prog, [gx[0], gb], gy[0])
    torch.cuda.synchronize()
    hx, hb = _host("normal", n * n, ko.F16, 0, 0).reshape(n, n), _host("normal", n, ko.F16, 1)
    rows = _sample_rows(n, 32)
    got = _download(ys[0], np.uint16, (n, n))[rows]
    xr, want = np.ascontiguousarray(hx[rows]), np.zeros((len(rows), n), np.uint16)
    assert ko.elementwise(ko.gelu_program(), [ko.mk_global(xr, len(rows), n, n, 1, ko.F16), ko.mk_global(hb, 1, n, n, 1, ko.F16)],
                          ko.mk_global(want, len(rows), n, n, 1, ko.F16)) == 0
    worst = int(np.abs(_line16(got) - _line16(want)).max())
    if worst > ULP_TOL:
        raise CheckFailed("gelu: %d ulp against the checker" % worst)
    wall, ev = _events(lambda i: kh.elementwise(prog, [gx[i % sets], gb], gy[i % sets]), steps, warmup)
    nbytes = 2 * n * n * 2 + n * 2
    out = {"workload": "C2 gelu_tanh(x*0.5+bias) fp16 8192x8192", "value": nbytes / (wall * 1e-3) / 1e9, "unit": "GB/s",
           "ms_per_step": wall, "kernel_ms": ev, "dtype": "f16", "roofline": _roof_hbm(nbytes, ev, "gelu"), "kernel": "affine_act_cols_kernel",
           "inputs": "x normal(0,1) seed 0, bias normal(0,1) seed 1, scale 0.5 (host-generated, as the configuration states)",
           "checked": True, "check": "32 rows of the timed result against the checker: max %d ulp (tolerance %d)" % (worst, ULP_TOL)}
    if cpu:
        hy = np.zeros((n, n), np.uint16)
        out["cpu_baseline"] = _cpu_repeat(lambda: ko.lib().ko_baseline_gelu_f16(hx.ctypes.data, hb.ctypes.data, 0.5, hy.ctypes.data, n, n, n),
                                          nbytes, 1e9, "GB/s", "the whole 8192x8192 workload, fused fp32 vector loop")
    return out


def bench_copy(kh, steps, warmup, cpu):
    """Plain row-major copy of the headline shape: the practical HBM ceiling the other kernels are read against,
    and the known-size kernel that calibrates the FETCH_SIZE / WRITE_SIZE counters."""
    import numpy as np
    import torch
    import ko
    n, sets = 8192, 4
    xs = [_dev("bits16", n * n, ko.F16, 0, k) for k in range(sets)]
    ys = [torch.empty(n * n, device="cuda", dtype=torch.int16) for _ in range(sets)]
    gx = [kh.mk_global(x.data_ptr(), n, n, n, 1, kh.F16) for x in xs]
    gy = [kh.mk_global(y.data_ptr(), n, n, n, 1, kh.F16) for y in ys]
    kh.copy(gx[0], gy[0])
    torch.cuda.synchronize()
    if not torch.equal(xs[0], ys[0]):
        raise CheckFailed("copy: result differs from the source")
    wall, ev = _events(lambda i: kh.copy(gx[i % sets], gy[i % sets]), steps, warmup)
    nbytes = 2 * n * n * 2
    return {"workload": "copy fp16 8192x8192 (ld_global -> st_global, no transpose)", "value": nbytes / (wall * 1e-3) / 1e9, "unit": "GB/s",
            "ms_per_step": wall, "kernel_ms": ev, "dtype": "u16", "roofline": _roof_hbm(nbytes, ev, "copy"), "kernel": "rows_kernel",
            "inputs": "uniform random 16-bit patterns seed 0", "checked": True, "check": "whole result bit-equal to the source"}


def bench_add(kh, steps, warmup, cpu, op="add"):
    """z = x + y in fp16 (the reference's elementwise_add.mlir fixture at the headline shape), a plain binary program,
    served by the fused affine kernel; op="expr": z = x*y + x with both roundings, a program outside the fused chains,
    served by the in-register stack machine; op="expr_compiled": the same program after kapy_elementwise_specialize has
    compiled it to a kernel of its own; op="swiglu": z = silu(x) * y in fp32 from fp16 operands (ten ops, x used twice), compiled."""
    import numpy as np
    import torch
    import ko
    n, sets = 8192, 3
    xs = [_dev("normal", n * n, ko.F16, 0, k) for k in range(sets)]
    ys = [_dev("normal", n * n, ko.F16, 0, 3 - k) for k in range(sets)]
    zs = [torch.empty(n * n, device="cuda", dtype=torch.int16) for _ in range(sets)]
    g = lambda t: kh.mk_global(t.data_ptr(), n, n, n, 1, kh.F16)
    gx, gy, gz = [g(t) for t in xs], [g(t) for t in ys], [g(t) for t in zs]
    insts = [dict(op=kh.EW_LD_GLOBAL, dst=0, a=0), dict(op=kh.EW_LD_GLOBAL, dst=1, a=1)]
    if op == "add":
        insts += [dict(op=kh.EW_ADDF, dst=2, a=0, b=1)]
    elif op == "swiglu":
        f32 = lambda r: dict(op=kh.EW_FPTOFP, dst=r, a=r, dtype=kh.F32)
        insts += [f32(0), f32(1), dict(op=kh.EW_NEGF, dst=2, a=0), dict(op=kh.EW_EXP, dst=2, a=2), dict(op=kh.EW_SPLAT, dst=3, dtype=kh.F32, imm=1.0),
                  dict(op=kh.EW_ADDF, dst=2, a=2, b=3), dict(op=kh.EW_DIVF, dst=2, a=0, b=2), dict(op=kh.EW_MULF, dst=2, a=2, b=1),
                  dict(op=kh.EW_FPTOFP, dst=2, a=2, dtype=kh.F16, rmode=kh.RN)]
    else:
        insts += [dict(op=kh.EW_MULF, dst=2, a=0, b=1), dict(op=kh.EW_ADDF, dst=2, a=2, b=0)]
    insts += [dict(op=kh.EW_ST_GLOBAL, a=2)]
    prog = kh.program(insts)
    if op in ("expr_compiled", "swiglu"):
        kh.elementwise_specialize(prog, [gx[0], gy[0]], gz[0])
    kh.elementwise(prog, [gx[0], gy[0]], gz[0])
    torch.cuda.synchronize()
    rows = _sample_rows(n, 16)
    hx, hy = _host("normal", n * n, ko.F16, 0, 0).reshape(n, n), _host("normal", n * n, ko.F16, 0, 3).reshape(n, n)
    xr, yr, want = np.ascontiguousarray(hx[rows]), np.ascontiguousarray(hy[rows]), np.zeros((len(rows), n), np.uint16)
    m = len(rows)
    assert ko.elementwise(ko.program(insts), [ko.mk_global(xr, m, n, n, 1, ko.F16), ko.mk_global(yr, m, n, n, 1, ko.F16)], ko.mk_global(want, m, n, n, 1, ko.F16)) == 0
    got = _download(zs[0], np.uint16, (n, n))[rows]
    worst = int(np.abs(_line16(got) - _line16(want)).max())
    tol = ULP_TOL if op == "swiglu" else 0     # add / mul: exactly rounded ops, bit-exact
    if worst > tol:
        raise CheckFailed("%s: %d ulp against the checker" % (op, worst))
    wall, ev = _events(lambda i: kh.elementwise(prog, [gx[i % sets], gy[i % sets]], gz[i % sets]), steps, warmup)
    nbytes = 3 * n * n * 2
    name = {"add": "elementwise_add fixture: z = x + y fp16 8192x8192", "expr": "z = x*y + x (two roundings) fp16 8192x8192",
            "expr_compiled": "z = x*y + x (two roundings) fp16 8192x8192, compiled at run time",
            "swiglu": "z = silu(x)*y fp16 8192x8192 in fp32, compiled at run time"}[op]
    kernel = {"add": "affine_act_kernel", "expr": "stack_kernel_narrow"}.get(op, "kapy_ew_flat_<hash> (compiled at run time)")
    return {"workload": name, "value": nbytes / (wall * 1e-3) / 1e9, "unit": "GB/s", "ms_per_step": wall, "kernel_ms": ev, "dtype": "f16",
            "roofline": _roof_hbm(nbytes, ev, op), "kernel": kernel, "inputs": "x, y normal(0,1), seeded",
            "checked": True, "check": "16 rows against the checker: max %d ulp (tolerance %d)" % (worst, tol)}


def bench_gelu_transposed(kh, steps, warmup, cpu):
    """y = gelu_tanh(x^T*0.5 + bias): the C3a transpose fused with the C2 chain - x is read through a view with swapped
    strides - compiled at run time onto the tiled skeleton (64 x 64 tiles, the column-major operand staged through LDS)."""
    import numpy as np
    import torch
    import ko
    n, sets = 8192, 4
    xs = [_dev("normal", n * n, ko.F16, 0, k) for k in range(sets)]
    ys = [torch.empty(n * n, device="cuda", dtype=torch.int16) for _ in range(sets)]
    bias = _dev("normal", n, ko.F16, 1)
    gx = [kh.mk_global(x.data_ptr(), n, n, 1, n, kh.F16) for x in xs]       # element (i, j) of the view is x[j, i]
    gy = [kh.mk_global(y.data_ptr(), n, n, n, 1, kh.F16) for y in ys]
    gb = kh.mk_global(bias.data_ptr(), 1, n, n, 1, kh.F16)
    prog = kh.gelu_program(kh.F16, 0.5)
    kh.elementwise_specialize(prog, [gx[0], gb], gy[0])
    kh.elementwise(prog, [gx[0], gb], gy[0])
    torch.cuda.synchronize()
    hx, hb = _host("normal", n * n, ko.F16, 0, 0).reshape(n, n), _host("normal", n, ko.F16, 1)
    rows = _sample_rows(n, 16)
    xr = np.ascontiguousarray(hx[:, rows].T)     # row i of the view is column i of x
    want = np.zeros((len(rows), n), np.uint16)
    assert ko.elementwise(ko.gelu_program(), [ko.mk_global(xr, len(rows), n, n, 1, ko.F16), ko.mk_global(hb, 1, n, n, 1, ko.F16)],
                          ko.mk_global(want, len(rows), n, n, 1, ko.F16)) == 0
    worst = int(np.abs(_line16(_download(ys[0], np.uint16, (n, n))[rows]) - _line16(want)).max())
    if worst > ULP_TOL:
        raise CheckFailed("gelu_transposed: %d ulp against the checker" % worst)
    wall, ev = _events(lambda i: kh.elementwise(prog, [gx[i % sets], gb], gy[i % sets]), steps, warmup)
    nbytes = 2 * n * n * 2 + n * 2
    return {"workload": "gelu_tanh(x^T*0.5+bias) fp16 8192x8192: transpose fused with the elementwise chain, compiled at run time",
            "value": nbytes / (wall * 1e-3) / 1e9, "unit": "GB/s", "ms_per_step": wall, "kernel_ms": ev, "dtype": "f16",
            "roofline": _roof_hbm(nbytes, ev, "gelu_transposed"), "kernel": "kapy_ew_flat_<hash> (tiled; compiled at run time)", "inputs": "as C2, x read through swapped strides",
            "checked": True, "check": "16 rows against the checker: max %d ulp (tolerance %d)" % (worst, ULP_TOL)}


def bench_reduce(kh, steps, warmup, cpu):
    """kapy.reduce (sum along rows) of the headline shape: the first adjacent op after the hot path proper."""
    import numpy as np
    import torch
    import ko
    n, sets = 8192, 4
    xs = [_dev("normal", n * n, ko.F16, 0, k) for k in range(sets)]
    y = torch.empty(n, device="cuda", dtype=torch.float32)
    gx = [kh.mk_global(x.data_ptr(), n, n, n, 1, kh.F16) for x in xs]
    gy = kh.mk_global(y.data_ptr(), n, 1, 1, n, kh.F32)
    kh.reduce(gx[0], gy, 1, 0)
    torch.cuda.synchronize()
    hx = _host("normal", n * n, ko.F16, 0, 0).reshape(n, n)
    want = hx.view(np.float16).astype(np.float64).sum(axis=1)
    err = float(np.abs(y.cpu().numpy().astype(np.float64) - want).max())
    if err > 2e-3:   # fp32 accumulation of 8192 values of magnitude ~1
        raise CheckFailed("reduce: max abs error %g" % err)
    wall, ev = _events(lambda i: kh.reduce(gx[i % sets], gy, 1, 0), steps, warmup)
    nbytes = n * n * 2 + n * 4
    return {"workload": "reduce_sum axis=1 fp16 8192x8192 -> f32 [8192x1]", "value": nbytes / (wall * 1e-3) / 1e9, "unit": "GB/s",
            "ms_per_step": wall, "kernel_ms": ev, "dtype": "f16", "roofline": _roof_hbm(nbytes, ev, "reduce"), "kernel": "reduce_rows_vec_kernel",
            "inputs": "x normal(0,1) seed 0", "checked": True, "check": "every row sum against fp64: max abs error %.2e" % err}


def bench_reduce_cols(kh, steps, warmup, cpu):
    """kapy.reduce along axis 0 (column sums) of the headline shape: strips x row chunks in one launch, the last workgroup to arrive
    at a strip folds its chunks."""
    import numpy as np
    import torch
    import ko
    n, sets = 8192, 4
    xs = [_dev("normal", n * n, ko.F16, 0, k) for k in range(sets)]
    y = torch.empty(n, device="cuda", dtype=torch.float32)
    gx = [kh.mk_global(x.data_ptr(), n, n, n, 1, kh.F16) for x in xs]
    gy = kh.mk_global(y.data_ptr(), 1, n, n, 1, kh.F32)
    kh.reduce(gx[0], gy, 0, 0)
    torch.cuda.synchronize()
    hx = _host("normal", n * n, ko.F16, 0, 0).reshape(n, n)
    want = hx.view(np.float16).astype(np.float64).sum(axis=0)
    err = float(np.abs(y.cpu().numpy().astype(np.float64) - want).max())
    if err > 2e-3:
        raise CheckFailed("reduce along axis 0: max abs error %g" % err)
    wall, ev = _events(lambda i: kh.reduce(gx[i % sets], gy, 0, 0), steps, warmup)
    nbytes = n * n * 2 + n * 4
    return {"workload": "reduce_sum axis=0 fp16 8192x8192 -> f32 [1x8192]", "value": nbytes / (wall * 1e-3) / 1e9, "unit": "GB/s",
            "ms_per_step": wall, "kernel_ms": ev, "dtype": "f16", "roofline": _roof_hbm(nbytes, ev, "reduce_cols"), "kernel": "reduce_cols_strip_kernel (one launch: the last workgroup of a strip folds the row chunks)",
            "inputs": "x normal(0,1) seed 0", "checked": True, "check": "every column sum against fp64: max abs error %.2e" % err}


def bench_softmax_cols(kh, steps, warmup, cpu):
    """Softmax of every column as one program with two reduces along axis 0: two launches over the matrix (per-column maximum and
    sum of exp with a running rescale, then the store), x read twice and y written once."""
    import numpy as np
    import torch
    import ko
    n, sets = 8192, 2
    xs = [_dev("normal", n * n, ko.F16, 0, k) for k in range(sets)]
    ys = [torch.empty(n * n, device="cuda", dtype=torch.int16) for _ in range(sets)]
    g = lambda t: kh.mk_global(t.data_ptr(), n, n, n, 1, kh.F16)
    gx, gy = [g(t) for t in xs], [g(t) for t in ys]
    insts = [dict(i) for i in kh.softmax_insts(kh.F16)]
    for i in insts:
        if i["op"] in (kh.EW_REDUCE_MAX, kh.EW_REDUCE_SUM):
            i["b"] = 0
    prog = kh.program(insts)
    kh.elementwise(prog, [gx[0]], gy[0])
    torch.cuda.synchronize()
    # gate: 16 columns against the checker (columns are independent)
    cols = _sample_rows(n, 16)
    hx = _host("normal", n * n, ko.F16, 0, 0).reshape(n, n)
    xc, want = np.ascontiguousarray(hx[:, cols]), np.zeros((n, len(cols)), np.uint16)
    assert ko.elementwise(ko.program(insts), [ko.mk_global(xc, n, len(cols), len(cols), 1, ko.F16)], ko.mk_global(want, n, len(cols), len(cols), 1, ko.F16)) == 0
    worst = int(np.abs(_line16(_download(ys[0], np.uint16, (n, n))[:, cols]) - _line16(want)).max())
    if worst > ULP_TOL:
        raise CheckFailed("column softmax: %d ulp against the checker" % worst)
    wall, ev = _events(lambda i: kh.elementwise(prog, [gx[i % sets]], gy[i % sets]), steps, warmup)
    nbytes = 2 * n * n * 2
    return {"workload": "softmax of every column, fp16 8192x8192, fp32 arithmetic (program with two reduces along axis 0)", "value": nbytes / (wall * 1e-3) / 1e9, "unit": "GB/s",
            "ms_per_step": wall, "kernel_ms": ev, "dtype": "f16", "roofline": _roof_hbm(nbytes, ev, "softmax_cols"),
            "kernel": "col_softmax_stats_kernel + col_softmax_apply_kernel", "inputs": "x normal(0,1) seed 0", "checked": True,
            "check": "16 columns of the timed result against the checker: max %d ulp (tolerance %d); bytes = one read and one write of the matrix (the two launches read it twice)" % (worst, ULP_TOL)}


def bench_rowwise(kh, steps, warmup, cpu, which):
    """Row-wise fusion of kapy.reduce with its elementwise neighbours at the headline shape: softmax or layer norm of
    every row in one pass over HBM (one read of x, one write of y; gamma and beta stay in cache)."""
    import numpy as np
    import torch
    import ko
    n, sets = 8192, 4
    xs = [_dev("normal", n * n, ko.F16, 0, k) for k in range(sets)]
    ys = [torch.empty(n * n, device="cuda", dtype=torch.int16) for _ in range(sets)]
    gamma, beta = _dev("normal", n, ko.F16, 2, 0, mean=1.0, std=0.1), _dev("normal", n, ko.F16, 2, 1, std=0.1)
    g = lambda t: kh.mk_global(t.data_ptr(), n, n, n, 1, kh.F16)
    row = lambda t: kh.mk_global(t.data_ptr(), 1, n, n, 1, kh.F16)
    gx, gy = [g(t) for t in xs], [g(t) for t in ys]
    hextra = []
    if which == "softmax":
        insts, extra = kh.softmax_insts(kh.F16), []
    elif which == "causal_softmax":    # softmax over the columns j <= i of every row: arange, cmpi and select in front of the softmax chain
        L, ST = kh.EW_LD_GLOBAL, kh.EW_ST_GLOBAL
        insts, extra = [dict(op=L, dst=0, a=0), dict(op=kh.EW_FPTOFP, dst=1, a=0, dtype=kh.F32),
                        dict(op=kh.EW_ARANGE, dst=2, a=0, b=0), dict(op=kh.EW_ARANGE, dst=3, a=0, b=1), dict(op=kh.EW_CMPI, dst=4, a=3, b=2, c=kh.CMPI_SLE),
                        dict(op=kh.EW_SPLAT, dst=5, dtype=kh.F32, imm=float("-inf")), dict(op=kh.EW_SELECT, dst=1, a=4, b=1, c=5),
                        dict(op=kh.EW_REDUCE_MAX, dst=6, a=1, b=1), dict(op=kh.EW_SUBF, dst=1, a=1, b=6), dict(op=kh.EW_EXP, dst=1, a=1),
                        dict(op=kh.EW_REDUCE_SUM, dst=6, a=1, b=1), dict(op=kh.EW_DIVF, dst=1, a=1, b=6),
                        dict(op=kh.EW_FPTOFP, dst=7, a=1, dtype=kh.F16, rmode=kh.RN), dict(op=ST, a=7)], []
    elif which == "l2norm_compiled":   # x / |x| per row: a row program without a hand-written kernel, compiled at run time
        f32 = dict(op=kh.EW_FPTOFP, dst=0, a=0, dtype=kh.F32)
        insts, extra = [dict(op=kh.EW_LD_GLOBAL, dst=0, a=0), f32, dict(op=kh.EW_MULF, dst=1, a=0, b=0), dict(op=kh.EW_REDUCE_SUM, dst=1, a=1, b=1),
                        dict(op=kh.EW_RSQRT, dst=1, a=1), dict(op=kh.EW_MULF, dst=0, a=0, b=1),
                        dict(op=kh.EW_FPTOFP, dst=2, a=0, dtype=kh.F16, rmode=kh.RN), dict(op=kh.EW_ST_GLOBAL, a=2)], []
    else:
        insts, extra = kh.layernorm_insts(n, kh.F16), [row(gamma), row(beta)]
        hextra = [_host("normal", n, ko.F16, 2, 0, mean=1.0, std=0.1), _host("normal", n, ko.F16, 2, 1, std=0.1)]
    prog = kh.program(insts)
    if which == "l2norm_compiled":
        kh.elementwise_specialize(prog, [gx[0]], gy[0])
    kh.elementwise(prog, [gx[0]] + extra, gy[0])
    torch.cuda.synchronize()
    rows = _sample_rows(n, 16)
    hx = _host("normal", n * n, ko.F16, 0, 0).reshape(n, n)
    if which == "causal_softmax":   # the mask depends on the row's index: a band of rows where they lie, through a sub-view of the whole matrix
        r0 = 5000
        rows = list(range(r0, r0 + 16))
        full, want_full = ko.mk_global(hx, n, n, n, 1, ko.F16), np.zeros((n, n), np.uint16)
        probe = [dict(i, a=r0) if i["op"] == kh.EW_ARANGE and i["b"] == 0 else i for i in insts]   # the band's first row as arange's start
        assert ko.elementwise(ko.program(probe), [ko.sv_global(full, r0, r0 + 16, 0, n)], ko.sv_global(ko.mk_global(want_full, n, n, n, 1, ko.F16), r0, r0 + 16, 0, n)) == 0
        want = want_full[rows]
    else:
        xr, want = np.ascontiguousarray(hx[rows]), np.zeros((len(rows), n), np.uint16)
        assert ko.elementwise(ko.program(insts), [ko.mk_global(xr, len(rows), n, n, 1, ko.F16)] + [ko.mk_global(h, 1, n, n, 1, ko.F16) for h in hextra],
                              ko.mk_global(want, len(rows), n, n, 1, ko.F16)) == 0
    worst = int(np.abs(_line16(_download(ys[0], np.uint16, (n, n))[rows]) - _line16(want)).max())
    if worst > ULP_TOL:
        raise CheckFailed("%s: %d ulp against the checker" % (which, worst))
    wall, ev = _events(lambda i: kh.elementwise(prog, [gx[i % sets]] + extra, gy[i % sets]), steps, warmup)
    nbytes = 2 * n * n * 2
    name = {"l2norm_compiled": "x * rsqrt(sum x^2) of every row, compiled at run time",
            "causal_softmax": "causal-masked softmax of every row (arange, cmpi, select + the softmax chain), compiled at run time"}.get(which, "%s of every row" % which)
    return {"workload": "%s, fp16 8192x8192, fp32 arithmetic" % name, "value": nbytes / (wall * 1e-3) / 1e9, "unit": "GB/s",
            "ms_per_step": wall, "kernel_ms": ev, "dtype": "f16", "roofline": _roof_hbm(nbytes, ev, which),
            "kernel": {"softmax": "softmax_kernel", "layernorm": "norm_kernel"}.get(which, "kapy_ew_rows_<hash> (compiled at run time)"),
            "inputs": "x normal(0,1) seed 0" + ("; gamma normal(1,0.1), beta normal(0,0.1) seed 2" if hextra else ""),
            "checked": True, "check": "16 rows against the checker: max %d ulp (tolerance %d)" % (worst, ULP_TOL)}


def bench_transpose(kh, steps, warmup, cpu):
    """C3a: fp16 8192x8192, uniform random 16-bit patterns seed 0; out[j,i] = in[i,j], bit-exact."""
    import numpy as np
    import torch
    import ko
    n, sets = 8192, 4
    xs = [_dev("bits16", n * n, ko.F16, 0, k) for k in range(sets)]
    ys = [torch.empty(n * n, device="cuda", dtype=torch.int16) for _ in range(sets)]
    gx = [kh.mk_global(x.data_ptr(), n, n, n, 1, kh.F16) for x in xs]
    gy = [kh.mk_global(y.data_ptr(), n, n, n, 1, kh.F16) for y in ys]
    kh.copy(gx[0], gy[0], transpose=True)
    torch.cuda.synchronize()
    # gate: 4 bands of 64 result rows against the checker's ld_global -> transpose -> st_global, and every element against
    # the index formula itself (a device-side comparison with the strided view of the source)
    hx = _host("bits16", n * n, ko.F16, 0, 0)
    gsrc = ko.mk_global(hx, n, n, n, 1, ko.F16)
    got = _download(ys[0], np.uint16, (n, n))
    for r0 in (0, 2752, 5440, n - 64):
        want = np.zeros((64, n), np.uint16)
        assert ko.lib().ko_copy(C.byref(ko.sv_global(gsrc, 0, n, r0, r0 + 64)), C.byref(ko.mk_global(want, 64, n, n, 1, ko.F16)), 1, 0) == 0
        if not np.array_equal(got[r0:r0 + 64], want):
            raise CheckFailed("transpose: rows %d.. differ from the checker" % r0)
    if not torch.equal(ys[0].view(n, n), xs[0].view(n, n).t()):
        raise CheckFailed("transpose: result is not the transpose of the source")
    wall, ev = _events(lambda i: kh.copy(gx[i % sets], gy[i % sets], transpose=True), steps, warmup)
    nbytes = 2 * n * n * 2
    out = {"workload": "C3a transpose fp16 8192x8192", "value": nbytes / (wall * 1e-3) / 1e9, "unit": "GB/s", "ms_per_step": wall,
           "kernel_ms": ev, "dtype": "u16", "roofline": _roof_hbm(nbytes, ev, "transpose"), "kernel": "transpose_lds_kernel",
           "inputs": "uniform random 16-bit patterns seed 0 (as the configuration states)", "checked": True,
           "check": "256 result rows bit-equal to the checker; every element bit-equal to in[j,i]"}
    if cpu:
        hy = np.zeros(n * n, np.uint16)
        out["cpu_baseline"] = _cpu_repeat(lambda: ko.lib().ko_baseline_transpose16(hx.ctypes.data, hy.ctypes.data, n, n), nbytes, 1e9, "GB/s",
                                          "the whole 8192x8192 transpose, 64x64 tiles")
    return out


def bench_permute(kh, steps, warmup, cpu):
    """C3b: bf16 [8,32,2048,128] random 16-bit patterns seed 1; out[b,s,h,d] = in[b,h,s,d], bit-exact."""
    import numpy as np
    import torch
    import ko
    b, h, s, d, sets = 8, 32, 2048, 128, 4
    tot = b * h * s * d
    xs = [_dev("bits16", tot, ko.F16, 1, k) for k in range(sets)]
    ys = [torch.empty(tot, device="cuda", dtype=torch.int16) for _ in range(sets)]
    gx = [kh.mk_global(x.data_ptr(), s, d, d, 1, kh.BF16) for x in xs]
    gy = [kh.mk_global(y.data_ptr(), s, d, h * d, 1, kh.BF16) for y in ys]
    grid = (b, h, h * s * d, s * d, s * h * d, d)
    kh.copy_batched(gx[0], gy[0], grid)
    torch.cuda.synchronize()
    # gate: 8 of the 256 (b,h) programs against the checker, and every element against the index formula
    hx = _host("bits16", tot, ko.F16, 1, 0)
    got = _download(ys[0], np.uint16, (b, s, h, d))
    for t in range(8):
        ib, ih = t, (5 * t + 3) % h
        want = np.zeros((s, d), np.uint16)
        src = hx[(ib * h + ih) * s * d:(ib * h + ih + 1) * s * d]
        assert ko.lib().ko_copy(C.byref(ko.mk_global(src, s, d, d, 1, ko.BF16)), C.byref(ko.mk_global(want, s, d, d, 1, ko.BF16)), 0, 0) == 0
        if not np.array_equal(got[ib, :, ih, :], want):
            raise CheckFailed("permute: program (%d,%d) differs from the checker" % (ib, ih))
    if not torch.equal(ys[0].view(b, s, h, d), xs[0].view(b, h, s, d).permute(0, 2, 1, 3)):
        raise CheckFailed("permute: result is not the permuted source")
    wall, ev = _events(lambda i: kh.copy_batched(gx[i % sets], gy[i % sets], grid), steps, warmup)
    nbytes = 2 * tot * 2
    out = {"workload": "C3b permute bf16 [8,32,2048,128] bhsd->bshd", "value": nbytes / (wall * 1e-3) / 1e9, "unit": "GB/s",
           "ms_per_step": wall, "kernel_ms": ev, "dtype": "u16", "roofline": _roof_hbm(nbytes, ev, "permute"), "kernel": "rows_kernel",
           "inputs": "uniform random 16-bit patterns seed 1 (as the configuration states)", "checked": True,
           "check": "8 of 256 (b,h) programs bit-equal to the checker; every element bit-equal to in[b,h,s,d]"}
    if cpu:
        hy = np.zeros(tot, np.uint16)
        out["cpu_baseline"] = _cpu_repeat(lambda: ko.lib().ko_baseline_permute_bhsd_bshd16(hx.ctypes.data, hy.ctypes.data, b, h, s, d), nbytes, 1e9, "GB/s",
                                          "the whole permute, 256-byte rows moved whole")
    return out


# ---------------------------------------------------------------- GEMMs
def _blocks_frobenius(ko, got, go_a, go_b, M, N, K, out_dtype, count, blk=64, scales=None):
    """Relative Frobenius error of `count` blk x blk blocks of the result against the fp64-accumulated checker."""
    import numpy as np
    num = den = 0.0
    for t in range(count):
        r0 = 0 if M <= blk else (t * (M // count) + 29 * t) % (M - blk)
        c0 = 0 if N <= blk else ((count - 1 - t) * (N // count) + 71 * t) % (N - blk)
        bm, bn = min(blk, M), min(blk, N)
        want = np.zeros((bm, bn), dtype=np.uint16)
        ga, gb, gw = ko.sv_global(go_a, r0, r0 + bm, 0, K), ko.sv_global(go_b, 0, K, c0, c0 + bn), ko.mk_global(want, bm, bn, bn, 1, out_dtype)
        if scales is None:
            assert ko.lib().ko_matmul(C.byref(ga), C.byref(gb), None, C.byref(gw), ko.RN) == 0
        else:
            rs, cs = np.ascontiguousarray(scales[0][r0:r0 + bm]), np.ascontiguousarray(scales[1][c0:c0 + bn])
            assert ko.lib().ko_matmul_scaled_f8(C.byref(ga), C.byref(gb), rs.ctypes.data, cs.ctypes.data, C.byref(gw)) == 0
        g, w = ko.decode(got[r0:r0 + bm, c0:c0 + bn], out_dtype), ko.decode(want, out_dtype)
        if not np.all(np.isfinite(g)):
            return float("inf")
        num += ((g - w) ** 2).sum()
        den += (w ** 2).sum()
    return float(np.sqrt(num / max(den, 1e-300)))


def _whole_frobenius(ko, got, go_a, go_b, M, N, K, out_dtype, scales=None, blocks=16):
    """Relative Frobenius error of the WHOLE result against the host GEMM of oracle/kapy_baseline.cpp (fp32 over K blocks of 512,
    the blocks summed in fp64, rounded once), and that host result's own error on `blocks` 64 x 64 blocks against the
    fp64-accumulated checker, which ties the fast host GEMM to the exact one.  Outside every timed region."""
    import numpy as np
    want = np.zeros((M, N), np.uint16)
    gw = ko.mk_global(want, M, N, N, 1, out_dtype)
    rs = scales[0].ctypes.data if scales else None
    cs = scales[1].ctypes.data if scales else None
    assert ko.lib().ko_baseline_gemm(C.byref(go_a), C.byref(go_b), rs, cs, C.byref(gw), None) == 0
    host_rel = _blocks_frobenius(ko, want, go_a, go_b, M, N, K, out_dtype, blocks, scales=scales)
    num = den = 0.0
    for r0 in range(0, M, 512):    # in slabs: the fp64 images of a 8192 x 8192 result would take 1 GiB
        g, w = ko.decode(got[r0:r0 + 512], out_dtype), ko.decode(want[r0:r0 + 512], out_dtype)
        if not np.all(np.isfinite(g)):
            return float("inf"), host_rel
        num += float(((g - w) ** 2).sum())
        den += float((w ** 2).sum())
    return float(np.sqrt(num / max(den, 1e-300))), host_rel


def _cpu_gemm(ko, go_a, go_b, go_d, rows, N, K, scales, what):
    """The packed, register-blocked fp32 GEMM of oracle/kapy_baseline.cpp on the first `rows` rows of the lhs."""
    import numpy as np
    secs = C.c_double(0.0)
    a, d = ko.sv_global(go_a, 0, rows, 0, K), ko.sv_global(go_d, 0, rows, 0, N)
    rs = scales[0].ctypes.data if scales else None
    cs = scales[1].ctypes.data if scales else None
    tot, reps, t0 = 0.0, 0, time.perf_counter()
    while True:
        assert ko.lib().ko_baseline_gemm(C.byref(a), C.byref(go_b), rs, cs, C.byref(d), C.byref(secs)) == 0
        tot += secs.value
        reps += 1
        if time.perf_counter() - t0 > CPU_SECONDS:
            break
    return {"value": round(2.0 * rows * N * K * reps / tot / 1e12, 4), "unit": "TFLOP/s", "cores": ko.lib().ko_num_threads(), "kind": "port",
            "sample": "%s; fp32 accumulate, operands widened to fp32 and packed outside the timed multiply; %d repetitions, %.2f s of multiplying" % (what, reps, tot)}


def bench_gemm(kh, steps, warmup, cpu, M, N, K, dtype, b_col_major, name, kernel, tile=(0, 0, 0), graph_of=0, fused_gelu=False, gen="normal", key=None, workspace=False, whole=True, a_col_major=False):
    """whole: gate the whole result against the host GEMM as well as 16 blocks against the fp64 checker (a second and third large
    problem of the same shape are gated on the blocks alone: the host GEMM takes its time).
    graph_of > 0: that many back-to-back launches recorded once into a HIP graph; a step is one replay, figures are per launch
    (what a launch-bound shape gains when the host's per-launch cost is taken out).
    fused_gelu: d = gelu_tanh(a.b*0.5 + bias) with the tail in the GEMM's epilogue (kapy_matmul_fused); flops counted are the GEMM's.
    gen: "normal" = normal(0, 0.02) seeds 0 / 1 (C4), "uniform" = uniform[-1,1) seed 0 streams 0 / 1 (C1).
    workspace: hand the library a workspace, which lets it split K across workgroups when the tiles alone would not fill the device,
    or turn a large row-major rhs K-contiguous before multiplying."""
    import numpy as np
    import torch
    import ko
    if gen == "uniform":
        ha, hb = _host("uniform", M * K, dtype, 0, 0), _host("uniform", K * N, dtype, 0, 1)
        a, b = _dev("uniform", M * K, dtype, 0, 0), _dev("uniform", K * N, dtype, 0, 1)
        what = "A, B uniform[-1,1) seed 0 (streams 0, 1)"
    else:
        ha, hb = _host("normal", M * K, dtype, 0, 0, std=0.02), _host("normal", K * N, dtype, 1, 0, std=0.02)
        a, b = _dev("normal", M * K, dtype, 0, 0, std=0.02), _dev("normal", K * N, dtype, 1, 0, std=0.02)
        what = "A normal(0,0.02) seed 0, B normal(0,0.02) seed 1"
    d = torch.empty(M * N, device="cuda", dtype=torch.int16)
    b_str = (1, K) if b_col_major else (N, 1)
    a_str = (1, M) if a_col_major else (K, 1)
    ga = kh.mk_global(a.data_ptr(), M, K, a_str[0], a_str[1], dtype)
    gb = kh.mk_global(b.data_ptr(), K, N, b_str[0], b_str[1], dtype)
    gd = kh.mk_global(d.data_ptr(), M, N, N, 1, dtype)
    go_a, go_b = ko.mk_global(ha, M, K, a_str[0], a_str[1], dtype), ko.mk_global(hb, K, N, b_str[0], b_str[1], dtype)
    if fused_gelu:
        hbias = _host("normal", N, dtype, 2)
        bias = _dev("normal", N, dtype, 2)
        gbias = kh.mk_global(bias.data_ptr(), 1, N, N, 1, dtype)
        run = lambda i: kh.matmul_fused(ga, gb, gd, bias=gbias, alpha=0.5, act=kh.EW_GELU_TANH, tile=tile)
    else:
        ws_bytes = max(kh.lib().kapy_matmul_workspace_bytes(M, N), kh.lib().kapy_matmul_turn_workspace_bytes(ga, gb))
        ws = torch.zeros(ws_bytes, dtype=torch.uint8, device="cuda") if workspace else None
        run = lambda i: kh.matmul(ga, gb, gd, tile=tile, workspace=ws)
    run(0)
    torch.cuda.synchronize()
    got = _download(d, np.uint16, (M, N))
    host_rel = None
    if fused_gelu:
        # gate: blocks of gelu(c*0.5 + bias) recomputed in fp64 from the checker's fp32-result GEMM of the same blocks
        num = den = 0.0
        for t in range(8):
            r0, c0 = (t * (M // 8) + 29 * t) % (M - 64), ((7 - t) * (N // 8) + 71 * t) % (N - 64)
            c32 = np.zeros((64, 64), np.float32)
            assert ko.lib().ko_matmul(C.byref(ko.sv_global(go_a, r0, r0 + 64, 0, K)), C.byref(ko.sv_global(go_b, 0, K, c0, c0 + 64)), None,
                                      C.byref(ko.mk_global(c32, 64, 64, 64, 1, ko.F32)), ko.RN) == 0
            v = c32.astype(np.float64) * 0.5 + ko.decode(hbias[c0:c0 + 64], dtype)[None, :]
            w = 0.5 * v * (1.0 + np.tanh(0.7978845608028654 * (v + 0.044715 * v ** 3)))
            g = ko.decode(got[r0:r0 + 64, c0:c0 + 64], dtype)
            num += ((g - w) ** 2).sum()
            den += (w ** 2).sum()
        rel, n_blocks = float(np.sqrt(num / den)), 8
        tol = 4e-3   # the bf16 result itself rounds at 2^-9 relative
    else:
        n_blocks = 16 if M * N > 1024 * 1024 else 0
        if n_blocks:
            rel = _blocks_frobenius(ko, got, go_a, go_b, M, N, K, dtype, n_blocks)
            if whole:
                whole_rel, host_rel = _whole_frobenius(ko, got, go_a, go_b, M, N, K, dtype)
                if not host_rel <= FROB_TOL:
                    raise CheckFailed("%s: the host GEMM itself is off the fp64 checker by %g" % (name, host_rel))
                rel = max(rel, whole_rel)
        else:   # small enough for the whole result
            want = np.zeros((M, N), np.uint16)
            assert ko.lib().ko_matmul(C.byref(go_a), C.byref(go_b), None, C.byref(ko.mk_global(want, M, N, N, 1, dtype)), ko.RN) == 0
            g, w = ko.decode(got, dtype), ko.decode(want, dtype)
            rel = float(np.linalg.norm(g - w) / np.linalg.norm(w)) if np.all(np.isfinite(g)) else float("inf")
        tol = FROB_TOL
    if not rel <= tol:
        raise CheckFailed("%s: relative Frobenius error %g" % (name, rel))
    if graph_of:
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            for _ in range(graph_of):
                run(0)
        wall, ev = _events(lambda i: graph.replay(), steps, warmup)
        wall, ev = wall / graph_of, ev / graph_of
    else:
        wall, ev = _events(run, steps, warmup)
    flops = 2.0 * M * N * K
    kind = "bf16" if dtype == kh.BF16 else "f16"
    out = {"workload": name, "value": flops / (wall * 1e-3) / 1e12, "unit": "TFLOP/s", "ms_per_step": wall, "kernel_ms": ev,
           "dtype": kind, "roofline": _roof_mfma(flops, ev, kind, key), "kernel": kernel, "inputs": what + " (host-generated, as the configuration states)",
           "checked": True, "check": "%s: relative Frobenius error %.2e (tolerance %.0e)" %
                                     ("the whole timed result against the host GEMM (fp64 sums of fp32 K blocks; itself %.1e off the fp64-accumulated checker on 16 blocks) "
                                      "and %d 64x64 blocks of it against the fp64-accumulated checker, the larger of the two" % (host_rel, n_blocks) if host_rel is not None else
                                      "%d 64x64 blocks of the timed result against the fp64 checker" % n_blocks if n_blocks else "the whole timed result against the fp64-accumulated checker", rel, tol)}
    if cpu and not graph_of and not fused_gelu:
        rows = min(M, 1024)
        hd = np.zeros(M * N, np.uint16)
        out["cpu_baseline"] = _cpu_gemm(ko, go_a, go_b, ko.mk_global(hd, M, N, N, 1, dtype), rows, N, K, None,
                                        "the first %d of %d rows of the result (all of N and K)" % (rows, M) if rows < M else "the whole workload")
    return out


_f8_cache = {}


def _f8_operands(ko, M, N, K):
    """C5: pre-quantisation values normal(0,1) fp32 (A seed 0, W seed 1, W stored K-contiguous per output column),
    per-row / per-column scales amax/448, values rounded once (RN-even, saturating) to e4m3."""
    import numpy as np
    vp = lambda x: x.ctypes.data_as(C.c_void_p)
    if ("w", N, K) not in _f8_cache:
        w = ko.fill_normal(N * K, ko.F32, 1, 0).reshape(N, K)
        wq, sb = np.zeros((N, K), np.uint8), np.zeros(N, np.float32)
        ko.lib().ko_quantize_e4m3(vp(w), N, K, K, 1, 1, vp(wq), vp(sb))
        _f8_cache[("w", N, K)] = (wq, sb)
    a = ko.fill_normal(M * K, ko.F32, 0, 0).reshape(M, K)
    aq, sa = np.zeros((M, K), np.uint8), np.zeros(M, np.float32)
    ko.lib().ko_quantize_e4m3(vp(a), M, K, K, 1, 1, vp(aq), vp(sa))
    wq, sb = _f8_cache[("w", N, K)]
    return aq, sa, wq, sb


def bench_f8(kh, steps, warmup, cpu, M, workspace=False):
    import numpy as np
    import torch
    import ko
    N = K = 8192
    aq, sa, wq, sb = _f8_operands(ko, M, N, K)
    a, dsa, dsb = _upload(aq), _upload(sa), _upload(sb)
    if ("wdev", N, K) not in _dev_cache:
        _dev_cache[("wdev", N, K)] = _upload(wq)
    w0 = _dev_cache[("wdev", N, K)]
    sets = 6 if M <= 512 else 1                # few rows: weight-streaming: 6 x 64 MiB > Infinity Cache (copies of the same weight)
    ws = [w0] + [w0.clone() for _ in range(sets - 1)]
    d = torch.empty(M * N, device="cuda", dtype=torch.int16)
    ga = kh.mk_global(a.data_ptr(), M, K, K, 1, kh.F8E4M3)
    gws = [kh.mk_global(w.data_ptr(), K, N, 1, K, kh.F8E4M3) for w in ws]
    gd = kh.mk_global(d.data_ptr(), M, N, N, 1, kh.BF16)
    ws = torch.zeros(kh.lib().kapy_matmul_workspace_bytes(M, N), dtype=torch.uint8, device="cuda") if workspace else None
    kh.matmul_scaled_f8(ga, gws[0], dsa.data_ptr(), dsb.data_ptr(), gd, workspace=ws)
    torch.cuda.synchronize()
    got = _download(d, np.uint16, (M, N))
    go_a, go_w = ko.mk_global(aq, M, K, K, 1, ko.F8E4M3), ko.mk_global(wq, K, N, 1, K, ko.F8E4M3)
    n_blocks = 16
    rel = _blocks_frobenius(ko, got, go_a, go_w, M, N, K, ko.BF16, n_blocks, scales=(sa, sb))
    whole = "%d %dx64 blocks of the timed result against the fp64-accumulated checker" % (n_blocks, min(M, 64))
    if M >= 1024:   # the whole result as well, against the host GEMM
        wrel, host_rel = _whole_frobenius(ko, got, go_a, go_w, M, N, K, ko.BF16, scales=(sa, sb))
        if not host_rel <= FROB_TOL:
            raise CheckFailed("f8 M=%d: the host GEMM itself is off the fp64 checker by %g" % (M, host_rel))
        rel = max(rel, wrel)
        whole = "the whole timed result against the host GEMM (fp64 sums of fp32 K blocks; itself %.1e off the fp64-accumulated checker on 16 blocks) and %s, the larger of the two" % (host_rel, whole)
    if not rel <= FROB_TOL:
        raise CheckFailed("f8 M=%d: relative Frobenius error %g" % (M, rel))
    wall, ev = _events(lambda i: kh.matmul_scaled_f8(ga, gws[i % sets], dsa.data_ptr(), dsb.data_ptr(), gd, workspace=ws), steps, warmup)
    flops = 2.0 * M * N * K
    nbytes = M * K + N * K + M * N * 2 + (M + N) * 4
    out = {"workload": "C5 W8A8 e4m3 M=%d N=K=8192%s" % (M, ", K split across workgroups (workspace given)" if workspace else ""), "value": flops / (wall * 1e-3) / 1e12, "unit": "TFLOP/s",
           "ms_per_step": wall, "kernel_ms": ev, "dtype": "f8e4m3", "kernel": "skinny_stream_kernel" if M <= 16 else "skinny_block_kernel" if (M <= 64 or (M <= 128 and not workspace)) else "tn_kernel<F8M16, 128x128x128> split K" if (workspace and M <= 128) else "tn_kernel<F8, 128x128x128, four stages>" if M <= 512 else "tn_kernel<F8>",
           "inputs": "normal(0,1) fp32 (A seed 0, W seed 1) quantised to e4m3 with per-row / per-column scales amax/448 (as the configuration states)",
           "checked": True, "check": "%s: relative Frobenius error %.2e (tolerance %.0e)" % (whole, rel, FROB_TOL)}
    out["roofline"] = _roof_hbm(nbytes, ev, "f8_m%d%s" % (M, "_splitk" if workspace else "")) if M <= 512 else _roof_mfma(flops, ev, "f8", "f8_m%d" % M)
    if cpu:
        rows = min(M, 1024)
        hd = np.zeros(M * N, np.uint16)
        out["cpu_baseline"] = _cpu_gemm(ko, go_a, go_w, ko.mk_global(hd, M, N, N, 1, ko.BF16), rows, N, K, (sa, sb),
                                        "the first %d of %d rows of the result (all of N and K)" % (rows, M) if rows < M else "the whole workload")
    return out


def bench_mlir(kh, steps, warmup, cpu):
    """The reference's three fixture programs (elementwise add, row sum, matmul; test/Conversion/KapyToKgpu/*.mlir) in the op syntax of
    kapy_programs.py, run through kapy_run_mlir on grids of program instances: per program the time of one call with the
    instances' stores merged into one call each and with one instance at a time (KAPY_MLIR_BATCH=0), both parsed and
    interpreted at every call (KAPY_MLIR_PLAN=0), and as the default does it: the device calls of the first run kept and made
    again.  A call synchronises its stream: the figures are those of a validation path."""
    import numpy as np
    import torch
    import ko
    import kapy_programs as kp
    out = {"workload": "the reference's three fixture programs through kapy_run_mlir", "unit": "GB/s", "dtype": "f16", "kernel": "one call per kapy.st_global over all instances (elementwise, reduce); in a replayed run also one launch per copy / product of the matmul program over all instances (copy_table_kernel, matmul_table_kernel)",
           "inputs": "normal(0,1) seeded, fp16", "programs": {}}
    rows_per_warp, cols, warps, programs = 4, 1024, 4, 256
    rows = rows_per_warp * warps * programs
    x, y = _dev("normal", rows * cols, ko.F16, 11), _dev("normal", rows * cols, ko.F16, 12)
    d = torch.empty(rows * cols, device="cuda", dtype=torch.int16)
    # (name, program text, arguments, grid, the tensor the program writes, algorithmic bytes or None)
    cases = [("x + y [%d x %d], %d programs x %d warps" % (rows, cols, programs, warps), kp.binary_program("arith.addf", rows_per_warp, cols, warps), [x, y, d, rows], [programs], d, 3 * rows * cols * 2),
             ("row sums [%d x %d], %d programs x %d warps" % (rows, cols, programs, warps), kp.reduce_program("arith.addf", rows_per_warp, cols, warps), [x, d, rows], [programs], d, rows * cols * 2 + rows * 2)]
    M, N, K = 512, 512, 256
    a, b = _dev("normal", M * K, ko.F16, 31, std=0.5), _dev("normal", K * N, ko.F16, 32, std=0.5)
    c = torch.empty(M * N, device="cuda", dtype=torch.int16)
    cases.append(("matmul %d x %d x %d, 64 x 64 x 16 per warp, f16 accumulator" % (M, N, K), kp.matmul_program(64, 64, 16, "mma_m16n8k8_f16", "f16"), [a, b, c, M, N, K], [(M // 128) * (N // 128)], c, None))
    checked = True
    for name, text, args, grid, target, nbytes in cases:
        row = {}
        results = []
        for label, env, plan in (("instances merged", "1", "0"), ("one instance at a time", "0", "0"), ("instances merged, calls replayed", "1", "1")):
            os.environ["KAPY_MLIR_BATCH"] = env
            os.environ["KAPY_MLIR_PLAN"] = plan
            target.zero_()
            before = kh.run_mlir_stats()
            kh.run_mlir(text, args, grid)
            torch.cuda.synchronize()
            row[label + ", merged stores per call"] = kh.run_mlir_stats() - before
            if plan == "1":                      # the result compared is that of a replayed call
                target.zero_()
                kh.run_mlir(text, args, grid)
                torch.cuda.synchronize()
            results.append(target.clone())
            kh.run_mlir(text, args, grid)        # (a chain that comes back is compiled at its second call: not in the timed ones)
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            reps = 3 if plan == "0" else 10
            for _ in range(reps):
                kh.run_mlir(text, args, grid)
            torch.cuda.synchronize()
            ms = (time.perf_counter() - t0) * 1e3 / reps
            row[label + ", ms per call"] = round(ms, 3)
            if nbytes:
                row[label + ", GB/s"] = round(nbytes / (ms * 1e-3) / 1e9, 2)
        os.environ.pop("KAPY_MLIR_BATCH", None)
        os.environ.pop("KAPY_MLIR_PLAN", None)
        if not (torch.equal(results[0], results[1]) and torch.equal(results[0], results[2])):
            checked = False
        out["programs"][name] = row
    if not checked:
        raise CheckFailed("run_mlir: merged, per-instance and replayed runs differ")
    first = out["programs"][cases[0][0]]
    key = "instances merged, calls replayed"
    out.update({"value": first[key + ", GB/s"], "ms_per_step": first[key + ", ms per call"], "kernel_ms": first[key + ", ms per call"],
                "checked": True, "check": "merged, per-instance and replayed runs give the same bits (the programs themselves are compared with the checker in the GPU tests)",
                "roofline": _roof_hbm(cases[0][5], first[key + ", ms per call"], None)})
    return out


def bench_ceilings(kh, steps, warmup, cpu):
    """What this device sustains, from the library's own probe kernels: a loop of nothing but matrix instructions per
    instruction shape (operands of the benchmark's distribution; the part is power-limited, so this, not the data-sheet
    figure, is what a GEMM can approach) with the shader clock it holds, and a plain 16-byte-per-lane copy of 2 x 128 MiB
    in every form a memory-bound kernel could take (vectors per lane, non-temporal or not, one pass or persistent)."""
    import numpy as np
    import torch
    import ko
    import kapy_probe as kp
    out = {"workload": "device ceilings (the probe library's kernels)", "checked": True, "check": "nothing to check: measurement only", "mfma": {}, "copy": {}}
    sink = torch.empty(1024 * 256, device="cuda", dtype=torch.float32)
    ticks = torch.zeros(4 * 1024, device="cuda", dtype=torch.int64)
    for name, way, dt, gen, peak in (("bf16 16x16x32", kh.MFMA_16X16X32_16B, kh.BF16, "normal002", 2500.0), ("bf16 32x32x16", kh.MFMA_32X32X16_16B, kh.BF16, "normal002", 2500.0),
                                     ("f16 16x16x32", kh.MFMA_16X16X32_16B, kh.F16, "uniform", 2500.0), ("e4m3 16x16x128", kh.MFMA_16X16X128_F8, kh.F8E4M3, "quant", 5000.0),
                                     ("e4m3 32x32x64", kh.MFMA_32X32X64_F8, kh.F8E4M3, "quant", 5000.0)):
        n = 131072 // kh.DTYPE_BYTES[dt]
        if gen == "normal002":
            ops = _upload(ko.fill_normal(n, dt, 0, 0, 0.0, 0.02))
        elif gen == "uniform":
            ops = _upload(ko.fill_uniform(n, dt, 0, 0))
        else:   # e4m3 values as the W8A8 quantiser leaves them: normal(0,1) scaled so that the largest of 8192 is 448
            x = ko.fill_normal(n, ko.F32, 0, 0).reshape(-1, 8192)
            q, sc = np.zeros(x.shape, np.uint8), np.zeros(x.shape[0], np.float32)
            ko.lib().ko_quantize_e4m3(x.ctypes.data, x.shape[0], x.shape[1], x.shape[1], 1, 1, q.ctypes.data, sc.ctypes.data)
            ops = _upload(q)
        iters = 2000
        wgs, flops = kp.probe_mfma(way, dt, ops.data_ptr(), iters, sink.data_ptr())
        wall, ev = _events(lambda i: kp.probe_mfma(way, dt, ops.data_ptr(), iters, sink.data_ptr(), ticks.data_ptr()), max(steps // 2, 5), warmup)
        torch.cuda.synchronize()
        t = ticks.cpu().numpy()[:4 * wgs].reshape(wgs, 4).astype(np.float64)
        ghz = float(np.median((t[:, 1] - t[:, 0]) / np.maximum(t[:, 3] - t[:, 2], 1.0)) * 0.1)    # shader ticks per 100 MHz tick
        tf = flops / (ev * 1e-3) / 1e12
        out["mfma"][name] = {"tflops": round(tf, 1), "frac_of_peak": round(tf / peak, 4), "shader_clock_ghz": round(ghz, 3), "kernel_ms": round(ev, 4)}
    nbytes, sets = 128 << 20, 4
    src = [_dev("bits16", nbytes // 2, ko.F16, 0, k) for k in range(sets)]
    dst = [torch.empty(nbytes // 2, device="cuda", dtype=torch.int16) for _ in range(sets)]
    kp.probe_copy(src[0].data_ptr(), dst[0].data_ptr(), nbytes)
    torch.cuda.synchronize()
    if not torch.equal(src[0], dst[0]):
        raise CheckFailed("probe_copy: result differs from the source")
    best = 0.0
    for u in (1, 2, 4, 8, 16):
        for ntl, nts in ((0, 0), (1, 0), (0, 1), (1, 1)):
            for pers in (0, 4, 8, 16):
                if pers and u > 8:
                    continue
                wall, ev = _events(lambda i: kp.probe_copy(src[i % sets].data_ptr(), dst[i % sets].data_ptr(), nbytes, u, ntl, nts, pers), 20, 3)
                gbs = 2 * nbytes / (ev * 1e-3) / 1e9
                best = max(best, gbs)
                out["copy"]["vec%d ntld%d ntst%d %s" % (u, ntl, nts, "persistent x%d" % pers if pers else "one pass")] = round(gbs, 0)
    # the same bytes with the access footprint of the 16-bit tile transpose (four 256-byte pieces of four rows per wave
    # instruction instead of one contiguous KiB), untransposed: what the transposes can reach
    n = 8192
    for lds in (0, 1):
        kp.probe_copy_tiled(src[0].data_ptr(), dst[0].data_ptr(), n, n * 2, lds)
        torch.cuda.synchronize()
        if not torch.equal(src[0], dst[0]):
            raise CheckFailed("probe_copy_tiled: result differs from the source")
        wall, ev = _events(lambda i: kp.probe_copy_tiled(src[i % sets].data_ptr(), dst[i % sets].data_ptr(), n, n * 2, lds), 40, 5)
        out["copy"]["transpose footprint (128 rows x 256 B per workgroup)%s" % (", through LDS and a barrier" if lds else "")] = round(2 * nbytes / (ev * 1e-3) / 1e9, 0)
    # ... and by the length of the contiguous runs alone (a transposing kernel's runs are as long as its tile is wide)
    for run in (256, 512, 1024, 2048, 4096):
        kp.probe_copy_runs(src[0].data_ptr(), dst[0].data_ptr(), n, n * 2, run)
        torch.cuda.synchronize()
        if not torch.equal(src[0], dst[0]):
            raise CheckFailed("probe_copy_runs: result differs from the source")
        wall, ev = _events(lambda i: kp.probe_copy_runs(src[i % sets].data_ptr(), dst[i % sets].data_ptr(), n, n * 2, run), 40, 5)
        out["copy"]["runs of %d B (%d rows x %d B per workgroup)" % (run, 32768 // run, run)] = round(2 * nbytes / (ev * 1e-3) / 1e9, 0)
    # a read-only stream (the weight matrix of a skinny GEMM, the operand of a reduce): 64 MiB buffers in rotation
    out["read"] = {}
    rsink = torch.zeros(1 << 20, dtype=torch.int32, device="cuda")
    rbytes, best_read = 64 << 20, 0.0
    for u in (1, 2, 4, 8):
        for ntl in (0, 1):
            for pers in (0, 4, 8):
                wall, ev = _events(lambda i: kp.probe_read(src[i % sets].data_ptr() + (i // sets % 2) * rbytes, rbytes, u, ntl, pers, rsink.data_ptr()), 24, 4)
                gbs = rbytes / (ev * 1e-3) / 1e9
                best_read = max(best_read, gbs)
                out["read"]["vec%d ntld%d %s" % (u, ntl, "persistent x%d" % pers if pers else "one pass")] = round(gbs, 0)
    out["read_best_gbs"] = round(best_read, 0)
    out["read_best_frac_of_peak"] = round(best_read / HBM_PEAK_GBS, 4)
    out["copy_best_gbs"] = round(best, 0)
    out["copy_best_frac_of_peak"] = round(best / HBM_PEAK_GBS, 4)
    # what the L2s hand to the CUs: every CU re-reads a window that stays in its XCD's L2 (2 MiB), that spills to the Infinity
    # Cache (8 MiB per XCD) or to HBM (64 MiB per XCD), as LDS-direct loads (the tiled matmuls' form) or into registers
    out["l2_read_tbs"] = {}
    sink = torch.zeros(4096, dtype=torch.int32, device="cuda")
    for window in (2 << 20, 8 << 20, 64 << 20):
        buf = torch.empty(8 * window, dtype=torch.uint8, device="cuda")
        buf.random_(0, 255)
        for to_lds in (True, False):
            _, nb = kp.probe_l2_read(buf.data_ptr(), window, 512, 1, to_lds, sink.data_ptr())
            wall, ev = _events(lambda i: kp.probe_l2_read(buf.data_ptr(), window, 512, 1, to_lds, sink.data_ptr()), 10, 3)
            out["l2_read_tbs"]["%d MiB per XCD, %s" % (window >> 20, "LDS-direct" if to_lds else "to registers")] = round(nb / (ev * 1e-3) / 1e12, 2)
        del buf
    # what a wave can issue beside its matrix instructions (one wave per SIMD, as in the tiled matmuls): fillers in the gap
    # behind every instruction, and the reads and loads of the matmuls' steady-state loop on L2-resident data
    out["issue_tflops"] = {}
    fsink = torch.empty(1024 * 256, device="cuda", dtype=torch.float32)
    window = torch.empty(8 * (2 << 20), dtype=torch.uint8, device="cuda")
    window.random_(0, 120)
    for name, way, fills in (("bf16 16x16x32", kh.MFMA_16X16X32_16B, ((0, 0), (1, 3), (1, 4), (1, 6), (2, 1), (2, 2), (2, 3), (3, 0), (4, 0))),
                             ("e4m3 16x16x128", kh.MFMA_16X16X128_F8, ((0, 0), (1, 6), (1, 8), (2, 2), (2, 3), (2, 4), (3, 0), (4, 0)))):
        row = {}
        for filler, count in fills:
            _, flops = kp.probe_issue(way, filler, count, window.data_ptr(), 2000, fsink.data_ptr())
            wall, ev = _events(lambda i: kp.probe_issue(way, filler, count, window.data_ptr(), 2000, fsink.data_ptr()), 6, 3)
            label = ("nothing", "%d scalar" % count, "%d vector ALU" % count, "matmul loop: 32 LDS reads + 16 LDS-direct loads per tile",
                     "rhs off the LDS: 16 LDS reads + 8 LDS-direct loads + 16 register loads per tile")[filler]
            row[label] = round(flops / (ev * 1e-3) / 1e12, 1)
        out["issue_tflops"][name] = row
    del window
    # the tiled matmuls' cost per launch that does not grow with K (epilogues, prologues, launch), and the rate beyond it:
    # the C4 / C5 shapes at K and 2K
    out["gemm_fixed_cost"] = {}
    for name, m, n, k, f8 in (("C4 bf16 8192 x 8192", 8192, 8192, 4096, False), ("C5 e4m3 4096 x 8192", 4096, 8192, 8192, True)):
        times = []
        for kk in (k, 2 * k):
            if f8:
                a = torch.randn(m, kk, device="cuda").mul_(100.0).to(torch.float8_e4m3fn).view(torch.uint8)
                w = torch.randn(n, kk, device="cuda").mul_(100.0).to(torch.float8_e4m3fn).view(torch.uint8)
                sa, sb = torch.rand(m, device="cuda") * 0.01 + 0.001, torch.rand(n, device="cuda") * 0.01 + 0.001
                d = torch.empty(m, n, device="cuda", dtype=torch.bfloat16)
                ga, gw, gd = kh.mk_global(a.data_ptr(), m, kk, kk, 1, kh.F8E4M3), kh.mk_global(w.data_ptr(), kk, n, 1, kk, kh.F8E4M3), kh.mk_global(d.data_ptr(), m, n, n, 1, kh.BF16)
                fn = lambda i: kh.matmul_scaled_f8(ga, gw, sa.data_ptr(), sb.data_ptr(), gd)
            else:
                a = torch.randn(m, kk, device="cuda", dtype=torch.bfloat16)
                w = torch.randn(n, kk, device="cuda", dtype=torch.bfloat16)
                d = torch.empty(m, n, device="cuda", dtype=torch.bfloat16)
                ga, gw, gd = kh.mk_global(a.data_ptr(), m, kk, kk, 1, kh.BF16), kh.mk_global(w.data_ptr(), kk, n, 1, kk, kh.BF16), kh.mk_global(d.data_ptr(), m, n, n, 1, kh.BF16)
                fn = lambda i: kh.matmul(ga, gw, gd)
            wall, ev = _events(fn, 30, 10)
            times.append(ev * 1e3)
            del a, w, d
        per_k = (times[1] - times[0]) / k   # us per K element beyond the fixed cost
        out["gemm_fixed_cost"][name] = {"us_at_K=%d" % k: round(times[0], 1), "us_at_K=%d" % (2 * k): round(times[1], 1), "fixed_us": round(times[0] - per_k * k, 1),
                                        "marginal_tflops": round(2.0 * m * n / per_k / 1e6, 1)}
    return out


WORKLOADS = ["gelu", "add", "expr", "expr_compiled", "swiglu", "copy", "reduce", "reduce_cols", "softmax", "softmax_cols", "causal_softmax", "layernorm", "l2norm_compiled", "gelu_transposed",
             "transpose", "permute", "gemm_bf16", "gemm_bf16_gelu", "gemm_bf16_nn", "gemm_bf16_nn_turned", "gemm_bf16_m128", "gemm_f16", "gemm_f16_splitk", "gemm_f16_graph", "f8_m16", "f8_m64", "f8_m128", "f8_m128_splitk", "f8_m256", "f8_m4096", "mlir_fixtures", "ceilings"]


# ---------------------------------------------------------------- HBM traffic summary from the profiler's counter files
# Which kernels' dispatches are one launch of which workload: (workload key, label, [(kernel-name pattern, grid size or None)]);
# the bytes of the listed kernels add up (a workload of two kernels launches each once per step).
TRAFFIC_KERNELS = [
    ("copy", "copy 2 x 128 MiB", [(r"rows_kernel<", None)]),           # (first: the calibration kernel)
    ("permute", "C3b permute", [(r"rows_kernel<", None)]),
    ("gelu", "C2 gelu fp16 8192^2", [(r"affine_act_cols_kernel", None)]),
    ("add", "x + y fp16 8192^2", [(r"affine_act_kernel", None)]),
    # the compiled kernels are named after a hash of their program and operand signature (a changed program shows up here as
    # "kernel not seen")
    ("expr", "x*y + x fp16 8192^2 (compiled from its second call)", [(r"kapy_ew_flat_4fe8d22e", None)]),
    ("expr_compiled", "x*y + x fp16 8192^2, compiled", [(r"kapy_ew_flat_4fe8d22e", None)]),
    ("swiglu", "silu(x)*y fp16 8192^2, compiled", [(r"kapy_ew_flat_3c2da24d", None)]),
    ("gelu_transposed", "gelu(x^T*0.5 + bias), compiled", [(r"kapy_ew_flat_b65a1568", None)]),
    ("l2norm_compiled", "x*rsqrt(sum x^2), compiled", [(r"kapy_ew_rows_7416033f", None)]),
    ("causal_softmax", "causal-masked softmax, compiled", [(r"kapy_ew_rows_575adad9", None)]),
    ("transpose", "C3a transpose fp16 8192^2", [(r"transpose_lds_kernel<", None)]),
    ("reduce", "row sums fp16 8192^2", [(r"reduce_rows_vec_kernel<", None)]),
    ("reduce_cols", "column sums fp16 8192^2", [(r"reduce_cols_strip_kernel<", None)]),
    ("softmax_cols", "column softmax fp16 8192^2", [(r"col_softmax_stats_kernel<", None), (r"col_softmax_apply_kernel<", None)]),
    ("softmax", "row softmax fp16 8192^2", [(r"softmax_kernel<", None)]),
    ("layernorm", "layer norm fp16 8192^2", [(r"norm_kernel<", None)]),
    ("gemm_bf16", "C4 gemm bf16 8192^3", [(r"tn_kernel<kapy::Bf16M16, 256, 256, 64, .*, false>[(]", None)]),
    ("gemm_bf16_gelu", "C4 gemm bf16 8192^3 + gelu", [(r"tn_kernel<kapy::Bf16M16, 256, 256, 64, .*, true>[(]", None)]),
    ("gemm_bf16_nn", "gemm bf16 8192^3, both operands row-major", [(r"nn256_kernel<kapy::Bf16M16", None)]),
    ("f8_m4096", "C5 W8A8 M=4096", [(r"tn_kernel<kapy::F8M16<0, 0>, 256, 256, 128", None)]),
    ("f8_m16", "C5 W8A8 M=16", [(r"skinny_stream_kernel<", None)]),
    ("f8_m64", "W8A8 M=64", [(r"skinny_block_kernel<0, 0, 4>", None)]),
    ("f8_m128", "W8A8 M=128", [(r"skinny_block_kernel<0, 0, 8>", None)]),
    ("f8_m128_splitk", "W8A8 M=128, K split over workgroups", [(r"tn_kernel<kapy::F8M16<0, 0>, 128, 128, 128", None)]),
    ("f8_m256", "W8A8 M=256", [(r"tn_kernel<kapy::F8<0, 0>, 128, 128, 128, 2, 2, 4", None)]),
    ("gemm_f16", "C1 gemm fp16 1024^3", [(r"nn_kernel<kapy::F16M16", 64 * 256)]),
    ("gemm_f16_graph", "C1 gemm fp16 1024^3, replayed from a graph", [(r"nn_kernel<kapy::F16M16", 64 * 256)]),
    ("gemm_f16_splitk", "C1 gemm fp16 1024^3, K split two ways", [(r"nn_kernel<kapy::F16M16", 128 * 256)]),
]


def pmc_summary(fetch_csv, write_csv):
    """The tracked HBM-traffic summary from two rocprofv3 counter files (FETCH_SIZE and WRITE_SIZE, KiB per dispatch): per kernel and
    grid the mean of each counter, the factor that makes the plain copy's counters read its known 128 MiB each way, and one line
    `traffic_bytes <workload> <bytes>` per workload of TRAFFIC_KERNELS, which is what the benchmark reports as `traffic`."""
    import collections
    import csv
    import re
    import subprocess

    def means(path, counter):
        acc = collections.defaultdict(lambda: [0.0, 0])
        for row in csv.DictReader(open(path)):
            if row["Counter_Name"] != counter:
                continue
            e = acc[(row["Kernel_Name"], int(row["Grid_Size"]))]
            e[0] += float(row["Counter_Value"])
            e[1] += 1
        return {k: (v[0] / v[1], v[1]) for k, v in acc.items()}

    fetch, write = means(fetch_csv, "FETCH_SIZE"), means(write_csv, "WRITE_SIZE")
    ours = sorted(k for k in set(fetch) | set(write) if "kapy" in k[0])
    names = {}
    try:
        tool = "/opt/rocm/llvm/bin/llvm-cxxfilt" if os.path.exists("/opt/rocm/llvm/bin/llvm-cxxfilt") else "c++filt"
        demangled = subprocess.run([tool], input="\n".join(k[0] for k in ours), capture_output=True, text=True).stdout.split("\n")
        names = {k: d.replace("void ", "").replace("kapy::(anonymous namespace)::", "") for k, d in zip(ours, demangled)}
    except OSError:
        names = {k: k[0] for k in ours}

    def pick(pattern, grid):
        hits = [k for k in ours if re.search(pattern, names[k]) and (grid is None or k[1] == grid)]
        if not hits:
            return None
        best = max(hits, key=lambda k: fetch.get(k, (0, 0))[1])       # the form launched most often is the timed one
        return best

    out = ["rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE, all bench workloads, one MI355X (gfx950)", "",
           "commands (two runs, one counter each; from the repository root after `cd /tmp && export TMPDIR=/tmp && cd <repo>`):",
           "  rocprofv3 --pmc FETCH_SIZE -d gpurun_out/prof/pmc_fetch -o pmc_fetch --output-format csv -- python3 bench.py --no-cpu --skip ceilings,mlir_fixtures --steps 3 --warmup 1",
           "  rocprofv3 --pmc WRITE_SIZE -d gpurun_out/prof/pmc_write -o pmc_write --output-format csv -- python3 bench.py --no-cpu --skip ceilings,mlir_fixtures --steps 3 --warmup 1",
           "  python3 bench.py --pmc-summary <pmc_fetch counter_collection.csv> <pmc_write counter_collection.csv> > profiles/bench_all_workloads.hbm_traffic_pmc.txt",
           "", "Per-dispatch mean of the counter (rocprofv3 reports KiB), by kernel and grid size (work-items); n = dispatches seen.", "",
           "%-86s %10s %20s %20s" % ("kernel", "grid", "FETCH_SIZE (n)", "WRITE_SIZE (n)")]
    for k in ours:
        f, w = fetch.get(k, (0.0, 0)), write.get(k, (0.0, 0))
        out.append("%-86s %10d %12.1f (%5d) %12.1f (%5d)" % (names[k][:86], k[1], f[0], f[1], w[0], w[1]))
    copy = pick(*TRAFFIC_KERNELS[0][2][0])
    if copy is None or copy not in fetch or copy not in write:
        raise SystemExit("bench.py --pmc-summary: the copy kernel (rows_kernel) is in neither counter file; nothing to calibrate against")
    known_kib = 128 * 1024
    ff, wf = known_kib / fetch[copy][0], known_kib / write[copy][0]
    out += ["", "Calibration on the plain copy (%s reads exactly %d KiB and writes exactly %d KiB per launch):" % (names[copy][:40], known_kib, known_kib),
            "  FETCH_SIZE reads %.1f -> factor %.4f" % (fetch[copy][0], ff), "  WRITE_SIZE reads %.1f -> factor %.4f" % (write[copy][0], wf), "",
            "Scaled HBM-side traffic per launch (fetch x %.4f + write x %.4f, KiB -> bytes):" % (ff, wf)]
    lines = []
    for key, label, kernels in TRAFFIC_KERNELS:
        total, parts, ok = 0.0, [], True
        for pattern, grid in kernels:
            k = pick(pattern, grid)
            if k is None or k not in fetch or k not in write:
                ok = False
                break
            total += (fetch[k][0] * ff + write[k][0] * wf) * 1024.0
            parts.append("%s: fetch %.0f KiB + write %.0f KiB" % (names[k][:48], fetch[k][0] * ff, write[k][0] * wf))
        if not ok:
            out.append("  %-44s (kernel not seen in the counter files)" % label)
            continue
        out.append("  %-44s %9.1f MB   %s" % (label, total / 1e6, "; ".join(parts)))
        lines.append("traffic_bytes %s %d" % (key, round(total)))
    out += ["", "What bench.py reads (workload key, HBM-side bytes per launch):"] + lines
    print("\n".join(out))


def stats_summary(stats_csv):
    """The tracked per-kernel summary from a rocprofv3 --kernel-trace --stats run of this script: this library's kernels (and the
    kernels it compiled at run time), calls, average, minimum and maximum duration in nanoseconds, by total time."""
    import csv
    import subprocess
    rows = [r for r in csv.DictReader(open(stats_csv)) if "kapy" in r["Name"]]
    tool = "/opt/rocm/llvm/bin/llvm-cxxfilt" if os.path.exists("/opt/rocm/llvm/bin/llvm-cxxfilt") else "c++filt"
    try:
        names = subprocess.run([tool], input="\n".join(r["Name"] for r in rows), capture_output=True, text=True).stdout.split("\n")
    except OSError:
        names = [r["Name"] for r in rows]
    def short(n):
        m = re.match(r"_ZN4kapy12_GLOBAL__N_1(\d+)", n)            # names with _Float16 arguments come back mangled
        if m:
            rest = n[m.end():]
            return rest[:int(m.group(1))] + "<" + rest[int(m.group(1)) + 1:].split("EEv")[0] + "> (mangled arguments)"
        return n.replace("void ", "").replace("kapy::(anonymous namespace)::", "").replace("kapy::", "").split("(")[0]
    out = ["rocprofv3 kernel statistics, all bench workloads, one MI355X (gfx950)", "",
           "commands (from the repository root, after `cd /tmp && export TMPDIR=/tmp && cd <repo>`):",
           "  rocprofv3 --kernel-trace --stats -d gpurun_out/prof/stats_all -o stats_all --output-format csv -- python3 bench.py --no-cpu --skip ceilings",
           "  python3 bench.py --stats-summary <stats_all_kernel_stats.csv> > profiles/bench_all_workloads.kernel_stats.txt", "",
           "Rows of this library's kernels (torch's fill / compare kernels omitted).  Calls include the untimed clock pre-warm launches of",
           "bench.py.  kapy_ew_flat_* / kapy_ew_rows_* are the kernels kapy_elementwise compiled at run time in that process (the name ends in",
           "a hash of program and operand signature).  tn_kernel<..., true> (last argument) is the build with the fused tail.", "",
           "%-96s %8s %12s %10s %10s" % ("kernel", "calls", "avg_ns", "min_ns", "max_ns")]
    for r, n in sorted(zip(rows, names), key=lambda rn: -float(rn[0]["TotalDurationNs"])):
        out.append("%-96s %8d %12.0f %10d %10d" % (short(n)[:96], int(r["Calls"]), float(r["AverageNs"]), int(float(r["MinNs"])), int(float(r["MaxNs"]))))
    print("\n".join(out))


def ceilings_summary(bench_json):
    """The tracked summary of the probe kernels' figures from the JSON line of `bench.py --workload ceilings --no-others`."""
    line = json.loads(open(bench_json).read().strip().split("\n")[-1])
    res = next((r for r in [line.get("config", {})] + line.get("other_workloads", []) if "mfma" in r), None)
    if res is None:
        res = line
    out = ["Device ceilings measured by the probe library's kernels (libkapy_probe.so) and the tiled GEMMs' fixed cost per launch, one MI355X (gfx950)", "",
           "commands (from the repository root):",
           "  python3 bench.py --no-cpu --no-others --workload ceilings > gpurun_out/ceilings.json",
           "  python3 bench.py --ceilings-summary gpurun_out/ceilings.json > profiles/device_ceilings.probe_kernels.txt", "",
           "bench.py's figures in that run (HIP events around back-to-back launches; the shader clock is what the kernel itself reads: s_memtime",
           "ticks of one wave against the 100 MHz s_memrealtime over the same interval)."]

    def dump(d, indent):
        for k, v in d.items():
            if isinstance(v, dict):
                out.append("%s%s:" % (" " * indent, k))
                dump(v, indent + 2)
            else:
                out.append("%s%-*s %s" % (" " * indent, max(4, 96 - indent), k, v))

    for key, title in (("mfma", "matrix instruction loop (every CU: 4 waves of independent matrix instructions on registers, no memory traffic)"),
                       ("copy", "plain copy of 128 MiB to another 128 MiB buffer, GB/s read + written (vecN = 16-byte vectors per lane and step, ntld / ntst = non-temporal loads / stores)"),
                       ("read", "read-only stream of 64 MiB buffers in rotation, GB/s"), ("l2_read_tbs", "reads of a window that stays in the XCD's L2 / the Infinity Cache / neither, TB/s"),
                       ("issue_tflops", "matrix instructions with fillers in the gaps behind them, TFLOP/s"), ("gemm_fixed_cost", "the tiled GEMMs at K and 2K")):
        if key in res:
            out += ["", title]
            dump(res[key], 2)
    for key in ("copy_best_gbs", "copy_best_frac_of_peak", "read_best_gbs", "read_best_frac_of_peak"):
        if key in res:
            out.append("%-40s %s" % (key, res[key]))
    print("\n".join(out))


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--workload", default="gelu", choices=WORKLOADS)
    ap.add_argument("--no-others", action="store_true", help="measure only the selected workload")
    ap.add_argument("--skip", default="", help="comma-separated workloads to leave out of the other workloads (e.g. ceilings, whose probe launches reuse the GEMM kernels at other sizes and would mix into a profiler's per-kernel averages)")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline legs")
    ap.add_argument("--pmc-summary", nargs=2, metavar=("FETCH_CSV", "WRITE_CSV"), help="no measurement: write the HBM-traffic summary that `traffic` is read from, from the counter_collection.csv files of two rocprofv3 --pmc runs of this script (FETCH_SIZE, then WRITE_SIZE)")
    ap.add_argument("--stats-summary", metavar="STATS_CSV", help="no measurement: the per-kernel summary kept under profiles/, from the kernel_stats.csv of a rocprofv3 --kernel-trace --stats run of this script")
    ap.add_argument("--ceilings-summary", metavar="BENCH_JSON", help="no measurement: the summary of the probe kernels' figures kept under profiles/, from the JSON line of --workload ceilings")
    args = ap.parse_args()
    if args.pmc_summary:
        pmc_summary(*args.pmc_summary)
        return
    if args.stats_summary:
        stats_summary(args.stats_summary)
        return
    if args.ceilings_summary:
        ceilings_summary(args.ceilings_summary)
        return
    if args.gpus != 1:
        sys.exit("bench.py: this build measures one GPU; --gpus %d is not supported (every path here runs on a single MI355X)" % args.gpus)
    import torch
    import kapy_hip as kh
    if not torch.cuda.is_available():
        sys.exit("bench.py: no GPU visible; the library has no CPU fallback to time")
    torch.cuda.set_device(0)
    kh.lib()
    cpu = not args.no_cpu
    table = {
        "gelu": lambda s, w: bench_gelu(kh, s, w, cpu),
        "add": lambda s, w: bench_add(kh, s, w, cpu),
        "expr": lambda s, w: bench_add(kh, s, w, cpu, "expr"),
        "expr_compiled": lambda s, w: bench_add(kh, s, w, cpu, "expr_compiled"),
        "swiglu": lambda s, w: bench_add(kh, s, w, cpu, "swiglu"),
        "copy": lambda s, w: bench_copy(kh, s, w, cpu),
        "transpose": lambda s, w: bench_transpose(kh, s, w, cpu),
        "gelu_transposed": lambda s, w: bench_gelu_transposed(kh, s, w, cpu),
        "reduce": lambda s, w: bench_reduce(kh, s, w, cpu),
        "reduce_cols": lambda s, w: bench_reduce_cols(kh, s, w, cpu),
        "softmax_cols": lambda s, w: bench_softmax_cols(kh, s, w, cpu),
        "softmax": lambda s, w: bench_rowwise(kh, s, w, cpu, "softmax"),
        "causal_softmax": lambda s, w: bench_rowwise(kh, s, w, cpu, "causal_softmax"),
        "layernorm": lambda s, w: bench_rowwise(kh, s, w, cpu, "layernorm"),
        "l2norm_compiled": lambda s, w: bench_rowwise(kh, s, w, cpu, "l2norm_compiled"),
        "permute": lambda s, w: bench_permute(kh, s, w, cpu),
        "gemm_bf16": lambda s, w: bench_gemm(kh, s, w, cpu, 8192, 8192, 8192, kh.BF16, True, "C4 gemm bf16 8192^3 A row-major B col-major", "tn_kernel", key="gemm_bf16"),
        "gemm_bf16_gelu": lambda s, w: bench_gemm(kh, s, w, cpu, 8192, 8192, 8192, kh.BF16, True, "C4 gemm bf16 8192^3 with gelu_tanh(c*0.5 + bias) fused into the epilogue", "tn_kernel", fused_gelu=True, key="gemm_bf16_gelu"),
        "mlir_fixtures": lambda s, w: bench_mlir(kh, s, w, cpu),
        "gemm_bf16_nn": lambda s, w: bench_gemm(kh, s, w, False, 8192, 8192, 8192, kh.BF16, False, "gemm bf16 8192^3, both operands row-major, the rhs read in place by transposing LDS reads (256 x 256 tiles)", "nn256_kernel", key="gemm_bf16_nn", whole=False),
        "gemm_bf16_nn_turned": lambda s, w: bench_gemm(kh, s, w, False, 8192, 8192, 8192, kh.BF16, True, "gemm bf16 8192^3, lhs column-major, rhs column-major, workspace given: the lhs is turned K-contiguous first (time and rate include the turn)", "transpose_lds_kernel + tn_kernel", key="gemm_bf16_nn_turned", workspace=True, whole=False, a_col_major=True),
        "gemm_bf16_m128": lambda s, w: bench_gemm(kh, s, w, False, 128, 8192, 8192, kh.BF16, True, "gemm bf16 128 x 8192 x 8192, rhs column-major: one 64 x 64 x 128 tile per CU (a weight-streaming shape: its 138 MB in 31 us are 4.4 TB/s of HBM reads, whatever the matrix-pipe fraction says)", "tn_kernel, 64 x 64 x 128 tiles, four stages", key="gemm_bf16_m128"),
        "gemm_f16": lambda s, w: bench_gemm(kh, s, w, cpu, 1024, 1024, 1024, kh.F16, False, "C1 gemm fp16 1024^3 row-major 128x128x32 tiles", "nn_kernel", tile=(128, 128, 32), gen="uniform", key="gemm_f16"),
        "gemm_f16_graph": lambda s, w: bench_gemm(kh, s, w, cpu, 1024, 1024, 1024, kh.F16, False, "C1 gemm fp16 1024^3, 20 launches replayed from a HIP graph (per launch)", "nn_kernel", tile=(128, 128, 32), graph_of=20, gen="uniform", key="gemm_f16_graph"),
        "gemm_f16_splitk": lambda s, w: bench_gemm(kh, s, w, False, 1024, 1024, 1024, kh.F16, False, "C1 gemm fp16 1024^3 row-major 128x128x32 tiles, K split across workgroups (workspace given)", "nn_kernel, split K", tile=(128, 128, 32), gen="uniform", workspace=True, key="gemm_f16_splitk"),
        "f8_m16": lambda s, w: bench_f8(kh, s, w, cpu, 16),
        "f8_m64": lambda s, w: bench_f8(kh, s, w, False, 64),
        "f8_m128": lambda s, w: bench_f8(kh, s, w, False, 128),
        "f8_m128_splitk": lambda s, w: bench_f8(kh, s, w, False, 128, workspace=True),
        "f8_m256": lambda s, w: bench_f8(kh, s, w, False, 256),
        "f8_m4096": lambda s, w: bench_f8(kh, s, w, cpu, 4096),
        "ceilings": lambda s, w: bench_ceilings(kh, s, w, cpu),
    }
    if args.workload == "ceilings":
        print(json.dumps(table["ceilings"](args.steps, args.warmup)))
        return
    try:
        main_res = table[args.workload](args.steps, args.warmup)
    except CheckFailed as e:
        sys.exit("bench.py: correctness gate failed, nothing timed: %s" % e)
    others, other_names = [], []
    if not args.no_others:
        for name, fn in table.items():
            if name == args.workload or (name == "expr" and args.workload == "expr_compiled"):   # once compiled, the program no longer reaches the machine
                continue
            if name in [w.strip() for w in args.skip.split(",") if w.strip()]:
                continue
            torch.cuda.empty_cache()
            other_names.append(name)
            try:
                r = fn(min(args.steps, 20), min(args.warmup, 10))
            except kh.KapyError as e:   # e.g. no runtime compiler on this machine for the compiled workloads
                others.append({"workload": name, "error": str(e), "checked": False})
                continue
            except CheckFailed as e:
                others.append({"workload": name, "error": "correctness gate failed, not timed: %s" % e, "checked": False})
                continue
            if "value" in r:
                r["value"] = round(r["value"], 2)
                r["ms_per_step"] = round(r["ms_per_step"], 4)
                r["kernel_ms"] = round(r["kernel_ms"], 4)
            others.append(r)
    # every benchmark configuration in one compact block inside "config" (a key that records of this line keep), and the long
    # tables first in the line, so that its end - what a truncated log keeps - holds the configurations and the headline
    by_name = dict([(args.workload, main_res)] + [(n, r) for n, r in zip(other_names, others)])
    configs = {}
    for cfg, name in (("C1", "gemm_f16"), ("C2", "gelu"), ("C3a", "transpose"), ("C3b", "permute"), ("C4", "gemm_bf16"), ("C5_M16", "f8_m16"), ("C5_M4096", "f8_m4096")):
        r = by_name.get(name)
        if r is None:
            continue
        if "roofline" not in r:
            configs[cfg] = {"checked": False, "error": r.get("error", "not run")}
            continue
        configs[cfg] = {"value": round(r["value"], 2), "unit": r["unit"], "kernel_ms": round(r["kernel_ms"], 4), "bound": r["roofline"]["bound"],
                        "frac": r["roofline"]["frac"], "checked": r["checked"], "kernel": r["kernel"],
                        "cpu_baseline": (r.get("cpu_baseline") or {}).get("value"), "cpu_unit": (r.get("cpu_baseline") or {}).get("unit")}
    others.sort(key=lambda r: 0 if r.get("workload", "").startswith("device ceilings") else 1)
    line = {
        "other_workloads": others,
        "metric": "GEMM TFLOP/s + % MFMA peak; elementwise/transpose GB/s + % HBM peak (1 GPU)",
        "value": round(main_res["value"], 2), "unit": main_res["unit"], "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(main_res["ms_per_step"], 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": main_res["dtype"], "data": "synthetic",
        "config": {"workload": main_res["workload"], "kernel": main_res["kernel"], "kernel_ms": round(main_res["kernel_ms"], 4),
                   "inputs": main_res["inputs"], "checked": main_res["checked"], "check": main_res["check"],
                   "buffers": "4 rotating sets (1 GiB) so reads miss the Infinity Cache" if main_res["unit"] == "GB/s" else "single set",
                   "configs": configs, **({"programs": main_res["programs"]} if "programs" in main_res else {})},
        "roofline": main_res["roofline"],
        "cpu_baseline": main_res.get("cpu_baseline"),
    }
    print(json.dumps(line))


if __name__ == "__main__":
    main()
