#!/usr/bin/env python3
"""Benchmark of the kapy hot path on one MI355X.

`python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload NAME] [--no-others] [--no-cpu]`

A step is one pass of the hot path over one batch of synthetic input, inputs resident in HBM.
The headline workload (the configuration the headline metric is quoted on) is the fused elementwise
y = GELU_tanh(x*0.5 + bias) on fp16 8192x8192; the JSON line also carries every other benchmark
configuration under "other_workloads", each with its own roofline.  One JSON line on stdout.

Timing: K launches bracketed by torch.cuda.synchronize() give ms_per_step / value; HIP events
recorded on the stream the kernels are launched on (torch's current stream, whose handle is
passed to the C ABI) give the per-launch duration used for roofline.achieved.  Memory-bound
workloads rotate over buffer sets larger than the 256 MB Infinity Cache so the rate is HBM's.
"""
import argparse
import ctypes as C
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.join(ROOT, "kapy-lang_amd", "python"))

HBM_PEAK_GBS = 8000.0
MFMA_PEAK_TFLOPS = {"bf16": 2500.0, "f16": 2500.0, "f8": 5000.0}


PREWARM_S = 0.25  # untimed launches before the W warm-up steps: the GPU clock needs ~0.2 s of load to settle


def _events(fn, steps, warmup):
    """Run fn(i) untimed until the clock has settled, then warmup + steps times;
    return (wall ms per step, event ms per launch)."""
    import torch
    t0, i = time.perf_counter(), 0
    while time.perf_counter() - t0 < PREWARM_S:
        fn(i)
        i += 1
        if i % 8 == 0:
            torch.cuda.synchronize()
    for i in range(warmup):
        fn(i)
    torch.cuda.synchronize()
    start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    start.record()
    for i in range(steps):
        fn(i)
    end.record()
    torch.cuda.synchronize()
    wall_ms = (time.perf_counter() - t0) * 1e3 / steps
    return wall_ms, start.elapsed_time(end) / steps


# HBM bytes per launch from rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE (two runs), each scaled by what the
# same counter reads for the rows copy of 2 x 128 MiB (workload "copy"); the summaries are under profiles/.
MEASURED_TRAFFIC = {"gelu": 268414976, "transpose": 268456960, "add": 402639872, "softmax": 268476416, "layernorm": 268788736,
                    "expr_compiled": 402619392, "swiglu": 402556928, "l2norm_compiled": 268408832}


def _roof_hbm(bytes_per_launch, ev_ms, key=None):
    a = bytes_per_launch / (ev_ms * 1e-3) / 1e9
    return {"bound": "hbm", "achieved": round(a, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": round(a / HBM_PEAK_GBS, 4),
            "traffic": MEASURED_TRAFFIC.get(key)}


def _roof_mfma(flops, ev_ms, kind):
    a = flops / (ev_ms * 1e-3) / 1e12
    p = MFMA_PEAK_TFLOPS[kind]
    return {"bound": "mfma", "achieved": round(a, 1), "peak": p, "unit": "TFLOP/s", "frac": round(a / p, 4), "traffic": None}


def bench_gelu(kh, steps, warmup):
    import torch
    n, sets = 8192, 4
    xs = [torch.randn(n, n, device="cuda", dtype=torch.float16) for _ in range(sets)]
    ys = [torch.empty(n, n, device="cuda", dtype=torch.float16) for _ in range(sets)]
    bias = torch.randn(n, device="cuda", dtype=torch.float16)
    prog = kh.gelu_program(kh.F16, 0.5)
    gx = [kh.mk_global(x.data_ptr(), n, n, n, 1, kh.F16) for x in xs]
    gy = [kh.mk_global(y.data_ptr(), n, n, n, 1, kh.F16) for y in ys]
    gb = kh.mk_global(bias.data_ptr(), 1, n, n, 1, kh.F16)
    wall, ev = _events(lambda i: kh.elementwise(prog, [gx[i % sets], gb], gy[i % sets]), steps, warmup)
    nbytes = 2 * n * n * 2 + n * 2
    return {"workload": "C2 gelu_tanh(x*0.5+bias) fp16 8192x8192", "value": nbytes / (wall * 1e-3) / 1e9, "unit": "GB/s",
            "ms_per_step": wall, "kernel_ms": ev, "dtype": "f16", "roofline": _roof_hbm(nbytes, ev, "gelu"), "kernel": "affine_act_cols_kernel"}


def bench_copy(kh, steps, warmup):
    """Plain row-major copy of the headline shape: the practical HBM ceiling the other kernels are read against,
    and the known-size kernel that calibrates the FETCH_SIZE / WRITE_SIZE counters."""
    import torch
    n, sets = 8192, 4
    xs = [torch.randint(-32768, 32767, (n, n), device="cuda", dtype=torch.int16) for _ in range(sets)]
    ys = [torch.empty(n, n, device="cuda", dtype=torch.int16) for _ in range(sets)]
    gx = [kh.mk_global(x.data_ptr(), n, n, n, 1, kh.F16) for x in xs]
    gy = [kh.mk_global(y.data_ptr(), n, n, n, 1, kh.F16) for y in ys]
    wall, ev = _events(lambda i: kh.copy(gx[i % sets], gy[i % sets]), steps, warmup)
    nbytes = 2 * n * n * 2
    return {"workload": "copy fp16 8192x8192 (ld_global -> st_global, no transpose)", "value": nbytes / (wall * 1e-3) / 1e9, "unit": "GB/s",
            "ms_per_step": wall, "kernel_ms": ev, "dtype": "u16", "roofline": _roof_hbm(nbytes, ev), "kernel": "rows_kernel"}


def bench_add(kh, steps, warmup, op="add"):
    """z = x + y in fp16 (the reference's elementwise_add.mlir fixture at the headline shape), a plain binary program,
    served by the fused affine kernel; op="expr": z = x*y + x with both roundings, a program outside the fused chains,
    served by the in-register stack machine; op="expr_compiled": the same program after kapy_elementwise_specialize has
    compiled it to a kernel of its own; op="swiglu": z = silu(x) * y in fp32 from fp16 operands (ten ops, x used twice), compiled."""
    import torch
    n, sets = 8192, 3
    xs = [torch.randn(n, n, device="cuda", dtype=torch.float16) for _ in range(sets)]
    ys = [torch.randn(n, n, device="cuda", dtype=torch.float16) for _ in range(sets)]
    zs = [torch.empty(n, n, device="cuda", dtype=torch.float16) for _ in range(sets)]
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
    prog = kh.program(insts + [dict(op=kh.EW_ST_GLOBAL, a=2)])
    if op in ("expr_compiled", "swiglu"):
        kh.elementwise_specialize(prog, [gx[0], gy[0]], gz[0])
    wall, ev = _events(lambda i: kh.elementwise(prog, [gx[i % sets], gy[i % sets]], gz[i % sets]), steps, warmup)
    nbytes = 3 * n * n * 2
    name = {"add": "elementwise_add fixture: z = x + y fp16 8192x8192", "expr": "z = x*y + x (two roundings) fp16 8192x8192",
            "expr_compiled": "z = x*y + x (two roundings) fp16 8192x8192, compiled at run time",
            "swiglu": "z = silu(x)*y fp16 8192x8192 in fp32, compiled at run time"}[op]
    kernel = {"add": "affine_act_kernel", "expr": "stack_kernel_narrow"}.get(op, "kapy_ew_flat_<hash> (compiled at run time)")
    return {"workload": name, "value": nbytes / (wall * 1e-3) / 1e9, "unit": "GB/s", "ms_per_step": wall, "kernel_ms": ev, "dtype": "f16",
            "roofline": _roof_hbm(nbytes, ev, op if op != "expr" else None), "kernel": kernel}


def bench_gelu_transposed(kh, steps, warmup):
    """y = gelu_tanh(x^T*0.5 + bias): the C3a transpose fused with the C2 chain - x is read through a view with swapped
    strides - compiled at run time onto the tiled skeleton (64 x 64 tiles, the column-major operand staged through LDS)."""
    import torch
    n, sets = 8192, 4
    xs = [torch.randn(n, n, device="cuda", dtype=torch.float16) for _ in range(sets)]
    ys = [torch.empty(n, n, device="cuda", dtype=torch.float16) for _ in range(sets)]
    bias = torch.randn(n, device="cuda", dtype=torch.float16)
    gx = [kh.mk_global(x.data_ptr(), n, n, 1, n, kh.F16) for x in xs]       # element (i, j) of the view is x[j, i]
    gy = [kh.mk_global(y.data_ptr(), n, n, n, 1, kh.F16) for y in ys]
    gb = kh.mk_global(bias.data_ptr(), 1, n, n, 1, kh.F16)
    prog = kh.gelu_program(kh.F16, 0.5)
    kh.elementwise_specialize(prog, [gx[0], gb], gy[0])
    wall, ev = _events(lambda i: kh.elementwise(prog, [gx[i % sets], gb], gy[i % sets]), steps, warmup)
    nbytes = 2 * n * n * 2 + n * 2
    return {"workload": "gelu_tanh(x^T*0.5+bias) fp16 8192x8192: transpose fused with the elementwise chain, compiled at run time",
            "value": nbytes / (wall * 1e-3) / 1e9, "unit": "GB/s", "ms_per_step": wall, "kernel_ms": ev, "dtype": "f16",
            "roofline": _roof_hbm(nbytes, ev), "kernel": "kapy_ew_flat_<hash> (tiled; compiled at run time)"}


def bench_reduce(kh, steps, warmup):
    """kapy.reduce (sum along rows) of the headline shape: the first adjacent op after the hot path proper."""
    import torch
    n, sets = 8192, 4
    xs = [torch.randn(n, n, device="cuda", dtype=torch.float16) for _ in range(sets)]
    y = torch.empty(n, device="cuda", dtype=torch.float32)
    gx = [kh.mk_global(x.data_ptr(), n, n, n, 1, kh.F16) for x in xs]
    gy = kh.mk_global(y.data_ptr(), n, 1, 1, n, kh.F32)
    wall, ev = _events(lambda i: kh.reduce(gx[i % sets], gy, 1, 0), steps, warmup)
    nbytes = n * n * 2 + n * 4
    return {"workload": "reduce_sum axis=1 fp16 8192x8192 -> f32 [8192x1]", "value": nbytes / (wall * 1e-3) / 1e9, "unit": "GB/s",
            "ms_per_step": wall, "kernel_ms": ev, "dtype": "f16", "roofline": _roof_hbm(nbytes, ev), "kernel": "reduce_rows_vec_kernel"}


def bench_rowwise(kh, steps, warmup, which):
    """Row-wise fusion of kapy.reduce with its elementwise neighbours at the headline shape: softmax or layer norm of
    every row in one pass over HBM (one read of x, one write of y; gamma and beta stay in cache)."""
    import torch
    n, sets = 8192, 4
    xs = [torch.randn(n, n, device="cuda", dtype=torch.float16) for _ in range(sets)]
    ys = [torch.empty(n, n, device="cuda", dtype=torch.float16) for _ in range(sets)]
    gamma, beta = torch.ones(n, device="cuda", dtype=torch.float16), torch.zeros(n, device="cuda", dtype=torch.float16)
    g = lambda t: kh.mk_global(t.data_ptr(), n, n, n, 1, kh.F16)
    row = lambda t: kh.mk_global(t.data_ptr(), 1, n, n, 1, kh.F16)
    gx, gy = [g(t) for t in xs], [g(t) for t in ys]
    if which == "softmax":
        prog, extra = kh.program(kh.softmax_insts(kh.F16)), []
    elif which == "l2norm_compiled":   # x / |x| per row: a row program without a hand-written kernel, compiled at run time
        f32 = dict(op=kh.EW_FPTOFP, dst=0, a=0, dtype=kh.F32)
        prog, extra = kh.program([dict(op=kh.EW_LD_GLOBAL, dst=0, a=0), f32, dict(op=kh.EW_MULF, dst=1, a=0, b=0), dict(op=kh.EW_REDUCE_SUM, dst=1, a=1, b=1),
                                  dict(op=kh.EW_RSQRT, dst=1, a=1), dict(op=kh.EW_MULF, dst=0, a=0, b=1),
                                  dict(op=kh.EW_FPTOFP, dst=2, a=0, dtype=kh.F16, rmode=kh.RN), dict(op=kh.EW_ST_GLOBAL, a=2)]), []
        kh.elementwise_specialize(prog, [gx[0]], gy[0])
    else:
        prog, extra = kh.program(kh.layernorm_insts(n, kh.F16)), [row(gamma), row(beta)]
    wall, ev = _events(lambda i: kh.elementwise(prog, [gx[i % sets]] + extra, gy[i % sets]), steps, warmup)
    nbytes = 2 * n * n * 2
    name = "x * rsqrt(sum x^2) of every row, compiled at run time" if which == "l2norm_compiled" else "%s of every row" % which
    return {"workload": "%s, fp16 8192x8192, fp32 arithmetic" % name, "value": nbytes / (wall * 1e-3) / 1e9, "unit": "GB/s",
            "ms_per_step": wall, "kernel_ms": ev, "dtype": "f16", "roofline": _roof_hbm(nbytes, ev, which),
            "kernel": {"softmax": "softmax_kernel", "layernorm": "norm_kernel"}.get(which, "kapy_ew_rows_<hash> (compiled at run time)")}


def bench_transpose(kh, steps, warmup):
    import torch
    n, sets = 8192, 4
    xs = [torch.randint(-32768, 32767, (n, n), device="cuda", dtype=torch.int16) for _ in range(sets)]
    ys = [torch.empty(n, n, device="cuda", dtype=torch.int16) for _ in range(sets)]
    gx = [kh.mk_global(x.data_ptr(), n, n, n, 1, kh.F16) for x in xs]
    gy = [kh.mk_global(y.data_ptr(), n, n, n, 1, kh.F16) for y in ys]
    wall, ev = _events(lambda i: kh.copy(gx[i % sets], gy[i % sets], transpose=True), steps, warmup)
    nbytes = 2 * n * n * 2
    return {"workload": "C3a transpose fp16 8192x8192", "value": nbytes / (wall * 1e-3) / 1e9, "unit": "GB/s", "ms_per_step": wall,
            "kernel_ms": ev, "dtype": "u16", "roofline": _roof_hbm(nbytes, ev, "transpose"), "kernel": "transpose_lds_kernel"}


def bench_permute(kh, steps, warmup):
    import torch
    b, h, s, d, sets = 8, 32, 2048, 128, 4
    xs = [torch.randint(-32768, 32767, (b * h * s * d,), device="cuda", dtype=torch.int16) for _ in range(sets)]
    ys = [torch.empty(b * h * s * d, device="cuda", dtype=torch.int16) for _ in range(sets)]
    gx = [kh.mk_global(x.data_ptr(), s, d, d, 1, kh.BF16) for x in xs]
    gy = [kh.mk_global(y.data_ptr(), s, d, h * d, 1, kh.BF16) for y in ys]
    grid = (b, h, h * s * d, s * d, s * h * d, d)
    wall, ev = _events(lambda i: kh.copy_batched(gx[i % sets], gy[i % sets], grid), steps, warmup)
    nbytes = 2 * b * h * s * d * 2
    return {"workload": "C3b permute bf16 [8,32,2048,128] bhsd->bshd", "value": nbytes / (wall * 1e-3) / 1e9, "unit": "GB/s",
            "ms_per_step": wall, "kernel_ms": ev, "dtype": "u16", "roofline": _roof_hbm(nbytes, ev), "kernel": "rows_kernel"}


def bench_gemm(kh, steps, warmup, M, N, K, dtype, b_col_major, name, kernel, tile=(0, 0, 0), graph_of=0, fused_gelu=False):
    """graph_of > 0: that many back-to-back launches recorded once into a HIP graph; a step is one replay, figures are per launch
    (what a launch-bound shape gains when the host's per-launch cost is taken out).
    fused_gelu: d = gelu_tanh(a.b*0.5 + bias) with the tail in the GEMM's epilogue (kapy_matmul_fused); flops counted are the GEMM's."""
    import torch
    tdt = torch.bfloat16 if dtype == kh.BF16 else torch.float16
    std = 0.02 if dtype == kh.BF16 else 0.5
    a = (torch.randn(M, K, device="cuda") * std).to(tdt)
    b = (torch.randn(N, K, device="cuda") * std).to(tdt) if b_col_major else (torch.randn(K, N, device="cuda") * std).to(tdt)
    d = torch.empty(M, N, device="cuda", dtype=tdt)
    ga = kh.mk_global(a.data_ptr(), M, K, K, 1, dtype)
    gb = kh.mk_global(b.data_ptr(), K, N, 1, K, dtype) if b_col_major else kh.mk_global(b.data_ptr(), K, N, N, 1, dtype)
    gd = kh.mk_global(d.data_ptr(), M, N, N, 1, dtype)
    if fused_gelu:
        bias = torch.randn(N, device="cuda").to(tdt)
        gbias = kh.mk_global(bias.data_ptr(), 1, N, N, 1, dtype)
        wall, ev = _events(lambda i: kh.matmul_fused(ga, gb, gd, bias=gbias, alpha=0.5, act=kh.EW_GELU_TANH, tile=tile), steps, warmup)
    elif graph_of:
        kh.matmul(ga, gb, gd, tile=tile)
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            for _ in range(graph_of):
                kh.matmul(ga, gb, gd, tile=tile)
        wall, ev = _events(lambda i: graph.replay(), steps, warmup)
        wall, ev = wall / graph_of, ev / graph_of
    else:
        wall, ev = _events(lambda i: kh.matmul(ga, gb, gd, tile=tile), steps, warmup)
    flops = 2.0 * M * N * K
    kind = "bf16" if dtype == kh.BF16 else "f16"
    return {"workload": name, "value": flops / (wall * 1e-3) / 1e12, "unit": "TFLOP/s", "ms_per_step": wall, "kernel_ms": ev,
            "dtype": kind, "roofline": _roof_mfma(flops, ev, kind), "kernel": kernel}


def bench_f8(kh, steps, warmup, M):
    import torch
    N = K = 8192
    a = torch.randint(0, 120, (M, K), device="cuda", dtype=torch.uint8)      # finite e4m3 patterns
    sets = 6 if M <= 64 else 2                                               # M<=64 is weight-streaming: 6 x 64 MiB > Infinity Cache
    ws = [torch.randint(0, 120, (N, K), device="cuda", dtype=torch.uint8) for _ in range(sets)]
    sa = torch.rand(M, device="cuda") * 0.01 + 0.001
    sb = torch.rand(N, device="cuda") * 0.01 + 0.001
    d = torch.empty(M, N, device="cuda", dtype=torch.bfloat16)
    ga = kh.mk_global(a.data_ptr(), M, K, K, 1, kh.F8E4M3)
    gws = [kh.mk_global(w.data_ptr(), K, N, 1, K, kh.F8E4M3) for w in ws]
    gd = kh.mk_global(d.data_ptr(), M, N, N, 1, kh.BF16)
    wall, ev = _events(lambda i: kh.matmul_scaled_f8(ga, gws[i % sets], sa.data_ptr(), sb.data_ptr(), gd), steps, warmup)
    flops = 2.0 * M * N * K
    nbytes = M * K + N * K + M * N * 2 + (M + N) * 4
    out = {"workload": "C5 W8A8 e4m3 M=%d N=K=8192" % M, "value": flops / (wall * 1e-3) / 1e12, "unit": "TFLOP/s",
           "ms_per_step": wall, "kernel_ms": ev, "dtype": "f8e4m3", "kernel": "skinny_stream_kernel" if M <= 64 else "tn_kernel<F8>"}
    out["roofline"] = _roof_hbm(nbytes, ev) if M <= 64 else _roof_mfma(flops, ev, "f8")
    return out


def cpu_baseline_gelu(sample_rows=256):
    """The oracle's elementwise program on a bounded sample (sample_rows x 8192) of the same workload,
    on this box's host cores.  Reported, never the optimisation target."""
    sys.path.insert(0, os.path.join(ROOT, "oracle"))
    import numpy as np
    import ko
    n = 8192
    x = ko.fill_normal(sample_rows * n, ko.F16, 0, 0).reshape(sample_rows, n)
    bias = ko.fill_normal(n, ko.F16, 1, 0)
    out = np.zeros((sample_rows, n), dtype=np.uint16)
    prog = ko.gelu_program()
    gx, gb, go = ko.mk_global(x, sample_rows, n, n, 1, ko.F16), ko.mk_global(bias, 1, n, n, 1, ko.F16), ko.mk_global(out, sample_rows, n, n, 1, ko.F16)
    ko.elementwise(prog, [gx, gb], go)  # warm-up
    reps, t0 = 0, time.perf_counter()
    while True:
        ko.elementwise(prog, [gx, gb], go)
        reps += 1
        dt = time.perf_counter() - t0
        if dt > 10.0:
            break
    nbytes = (2 * sample_rows * n * 2 + n * 2) * reps
    return {"value": round(nbytes / dt / 1e9, 4), "unit": "GB/s", "cores": ko.lib().ko_num_threads(), "kind": "port",
            "sample": "%d of 8192 rows of the same workload, %d repetitions, %.1f s" % (sample_rows, reps, dt)}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--workload", default="gelu", choices=["gelu", "add", "expr", "expr_compiled", "swiglu", "copy", "reduce", "softmax", "layernorm", "l2norm_compiled", "gelu_transposed", "transpose", "permute", "gemm_bf16", "gemm_bf16_gelu", "gemm_f16", "gemm_f16_graph", "f8_m16", "f8_m4096"])
    ap.add_argument("--no-others", action="store_true", help="measure only the selected workload")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build measures one GPU; --gpus %d is not supported (every path here runs on a single MI355X)" % args.gpus)
    import torch
    import kapy_hip as kh
    if not torch.cuda.is_available():
        sys.exit("bench.py: no GPU visible; the library has no CPU fallback to time")
    torch.cuda.set_device(0)
    kh.lib()
    table = {
        "gelu": lambda s, w: bench_gelu(kh, s, w),
        "add": lambda s, w: bench_add(kh, s, w),
        "expr": lambda s, w: bench_add(kh, s, w, "expr"),
        "expr_compiled": lambda s, w: bench_add(kh, s, w, "expr_compiled"),
        "swiglu": lambda s, w: bench_add(kh, s, w, "swiglu"),
        "copy": lambda s, w: bench_copy(kh, s, w),
        "transpose": lambda s, w: bench_transpose(kh, s, w),
        "gelu_transposed": lambda s, w: bench_gelu_transposed(kh, s, w),
        "reduce": lambda s, w: bench_reduce(kh, s, w),
        "softmax": lambda s, w: bench_rowwise(kh, s, w, "softmax"),
        "layernorm": lambda s, w: bench_rowwise(kh, s, w, "layernorm"),
        "l2norm_compiled": lambda s, w: bench_rowwise(kh, s, w, "l2norm_compiled"),
        "permute": lambda s, w: bench_permute(kh, s, w),
        "gemm_bf16": lambda s, w: bench_gemm(kh, s, w, 8192, 8192, 8192, kh.BF16, True, "C4 gemm bf16 8192^3 A row-major B col-major", "tn_kernel"),
        "gemm_bf16_gelu": lambda s, w: bench_gemm(kh, s, w, 8192, 8192, 8192, kh.BF16, True, "C4 gemm bf16 8192^3 with gelu_tanh(c*0.5 + bias) fused into the epilogue", "tn_kernel", fused_gelu=True),
        "gemm_f16": lambda s, w: bench_gemm(kh, s, w, 1024, 1024, 1024, kh.F16, False, "C1 gemm fp16 1024^3 row-major 128x128x32 tiles", "nn_kernel", tile=(128, 128, 32)),
        "gemm_f16_graph": lambda s, w: bench_gemm(kh, s, w, 1024, 1024, 1024, kh.F16, False, "C1 gemm fp16 1024^3, 20 launches replayed from a HIP graph (per launch)", "nn_kernel", tile=(128, 128, 32), graph_of=20),
        "f8_m16": lambda s, w: bench_f8(kh, s, w, 16),
        "f8_m4096": lambda s, w: bench_f8(kh, s, w, 4096),
    }
    main_res = table[args.workload](args.steps, args.warmup)
    others = []
    if not args.no_others:
        for name, fn in table.items():
            if name == args.workload or (name == "expr" and args.workload == "expr_compiled"):   # once compiled, the program no longer reaches the machine
                continue
            torch.cuda.empty_cache()
            try:
                r = fn(min(args.steps, 20), min(args.warmup, 10))
            except kh.KapyError as e:   # e.g. no runtime compiler on this machine for the compiled workloads
                others.append({"workload": name, "error": str(e)})
                continue
            r["value"] = round(r["value"], 2)
            r["ms_per_step"] = round(r["ms_per_step"], 4)
            r["kernel_ms"] = round(r["kernel_ms"], 4)
            others.append(r)
    line = {
        "metric": "GEMM TFLOP/s + % MFMA peak; elementwise/transpose GB/s + % HBM peak (1 GPU)",
        "value": round(main_res["value"], 2), "unit": main_res["unit"], "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(main_res["ms_per_step"], 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": main_res["dtype"], "data": "synthetic",
        "config": {"workload": main_res["workload"], "kernel": main_res["kernel"], "kernel_ms": round(main_res["kernel_ms"], 4),
                   "buffers": "4 rotating sets (1 GiB) so reads miss the Infinity Cache" if main_res["unit"] == "GB/s" else "single set"},
        "roofline": main_res["roofline"],
        "cpu_baseline": None if args.no_cpu else cpu_baseline_gelu(),
        "other_workloads": others,
    }
    print(json.dumps(line))


if __name__ == "__main__":
    main()
