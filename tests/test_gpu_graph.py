"""The entry points under HIP graph capture: every kernel family of the hot path is recorded once into a graph and
replayed with fresh operand contents; each replay must reproduce, bit for bit, what the same calls give eagerly.
(The library launches on the caller's stream, allocates nothing and clears nothing, so a capture sees only kernels.)"""
import numpy as np
import pytest
import torch

import kapy_hip as kh
from gpu_util import dglobal, sync

pytestmark = pytest.mark.gpu


def _calls(bufs, out):
    """One pass of the hot path over static buffers: GELU -> transpose -> softmax, a compiled program, two GEMMs, W8A8."""
    m, n = bufs["m"], bufs["n"]
    g16 = lambda t, r=m, c=n, dt=kh.F16: dglobal(t, r, c, c, 1, dt)
    kh.elementwise(kh.gelu_program(kh.F16, 0.5), [g16(bufs["x"]), dglobal(bufs["bias"], 1, n, n, 1, kh.F16)], g16(out["gelu"]))
    kh.copy(g16(out["gelu"]), dglobal(out["tr"], n, m, m, 1, kh.F16), transpose=True)
    kh.elementwise(kh.program(kh.softmax_insts(kh.F16)), [dglobal(out["tr"], n, m, m, 1, kh.F16)], dglobal(out["soft"], n, m, m, 1, kh.F16))
    kh.elementwise(bufs["expr"], [g16(bufs["x"]), g16(bufs["y"])], g16(out["expr"]))
    M, N, K = bufs["gemm"]
    kh.matmul(dglobal(bufs["a"], M, K, K, 1, kh.BF16), dglobal(bufs["bt"], K, N, 1, K, kh.BF16), dglobal(out["tn"], M, N, N, 1, kh.BF16))
    kh.matmul(dglobal(bufs["a"], M, K, K, 1, kh.BF16), dglobal(bufs["bt"], K, N, N, 1, kh.BF16), dglobal(out["nn"], M, N, N, 1, kh.BF16))
    for key, rows in (("f8_16", 16), ("f8_256", 256)):
        kh.matmul_scaled_f8(dglobal(bufs["a8"], rows, K, K, 1, kh.F8E4M3), dglobal(bufs["w8"], K, N, 1, K, kh.F8E4M3),
                            bufs["rs"].data_ptr(), bufs["cs"].data_ptr(), dglobal(out[key], rows, N, N, 1, kh.BF16))


def _outputs(bufs):
    m, n = bufs["m"], bufs["n"]
    M, N, K = bufs["gemm"]
    z16 = lambda count: torch.zeros(count, dtype=torch.int16, device="cuda")
    return {"gelu": z16(m * n), "tr": z16(m * n), "soft": z16(m * n), "expr": z16(m * n), "tn": z16(M * N), "nn": z16(M * N),
            "f8_16": z16(16 * N), "f8_256": z16(256 * N)}


def _refill(bufs, seed):
    gen = torch.Generator(device="cuda").manual_seed(seed)
    m, n = bufs["m"], bufs["n"]
    M, N, K = bufs["gemm"]
    bufs["x"].copy_(torch.randn(m * n, generator=gen, device="cuda").half().view(torch.int16))
    bufs["y"].copy_(torch.randn(m * n, generator=gen, device="cuda").half().view(torch.int16))
    bufs["bias"].copy_(torch.randn(n, generator=gen, device="cuda").half().view(torch.int16))
    bufs["a"].copy_((0.05 * torch.randn(M * K, generator=gen, device="cuda")).bfloat16().view(torch.int16))
    bufs["bt"].copy_((0.05 * torch.randn(N * K, generator=gen, device="cuda")).bfloat16().view(torch.int16))
    bufs["a8"].copy_(torch.randn(256 * K, generator=gen, device="cuda").to(torch.float8_e4m3fn).view(torch.uint8))
    bufs["w8"].copy_(torch.randn(N * K, generator=gen, device="cuda").to(torch.float8_e4m3fn).view(torch.uint8))
    bufs["rs"].copy_(torch.rand(256, generator=gen, device="cuda") + 0.5)
    bufs["cs"].copy_(torch.rand(N, generator=gen, device="cuda") + 0.5)


def test_every_kernel_family_replays_from_a_graph():
    if not hasattr(kh, "matmul_scaled_f8"):
        pytest.skip("no W8A8 binding")
    m, n = 96, 512
    M, N, K = 256, 512, 1024
    i16 = lambda count: torch.zeros(count, dtype=torch.int16, device="cuda")
    bufs = {"m": m, "n": n, "gemm": (M, N, K), "x": i16(m * n), "y": i16(m * n), "bias": i16(n), "a": i16(M * K), "bt": i16(N * K),
            "a8": torch.zeros(256 * K, dtype=torch.uint8, device="cuda"), "w8": torch.zeros(N * K, dtype=torch.uint8, device="cuda"),
            "rs": torch.zeros(256, dtype=torch.float32, device="cuda"), "cs": torch.zeros(N, dtype=torch.float32, device="cuda")}
    L, ADD, MUL, ST = kh.EW_LD_GLOBAL, kh.EW_ADDF, kh.EW_MULF, kh.EW_ST_GLOBAL
    bufs["expr"] = kh.program([dict(op=L, dst=0, a=0), dict(op=L, dst=1, a=1), dict(op=MUL, dst=2, a=0, b=1), dict(op=ADD, dst=2, a=2, b=1),
                               dict(op=ADD, dst=2, a=2, b=0), dict(op=ST, a=2)])
    g16 = lambda t: dglobal(t, m, n, n, 1, kh.F16)
    kh.elementwise_specialize(bufs["expr"], [g16(bufs["x"]), g16(bufs["y"])], g16(bufs["x"]))   # compiling loads a module: before the capture
    captured, eager = _outputs(bufs), _outputs(bufs)
    _refill(bufs, 1)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):           # one eager pass first: lazy module loading and attribute calls happen outside the capture
        _calls(bufs, eager)
    torch.cuda.current_stream().wait_stream(side)
    sync()
    launches_before = kh.elementwise_specialize_stats()[1]
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        _calls(bufs, captured)
    # the compiled kernel is part of the graph (more than one, if tests that ran earlier in this process compiled other programs of _calls)
    assert kh.elementwise_specialize_stats()[1] >= launches_before + 1
    for seed in (2, 3, 4):
        _refill(bufs, seed)
        for t in captured.values():
            t.fill_(0x1111)                 # eager work between the replays
        graph.replay()
        _calls(bufs, eager)
        sync()
        for name in captured:
            assert torch.equal(captured[name], eager[name]), "replay with seed %d differs from the eager call in %s" % (seed, name)
        assert int((captured["soft"] != 0x1111).sum()) > 0


def test_matmul_layouts_and_tile_choices_replay_from_a_graph():
    """The matmul kernels behind the layout and tile rules - row-major x row-major on 256-wide tiles, the same with a fused tail, a
    column-major result (the transposed problem), few tiles on 64 x 64 and 128 x 64 tiles - recorded once and replayed with fresh
    operands: every replay has the bits of the eager calls."""
    M, N, K = 3072, 3072, 128
    i16 = lambda count: torch.zeros(count, dtype=torch.int16, device="cuda")
    a, b, bias = i16(M * K), i16(K * N), i16(N)

    def calls(out):
        ga, gb = dglobal(a, M, K, K, 1, kh.BF16), dglobal(b, K, N, N, 1, kh.BF16)
        kh.matmul(ga, gb, dglobal(out["wide"], M, N, N, 1, kh.BF16))
        kh.matmul_fused(ga, gb, dglobal(out["wide_tail"], M, N, N, 1, kh.BF16), bias=dglobal(bias, 1, N, N, 1, kh.BF16), alpha=0.5, act=kh.EW_GELU_TANH)
        # K-contiguous operands cut from the same buffers: [256 x 1024] . [1024 x 384]^T-stored, column-major result
        kh.matmul(dglobal(a, 256, 1024, 1024, 1, kh.BF16), dglobal(b, 1024, 384, 1, 1024, kh.BF16), dglobal(out["col"], 256, 384, 1, 256, kh.BF16))
        kh.matmul(dglobal(a, 64, 1024, 1024, 1, kh.BF16), dglobal(b, 1024, 384, 1, 1024, kh.BF16), dglobal(out["t64"], 64, 384, 384, 1, kh.BF16))
        kh.matmul(dglobal(a, 250, 320, 320, 1, kh.BF16), dglobal(b, 320, 1024, 1, 320, kh.BF16), dglobal(out["t128x64"], 250, 1024, 1024, 1, kh.BF16))

    outputs = lambda: {"wide": i16(M * N), "wide_tail": i16(M * N), "col": i16(256 * 384), "t64": i16(64 * 384), "t128x64": i16(250 * 1024)}

    def refill(seed):
        gen = torch.Generator(device="cuda").manual_seed(seed)
        a.copy_((0.1 * torch.randn(M * K, generator=gen, device="cuda")).bfloat16().view(torch.int16))
        b.copy_((0.1 * torch.randn(K * N, generator=gen, device="cuda")).bfloat16().view(torch.int16))
        bias.copy_(torch.randn(N, generator=gen, device="cuda").bfloat16().view(torch.int16))

    captured, eager = outputs(), outputs()
    refill(1)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):           # one eager pass first: attribute queries happen outside the capture
        calls(eager)
    torch.cuda.current_stream().wait_stream(side)
    sync()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        calls(captured)
    for seed in (2, 3, 4):
        refill(seed)
        for t in captured.values():
            t.fill_(0x1111)
        graph.replay()
        calls(eager)
        sync()
        for name in captured:
            assert torch.equal(captured[name], eager[name]), "replay with seed %d differs from the eager call in %s" % (seed, name)
            assert int((captured[name] != 0x1111).sum()) > captured[name].numel() // 2


def test_nothing_is_compiled_or_loaded_while_a_stream_is_captured():
    """A row program the row machine refuses (a width that is no multiple of 8) is normally served by compiling a kernel on its
    first call.  Inside a capture that must not happen (compiling and loading a module are not stream work): the call is refused
    with a message that says what to do, and the capture stays usable."""
    m, n = 4, 104
    x = (torch.randn(m * n, device="cuda") * 2).half().view(torch.int16)
    soft, copy = torch.zeros(m * n, dtype=torch.int16, device="cuda"), torch.zeros(m * n, dtype=torch.int16, device="cuda")
    prog = kh.program(kh.softmax_insts(kh.F16))
    narrow = lambda t: kh.sv_global(dglobal(t, m, n, n, 1, kh.F16), 0, m, 0, 100)      # rows of 100 that start aligned to 8 elements
    xin = kh.sv_global(dglobal(x, m, n, n, 1, kh.F16), 0, m, 0, 100)
    kh.copy(dglobal(x, m, n, n, 1, kh.F16), dglobal(copy, m, n, n, 1, kh.F16))     # lazy loading of the copy kernel: outside the capture
    copy.zero_()
    sync()
    loaded_before = kh.elementwise_specialize_stats()[0]
    refused = None
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        kh.copy(dglobal(x, m, n, n, 1, kh.F16), dglobal(copy, m, n, n, 1, kh.F16))
        try:
            kh.elementwise(prog, [xin], narrow(soft))
        except kh.KapyError as e:
            refused = e
    assert refused is not None and refused.status == kh.ERR_UNSUPPORTED and "captured" in refused.message
    assert kh.elementwise_specialize_stats()[0] == loaded_before
    graph.replay()
    sync()
    assert torch.equal(copy, x) and int(soft.count_nonzero()) == 0
    # outside a capture the same call compiles its kernel and runs
    kh.elementwise(prog, [xin], narrow(soft))
    sync()
    assert kh.elementwise_specialize_stats()[0] == loaded_before + 1
    sums = soft.view(torch.float16).float().view(m, n)[:, :100].sum(dim=1)
    assert torch.allclose(sums, torch.ones_like(sums), atol=2e-2)
