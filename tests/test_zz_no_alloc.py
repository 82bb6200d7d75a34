"""kapy_matmul_static_workspace: the entry point that allocates nothing (the workspace of a split K is an array inside the
library's device image) against kapy_matmul with a caller-provided workspace: same bits, on two calls in a row, the second
on a smaller problem (the array keeps the first call's partial sums; only the counters must be, and are, back at zero)."""
import numpy as np
import pytest
import torch

import kapy_hip as kh
from gpu_util import dev_zeros, dglobal, sync, to_dev, to_host

pytestmark = pytest.mark.gpu


def _pair(ko, dt, M, N, K, tile, seed, split_k):
    a, b = ko.fill_uniform(M * K, dt, seed, 0), ko.fill_uniform(K * N, dt, seed, 1)
    da, db = to_dev(a), to_dev(b)
    ga, gb = dglobal(da, M, K, K, 1, dt), dglobal(db, K, N, N, 1, dt)
    ws = torch.zeros(kh.lib().kapy_matmul_workspace_bytes(M, N), dtype=torch.uint8, device="cuda")
    d_ws, d_static = dev_zeros(M * N, 2, fill=0x7E7E), dev_zeros(M * N, 2, fill=0x7E7E)
    kh.matmul(ga, gb, dglobal(d_ws, M, N, N, 1, dt), tile=tile, split_k=split_k, workspace=ws)
    kh.matmul(ga, gb, dglobal(d_static, M, N, N, 1, dt), tile=tile, split_k=split_k, static_workspace=True)
    sync()
    d_plain = dev_zeros(M * N, 2)
    kh.matmul(ga, gb, dglobal(d_plain, M, N, N, 1, dt), tile=tile, split_k=1)
    sync()
    return to_host(d_ws, np.uint16), to_host(d_static, np.uint16), to_host(d_plain, np.uint16), (a, b)


def test_static_workspace_equals_caller_workspace_on_two_calls_in_a_row(ko):
    import ctypes as C
    # first call: benchmark configuration 1, 64 tiles split four ways: 16 MiB of partial sums, all of the array
    with_ws, static, plain, (a, b) = _pair(ko, kh.F16, 1024, 1024, 1024, (128, 128, 32), seed=0, split_k=4)
    assert np.array_equal(static, with_ws)
    want = np.zeros(1024 * 1024, np.uint16)
    assert ko.lib().ko_matmul(C.byref(ko.mk_global(a, 1024, 1024, 1024, 1, ko.F16)), C.byref(ko.mk_global(b, 1024, 1024, 1024, 1, ko.F16)), None,
                              C.byref(ko.mk_global(want, 1024, 1024, 1024, 1, ko.F16)), ko.RN) == 0
    g, w = ko.decode(static, ko.F16), ko.decode(want, ko.F16)
    assert np.linalg.norm(g - w) / np.linalg.norm(w) <= 1e-3
    # second call, smaller: 6 tiles, split eight ways where the first call's partial sums still lie
    with_ws2, static2, plain2, _ = _pair(ko, kh.BF16, 384, 256, 2048, (128, 128, 64), seed=3, split_k=8)
    # ... and a third with the library's own choice of split
    with_ws3, static3, _, _ = _pair(ko, kh.F16, 256, 512, 4096, (128, 128, 64), seed=4, split_k=0)
    assert np.array_equal(static3, with_ws3)
    assert np.array_equal(static2, with_ws2)
    gp, gs = ko.decode(plain2, ko.BF16), ko.decode(static2, ko.BF16)
    assert np.linalg.norm(gp - gs) / np.linalg.norm(gp) <= 1e-3     # (the unsplit kernel sums in another order)
    # a split that was asked for and does not fit the array is refused, with the sizes in the message
    d = dev_zeros(2048 * 2048, 2)
    g2 = dglobal(d, 2048, 2048, 2048, 1, kh.F16)
    with pytest.raises(kh.KapyError) as e:
        kh.matmul(g2, g2, g2, tile=(128, 128, 32), split_k=2, static_workspace=True)
    assert e.value.status == kh.ERR_UNSUPPORTED and "workspace" in e.value.message


def test_static_workspace_under_graph_capture_replays_the_eager_bits(ko):
    """The callers this entry point is for: a first eager call on the device (it asks the runtime where the device's copy of the
    array lives), then the same call recorded into a graph; every replay, with eager work of another shape in between that dirties
    the array, gives the eager call's bits."""
    M, N, K, dt = 512, 384, 4096, kh.BF16
    a, b = ko.fill_uniform(M * K, dt, 21, 0), ko.fill_uniform(K * N, dt, 21, 1)
    da, db = to_dev(a), to_dev(b)
    ga, gb = dglobal(da, M, K, K, 1, dt), dglobal(db, K, N, N, 1, dt)
    eager, out = dev_zeros(M * N, 2), dev_zeros(M * N, 2)
    kh.matmul(ga, gb, dglobal(eager, M, N, N, 1, dt), tile=(128, 128, 64), split_k=8, static_workspace=True)
    sync()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            kh.matmul(ga, gb, dglobal(out, M, N, N, 1, dt), tile=(128, 128, 64), split_k=8, static_workspace=True, stream=side.cuda_stream)
    other = dev_zeros(256 * 256, 2)
    g_small = dglobal(to_dev(ko.fill_uniform(256 * 2048, kh.F16, 5, 0)), 256, 2048, 2048, 1, kh.F16)
    g_small_b = dglobal(to_dev(ko.fill_uniform(2048 * 256, kh.F16, 5, 1)), 2048, 256, 256, 1, kh.F16)
    for rep in range(3):
        out.fill_(0x7E7E)
        sync()
        graph.replay()
        sync()
        assert torch.equal(out, eager), rep
        kh.matmul(g_small, g_small_b, dglobal(other, 256, 256, 256, 1, kh.F16), tile=(128, 128, 64), split_k=4, static_workspace=True)
        sync()


def test_static_workspace_calls_leave_the_device_memory_as_it_was(ko):
    """After a first call (the runtime loads the kernels' code on first use), calls through the entry point change nothing
    about how much device memory is free: nothing is allocated and nothing released."""
    M, N, K, dt = 256, 384, 4096, kh.F16
    da, db = to_dev(ko.fill_uniform(M * K, dt, 7, 0)), to_dev(ko.fill_uniform(K * N, dt, 7, 1))
    ga, gb = dglobal(da, M, K, K, 1, dt), dglobal(db, K, N, N, 1, dt)
    out = dev_zeros(M * N, 2)
    go = dglobal(out, M, N, N, 1, dt)
    for split in (8, 0):
        kh.matmul(ga, gb, go, tile=(128, 128, 64), split_k=split, static_workspace=True)
    sync()
    free_before = torch.cuda.mem_get_info()[0]
    for rep in range(20):
        kh.matmul(ga, gb, go, tile=(128, 128, 64), split_k=8 if rep % 2 else 0, static_workspace=True)
    sync()
    assert torch.cuda.mem_get_info()[0] == free_before
