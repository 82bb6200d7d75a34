"""kapy_matmul with accumulate = KAPY_ACCUMULATE_ELEMENT: f16 accumulators rounded once per instruction of 8 or 16 lhs columns, the
arithmetic of the reference's f16-result instruction (MatmulOpToLLVM.cpp:270-291), against the checker's restatement and the
hand-computed answers that pin it; and the reference fixture's matmul program run in that arithmetic through the front-end."""
import ctypes as C

import numpy as np
import pytest

import kapy_hip as kh
import kapy_programs as kp
from gpu_util import dev_zeros, dglobal, sync, to_dev, to_host

pytestmark = pytest.mark.gpu


def _gpu(a, b, acc, way, col_major_b=False):
    m, k = a.shape
    n = b.shape[1]
    da = to_dev(np.ascontiguousarray(a).view(np.uint16))
    if col_major_b:
        db, gb = to_dev(np.ascontiguousarray(b.T).view(np.uint16)), None
        gb = dglobal(db, k, n, 1, k, kh.F16)
    else:
        db = to_dev(np.ascontiguousarray(b).view(np.uint16))
        gb = dglobal(db, k, n, n, 1, kh.F16)
    dd = dev_zeros(m * n + 64, 2, fill=0x1234)
    dc = to_dev(np.ascontiguousarray(acc).view(np.uint16)) if acc is not None else None
    kh.matmul(dglobal(da, m, k, k, 1, kh.F16), gb, dglobal(dd, m, n, n, 1, kh.F16), acc=dglobal(dc, m, n, n, 1, kh.F16) if dc is not None else None,
              impl_way=way, accumulate=kh.ACCUMULATE_ELEMENT)
    sync()
    got = to_host(dd, np.uint16)
    assert np.all(got[m * n:] == 0x1234)
    return got[:m * n].reshape(m, n).view(np.float16)


def _oracle(ko, a, b, acc, k_step):
    m, k = a.shape
    n = b.shape[1]
    out = np.zeros((m, n), np.uint16)
    gc = ko.mk_global(np.ascontiguousarray(acc).view(np.uint16), m, n, n, 1, ko.F16) if acc is not None else None
    assert ko.lib().ko_matmul_f16acc(C.byref(ko.mk_global(np.ascontiguousarray(a).view(np.uint16), m, k, k, 1, ko.F16)),
                                     C.byref(ko.mk_global(np.ascontiguousarray(b).view(np.uint16), k, n, n, 1, ko.F16)),
                                     C.byref(gc) if gc is not None else None, C.byref(ko.mk_global(out, m, n, n, 1, ko.F16)), k_step) == 0
    return out.view(np.float16)


def test_known_answers_on_the_device():
    """The cases that pin the checker, with integers that fp32 adds exactly inside a step: the device must give the same numbers."""
    a, b = np.ones((16, 40000), np.float16), np.ones((40000, 16), np.float16)
    assert np.all(_gpu(a, b, None, kh.MMA_M16N8K16_F16) == 32768.0)
    assert np.all(_gpu(a, b, None, kh.MMA_M16N8K8_F16) == 16384.0)
    a = np.zeros((16, 32), np.float16)
    a[:, 0], a[:, 1], a[:, 8], a[:, 16] = 2048, 1, 1, 1
    b = np.ones((32, 16), np.float16)
    assert np.all(_gpu(a, b, None, kh.MMA_M16N8K8_F16) == 2048.0)
    assert np.all(_gpu(a, b, None, kh.MMA_M16N8K16_F16) == 2052.0)
    ones = np.zeros((16, 48), np.float16)
    ones[:, ::16] = 1
    assert np.all(_gpu(ones, np.ones((48, 16), np.float16), np.full((16, 16), 2048, np.float16), kh.MMA_M16N8K16_F16) == 2048.0)


@pytest.mark.parametrize("way,k_step", [(kh.MMA_M16N8K8_F16, 8), (kh.MMA_M16N8K16_F16, 16), (kh.MATMUL_AUTO, 16)])
@pytest.mark.parametrize("m,n,k,col_major_b", [(16, 16, 16, False), (64, 64, 256, False), (33, 20, 100, True), (130, 75, 1000, False), (16, 8, 4096, True)])
def test_against_the_checker(ko, way, k_step, m, n, k, col_major_b):
    """Inside a step the matrix unit adds in fp32 where the checker adds exactly, so a sum within fp32 round-off of an f16 tie may
    land one f16 unit away - and, carried along, move later roundings: nearly every element equal, the rest within the f16
    spacing of the largest partial sum, the whole within 1e-3 (tolerance of this test: relative Frobenius distance)."""
    rng = np.random.default_rng(m + n + k)
    a, b = rng.standard_normal((m, k)).astype(np.float16), rng.standard_normal((k, n)).astype(np.float16)
    acc = rng.standard_normal((m, n)).astype(np.float16)
    got, want = _gpu(a, b, acc, way, col_major_b).astype(np.float64), _oracle(ko, a, b, acc, k_step).astype(np.float64)
    assert np.mean(got != want) <= 0.02
    assert np.linalg.norm(got - want) / np.linalg.norm(want) <= 1e-3
    # and it is not the fp32-accumulate product: over a long K the two differ by far more than that
    if k >= 1000:
        da, db, dd = to_dev(np.ascontiguousarray(a).view(np.uint16)), to_dev(np.ascontiguousarray(b).view(np.uint16)), dev_zeros(m * n, 2)
        kh.matmul(dglobal(da, m, k, k, 1, kh.F16), dglobal(db, k, n, n, 1, kh.F16), dglobal(dd, m, n, n, 1, kh.F16),
                  acc=dglobal(to_dev(np.ascontiguousarray(acc).view(np.uint16)), m, n, n, 1, kh.F16))
        sync()
        wide = to_host(dd, np.uint16, (m, n)).view(np.float16).astype(np.float64)
        assert np.mean(wide != want) > 0.2


def test_refusals():
    d = dev_zeros(64 * 64, 2)
    g16, gbf = dglobal(d, 64, 64, 64, 1, kh.F16), dglobal(d, 64, 64, 64, 1, kh.BF16)
    with pytest.raises(kh.KapyError) as e:
        kh.matmul(gbf, gbf, gbf, accumulate=kh.ACCUMULATE_ELEMENT)
    assert e.value.status == kh.ERR_UNSUPPORTED and "f16" in e.value.message
    with pytest.raises(kh.KapyError) as e:
        kh.matmul(g16, g16, g16, accumulate=7)
    assert e.value.status == kh.ERR_INVALID
    with pytest.raises(kh.KapyError):
        kh.matmul(g16, g16, g16, accumulate=kh.ACCUMULATE_ELEMENT, rmode=kh.RZ)


def test_the_fixture_shaped_program_in_the_reference_arithmetic(ko, monkeypatch):
    """test/Conversion/KapyToKgpu/matmul.mlir's tiling (64 x 64 x 16 per warp, mma_m16n8k8_f16, f16 accumulator carried through the
    K loop) with KAPY_MLIR_MATMUL=reference: every kapy.matmul rounds its f16 accumulator once per 8 columns, so the whole program
    is the checker's f16-accumulate product with k_step = 8 over the whole K."""
    monkeypatch.setenv("KAPY_MLIR_MATMUL", "reference")
    M, N, K, bm, bn, bk = 256, 128, 256, 64, 64, 16
    a, b = ko.fill_normal(M * K, ko.F16, 31, std=0.5), ko.fill_normal(K * N, ko.F16, 32, std=0.5)
    da, db, dc = to_dev(a), to_dev(b), dev_zeros(M * N, 2, fill=-1)
    kh.run_mlir(kp.matmul_program(bm, bn, bk, "mma_m16n8k8_f16", "f16"), [da, db, dc, M, N, K], [(M // (2 * bm)) * (N // (2 * bn))])
    sync()
    got = to_host(dc, np.float16, (M, N)).astype(np.float64)
    want = _oracle(ko, a.view(np.float16).reshape(M, K), b.view(np.float16).reshape(K, N), None, 8).astype(np.float64)
    assert np.mean(got != want) <= 0.02
    assert np.linalg.norm(got - want) / np.linalg.norm(want) <= 1e-3
    monkeypatch.delenv("KAPY_MLIR_MATMUL")
    dc2 = dev_zeros(M * N, 2, fill=-1)
    kh.run_mlir(kp.matmul_program(bm, bn, bk, "mma_m16n8k8_f16", "f16"), [da, db, dc2, M, N, K], [(M // (2 * bm)) * (N // (2 * bn))])
    sync()
    assert np.mean(to_host(dc2, np.float16, (M, N)).astype(np.float64) != want) > 0.05     # (one rounding per 16 columns by default)
