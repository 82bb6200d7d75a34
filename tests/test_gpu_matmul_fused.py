"""GPU parity for kapy_matmul_fused: the elementwise tail (mulf by a splat, addf of a broadcast bias row, an activation,
the cast) in the GEMM's epilogue, against the oracle's matmul (fp64 accumulate, fp32 result) followed by the oracle's
elementwise program: relative Frobenius error <= 1e-3; and against the same two steps run separately on the device
(same kernel, same accumulation order): <= 2 ulp of the 16-bit result."""
import ctypes as C

import numpy as np
import pytest

import kapy_hip as kh
from gpu_util import dev_zeros, dglobal, sync, to_dev, to_host, ulp_diff_f16

pytestmark = pytest.mark.gpu
L, ADD, MUL, MAX, MIN, ST, CAST, SPL = (kh.EW_LD_GLOBAL, kh.EW_ADDF, kh.EW_MULF, kh.EW_MAXIMUMF, kh.EW_MINIMUMF, kh.EW_ST_GLOBAL, kh.EW_FPTOFP, kh.EW_SPLAT)


def _tail_program(dt, bias_dt, alpha, act, operand):
    """The tail as a kapy program over the fp32 matmul result (input 0) and the bias row (input 1)."""
    insts = [dict(op=L, dst=0, a=0)]
    if alpha != 1.0:
        insts += [dict(op=SPL, dst=1, dtype=kh.F32, imm=alpha), dict(op=MUL, dst=0, a=0, b=1)]
    if bias_dt is not None:
        insts += [dict(op=L, dst=2, a=1)] + ([dict(op=CAST, dst=2, a=2, dtype=kh.F32)] if bias_dt != kh.F32 else []) + [dict(op=ADD, dst=0, a=0, b=2)]
    if act in (MAX, MIN):
        insts += [dict(op=SPL, dst=3, dtype=kh.F32, imm=operand), dict(op=act, dst=0, a=0, b=3)]
    elif act >= 0:
        insts += [dict(op=act, dst=0, a=0)]
    return insts + [dict(op=CAST, dst=4, a=0, dtype=dt, rmode=kh.RN), dict(op=ST, a=4)]


def _case(ko, dt, M, N, K, b_row_major, bias_dt, alpha, act, operand=0.0, tile=(0, 0, 0)):
    a, b = ko.fill_normal(M * K, dt, 7, 0, 0.0, 0.25), ko.fill_normal(K * N, dt, 7, 1, 0.0, 0.25)
    b_str = (N, 1) if b_row_major else (1, K)
    bias = ko.fill_normal(N, bias_dt, 7, 2, 0.0, 1.0) if bias_dt is not None else None
    # oracle: matmul into fp32, then the tail program
    c32 = np.zeros(M * N, np.float32)
    assert ko.lib().ko_matmul(C.byref(ko.mk_global(a, M, K, K, 1, dt)), C.byref(ko.mk_global(b, K, N, *b_str, dt)), None,
                              C.byref(ko.mk_global(c32, M, N, N, 1, kh.F32)), kh.RN) == 0
    want = np.zeros(M * N, np.uint16)
    insts = _tail_program(dt, bias_dt, alpha, act, operand)
    o_ins = [ko.mk_global(c32.view(np.uint32), M, N, N, 1, kh.F32)] + ([ko.mk_global(bias, 1, N, N, 1, bias_dt)] if bias is not None else [])
    assert ko.elementwise(ko.program(insts), o_ins, ko.mk_global(want, M, N, N, 1, dt)) == 0
    # device, fused
    da, db, dd = to_dev(a), to_dev(b), dev_zeros(M * N, 2)
    dbias = to_dev(bias) if bias is not None else None
    gb = dglobal(dbias, 1, N, N, 1, bias_dt) if bias is not None else None
    kh.matmul_fused(dglobal(da, M, K, K, 1, dt), dglobal(db, K, N, *b_str, dt), dglobal(dd, M, N, N, 1, dt), bias=gb, alpha=alpha, act=act,
                    act_operand=operand, tile=tile)
    # device, in two steps
    d32, d2 = dev_zeros(M * N, 4), dev_zeros(M * N, 2)
    kh.matmul(dglobal(da, M, K, K, 1, dt), dglobal(db, K, N, *b_str, dt), dglobal(d32, M, N, N, 1, kh.F32), tile=tile)
    kh.elementwise(kh.program(insts), [dglobal(d32, M, N, N, 1, kh.F32)] + ([gb] if gb is not None else []), dglobal(d2, M, N, N, 1, dt))
    sync()
    got, two_step = to_host(dd, np.uint16), to_host(d2, np.uint16)
    g, w = ko.decode(got, dt), ko.decode(want, dt)
    assert np.all(np.isfinite(g))
    rel = np.linalg.norm(g - w) / max(np.linalg.norm(w), 1e-30)
    assert rel <= 1e-3, "relative Frobenius error %g" % rel
    assert ulp_diff_f16(got, two_step).max() <= 2
    return got, want


@pytest.mark.parametrize("dt", [kh.BF16, kh.F16])
@pytest.mark.parametrize("act,operand", [(-1, 0.0), (kh.EW_GELU_TANH, 0.0), (MAX, 0.0), (MIN, 0.25), (kh.EW_NEGF, 0.0), (kh.EW_ABSF, 0.0)])
def test_bias_scale_activation_on_the_ring_kernel(ko, dt, act, operand):
    _case(ko, dt, 512, 512, 256, False, dt, 0.5, act, operand)


@pytest.mark.parametrize("M,N,K,b_row_major,tile", [(256, 256, 128, True, (0, 0, 0)),     # row-major x row-major: the transposing-read kernel
                                                    (300, 264, 200, False, (0, 0, 0)),    # ragged extents on the ring kernel (bounded packed epilogue)
                                                    (256, 512, 256, False, (256, 256, 64)),
                                                    (100, 52, 72, False, (0, 0, 0)),      # rows of the result not 16-byte aligned: element stores
                                                    (96, 200, 64, True, (0, 0, 0))])      # the general kernel
def test_every_epilogue_path_carries_the_tail(ko, M, N, K, b_row_major, tile):
    _case(ko, kh.BF16, M, N, K, b_row_major, kh.BF16, 1.0, kh.EW_GELU_TANH, tile=tile)
    _case(ko, kh.F16, M, N, K, b_row_major, kh.F32, 2.0, MAX, 0.0, tile=tile)


@pytest.mark.parametrize("dt,bias_dt,alpha,act", [(kh.BF16, kh.BF16, 1.0, kh.EW_GELU_TANH), (kh.F16, kh.F32, 0.5, MAX), (kh.BF16, None, 2.0, -1)])
def test_the_tail_on_256_wide_tiles_of_row_major_operands(ko, dt, bias_dt, alpha, act):
    """Large row-major x row-major with a tail: the 256-wide kernel's build with the tail in its strip epilogue.  Against the
    128-wide kernel (which applies the tail in its element stores; same accumulation order) <= 2 ulp, and sampled 64 x 64 blocks
    against the checker's matmul + tail program."""
    M, N, K = 3072, 3072, 192
    a, b = ko.fill_normal(M * K, dt, 9, 0, 0.0, 0.25), ko.fill_normal(K * N, dt, 9, 1, 0.0, 0.25)
    bias = ko.fill_normal(N, bias_dt, 9, 2, 0.0, 1.0) if bias_dt is not None else None
    da, db = to_dev(a), to_dev(b)
    dbias = to_dev(bias) if bias is not None else None
    gb = dglobal(dbias, 1, N, N, 1, bias_dt) if bias is not None else None
    outs = []
    for tile in ((0, 0, 0), (128, 128, 64)):
        dd = dev_zeros(M * N + 64, 2, fill=0x1234)
        kh.matmul_fused(dglobal(da, M, K, K, 1, dt), dglobal(db, K, N, N, 1, dt), dglobal(dd, M, N, N, 1, dt), bias=gb, alpha=alpha, act=act,
                        act_operand=0.0, tile=tile)
        sync()
        got = to_host(dd, np.uint16)
        assert np.all(got[M * N:] == 0x1234)
        outs.append(got[:M * N].reshape(M, N))
    assert np.all(np.isfinite(ko.decode(outs[0].ravel(), dt)))
    assert ulp_diff_f16(outs[0].ravel(), outs[1].ravel()).max() <= 2
    insts = _tail_program(dt, bias_dt, alpha, act, 0.0)
    goa, gob = ko.mk_global(a, M, K, K, 1, dt), ko.mk_global(b, K, N, N, 1, dt)
    for t in range(6):
        r0, c0 = (t * 331 + 37 * (t % 4) * 16) % (M - 64), ((t * 577 + 128 * (t % 2)) % (N - 64)) // 8 * 8
        c32 = np.zeros(64 * 64, np.float32)
        assert ko.lib().ko_matmul(C.byref(ko.sv_global(goa, r0, r0 + 64, 0, K)), C.byref(ko.sv_global(gob, 0, K, c0, c0 + 64)), None,
                                  C.byref(ko.mk_global(c32, 64, 64, 64, 1, kh.F32)), kh.RN) == 0
        want = np.zeros(64 * 64, np.uint16)
        o_ins = [ko.mk_global(c32.view(np.uint32), 64, 64, 64, 1, kh.F32)]
        if bias is not None:
            piece = np.ascontiguousarray(bias[c0:c0 + 64])
            o_ins.append(ko.mk_global(piece, 1, 64, 64, 1, bias_dt))
        assert ko.elementwise(ko.program(insts), o_ins, ko.mk_global(want, 64, 64, 64, 1, dt)) == 0
        g, w = ko.decode(np.ascontiguousarray(outs[0][r0:r0 + 64, c0:c0 + 64]).ravel(), dt), ko.decode(want, dt)
        rel = np.linalg.norm(g - w) / max(np.linalg.norm(w), 1e-30)
        assert rel <= 1e-3, (t, rel)


@pytest.mark.parametrize("with_bias", [False, True])
def test_a_column_major_result_carries_the_tail(ko, with_bias):
    """Scale and activation commute with the transposition, so a column-major result without a bias is the transposed problem
    (bit for bit the row-major result); with a bias row the call stays as it is and goes through the element stores."""
    dt, M, N, K = kh.BF16, 320, 264, 192
    a, b = ko.fill_normal(M * K, dt, 7, 0, 0.0, 0.25), ko.fill_normal(K * N, dt, 7, 1, 0.0, 0.25)
    bias = ko.fill_normal(N, dt, 7, 2, 0.0, 1.0)   # (the operands of _case)
    da, db, dbias = to_dev(a), to_dev(b), to_dev(bias)
    gb = dglobal(dbias, 1, N, N, 1, dt) if with_bias else None
    d_col, d_row = dev_zeros(M * N + 64, 2, fill=0x1234), dev_zeros(M * N, 2)
    for dd, strides in ((d_col, (1, M)), (d_row, (N, 1))):
        kh.matmul_fused(dglobal(da, M, K, K, 1, dt), dglobal(db, K, N, 1, K, dt), dglobal(dd, M, N, *strides, dt), bias=gb, alpha=0.5, act=kh.EW_GELU_TANH)
    sync()
    col = to_host(d_col, np.uint16)
    assert np.all(col[M * N:] == 0x1234)
    col_as_rows = np.ascontiguousarray(col[:M * N].reshape(N, M).T).ravel()
    row = to_host(d_row, np.uint16)
    assert np.all(np.isfinite(ko.decode(col_as_rows, dt)))
    if with_bias:
        assert ulp_diff_f16(col_as_rows, row).max() <= 2
    else:
        assert np.array_equal(col_as_rows, row)
    got_row, want = _case(ko, dt, M, N, K, False, dt if with_bias else None, 0.5, kh.EW_GELU_TANH)
    assert np.array_equal(got_row, row)


def test_parts_of_the_tail_alone_and_relu_really_clamps(ko):
    _case(ko, kh.BF16, 256, 256, 128, False, None, 0.125, -1)                  # scale only
    _case(ko, kh.BF16, 256, 256, 128, False, kh.BF16, 1.0, -1)                 # bias only
    got, want = _case(ko, kh.F16, 256, 256, 128, False, None, 1.0, MAX, 0.0)   # relu only
    assert (got.view(np.float16) >= 0).all() and (got.view(np.float16) == 0).mean() > 0.3


def test_refusals(ko):
    M = N = K = 128
    a = to_dev(ko.fill_normal(M * K, kh.BF16, 1))
    g = lambda r, c: dglobal(a, r, c, c, 1, kh.BF16)
    with pytest.raises(kh.KapyError) as e:
        kh.matmul_fused(g(M, K), g(K, N), g(M, N), act=kh.EW_TANH)
    assert e.value.status == kh.ERR_UNSUPPORTED
    with pytest.raises(kh.KapyError) as e:
        kh.matmul_fused(g(M, K), g(K, N), g(M, N), act=kh.EW_ADDF)
    assert e.value.status == kh.ERR_INVALID
    with pytest.raises(kh.KapyError) as e:
        kh.matmul_fused(g(M, K), g(K, N), g(M, N), bias=g(1, N // 2))
    assert e.value.status == kh.ERR_VERIFY and "broadcast" in e.value.message
