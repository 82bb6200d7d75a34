"""Seeded random instances of the programs the hand-written kernels match - act(x*s + bias) with every activation, bias
kind, type, width (ragged ones too) and row pitch, plain binary programs - and of the row programs (softmax, layer norm,
RMS norm over random shapes, pitches and ragged widths, through the default path and compiled): <= 2 ulp of the 16-bit
result against the oracle (an absolute floor where a norm's gamma*xhat + beta cancels)."""
import numpy as np
import pytest

import kapy_hip as kh
from gpu_util import dglobal, sync, to_dev, to_host
from test_gpu_elementwise import _check_ulp
from test_gpu_specialize import _check_ulp_away_from_cancellation

pytestmark = pytest.mark.gpu
L, ADD, MUL, ST, CAST, SPL = kh.EW_LD_GLOBAL, kh.EW_ADDF, kh.EW_MULF, kh.EW_ST_GLOBAL, kh.EW_FPTOFP, kh.EW_SPLAT
ACTS = [-1, kh.EW_GELU_TANH, kh.EW_NEGF, kh.EW_ABSF, kh.EW_EXP, kh.EW_EXP2, kh.EW_TANH, kh.EW_ERF, kh.EW_SQRT, kh.EW_RSQRT, kh.EW_LOG, kh.EW_LOG2]


def _run(ko, insts, views, out_view, dt, m, width, check):
    """views: per operand (array, rows, cols, pitch); out_view: (pitch).  Everything else in the buffers must stay as it was."""
    o_ins = [ko.mk_global(a, r, c, p, 1, dt) for a, r, c, p in views]
    devs = [to_dev(a) for a, _, _, _ in views]
    d_ins = [dglobal(t, r, c, p, 1, dt) for t, (_, r, c, p) in zip(devs, views)]
    pitch = out_view
    want = np.full(m * pitch, 0x5a5a, np.uint16)
    assert ko.elementwise(ko.program(insts), o_ins, ko.mk_global(want, m, width, pitch, 1, dt)) == 0
    dout = to_dev(np.full(m * pitch, 0x5a5a, np.uint16))
    kh.elementwise(kh.program(insts), d_ins, dglobal(dout, m, width, pitch, 1, dt))
    sync()
    got, want = to_host(dout, np.uint16, (m, pitch)), want.reshape(m, pitch)
    assert np.array_equal(got[:, width:], want[:, width:]), "written outside the view"
    check(np.ascontiguousarray(got[:, :width]), np.ascontiguousarray(want[:, :width]), dt)
    return dout, d_ins


@pytest.mark.parametrize("seed", list(range(60)) + [130, 167])
def test_random_affine_activation(ko, seed):
    rng = np.random.RandomState(9000 + seed)
    dt = [kh.F16, kh.BF16][rng.randint(2)]
    m = [1, 7, 33, 64, 200][rng.randint(5)]
    width = [8, 24, 100, 256, 1001, 1000, 4096, 37][rng.randint(8)]
    pitch = (width + 7) // 8 * 8 + [0, 8, 64][rng.randint(3)] if rng.randint(4) else width      # (an unaligned pitch takes the interpreter)
    act = ACTS[rng.randint(len(ACTS))]
    bias_kind = ["none", "row", "full", "col"][rng.randint(4)]
    scale = [None, 0.5, -1.25, 3.0][rng.randint(4)]
    positive = act in (kh.EW_SQRT, kh.EW_RSQRT, kh.EW_LOG, kh.EW_LOG2)
    x = ko.fill_uniform(m * pitch, dt, seed, 0, 0.25, 4.0) if positive else ko.fill_normal(m * pitch, dt, seed, 0, 0.0, 1.5)
    insts = [dict(op=L, dst=0, a=0), dict(op=CAST, dst=0, a=0, dtype=kh.F32)]
    views = [(x, m, width, pitch)]
    if scale is not None and not (positive and scale < 0):
        insts += [dict(op=SPL, dst=1, dtype=kh.F32, imm=scale), dict(op=MUL, dst=0, a=0, b=1)]
    if bias_kind != "none":
        shape = {"row": (1, width, pitch), "full": (m, width, pitch), "col": (m, 1, 1)}[bias_kind]
        b = ko.fill_uniform(shape[0] * shape[2], dt, seed, 1, 0.0, 1.0)
        views.append((b, shape[0], shape[1], shape[2]))
        insts += [dict(op=L, dst=2, a=1), dict(op=CAST, dst=2, a=2, dtype=kh.F32), dict(op=ADD, dst=0, a=0, b=2)]
    if act >= 0:
        insts += [dict(op=act, dst=0, a=0)]
    insts += [dict(op=CAST, dst=3, a=0, dtype=dt, rmode=kh.RN), dict(op=ST, a=3)]
    # (a GELU result below fp32's normal range - gelu(-12) ~ 1e-38, representable in bf16 - comes out of rcp / exp2 flushed: an
    # absolute error of 1e-30 passes as well)
    _run(ko, insts, views, pitch, dt, m, width, lambda g, w, d: _check_ulp_away_from_cancellation(g, w, d, floor=1e-30))


@pytest.mark.parametrize("seed", range(40))
def test_random_row_program(ko, seed):
    rng = np.random.RandomState(9500 + seed)
    dt = [kh.F16, kh.BF16][rng.randint(2)]
    m = [1, 5, 37, 300][rng.randint(4)]
    width = [8, 64, 200, 1000, 1024, 2048, 4096, 5000, 8192, 100, 1001][rng.randint(11)]
    pitch = (width + 7) // 8 * 8 + [0, 8][rng.randint(2)]
    which = rng.randint(4)
    x = ko.fill_normal(m * pitch, dt, seed, 0, 0.0, 2.0)
    views = [(x, m, width, pitch)]
    if which == 0:
        insts, check = kh.softmax_insts(dt), _check_ulp
    elif which == 1:
        insts, check = kh.layernorm_insts(width, dt), _check_ulp_away_from_cancellation
        views += [(ko.fill_normal(pitch, dt, seed, 1, 1.0, 0.5), 1, width, pitch), (ko.fill_normal(pitch, dt, seed, 2, 0.0, 0.5), 1, width, pitch)]
    elif which == 2:
        insts, check = kh.rmsnorm_insts(width, dt), _check_ulp
        views += [(ko.fill_normal(pitch, dt, seed, 1, 1.0, 0.5), 1, width, pitch)]
    else:
        insts, check = kh.layernorm_insts(width, dt, affine=False), _check_ulp
    dout, d_ins = _run(ko, insts, views, pitch, dt, m, width, check)      # the default path (a ragged width compiles by itself)
    prog = kh.program(insts)
    kh.elementwise_specialize(prog, d_ins, dglobal(dout, m, width, pitch, 1, dt))
    before = kh.elementwise_specialize_stats()[1]
    _run(ko, insts, views, pitch, dt, m, width, check)
    assert kh.elementwise_specialize_stats()[1] == before + 1
