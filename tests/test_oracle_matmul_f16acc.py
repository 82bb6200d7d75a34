"""Pins the checker's f16-accumulate matmul (the arithmetic of the reference's f16-result instruction, MatmulOpToLLVM.cpp:270-291:
the running sum is an f16 register, rounded once per instruction of 8 or 16 lhs columns) by hand-computed answers in which the
cadence of the roundings decides the result, and by an independent numpy float16 walk."""
import ctypes as C

import numpy as np
import pytest


def _run(ko, a, b, acc, k_step, wide=False):
    m, k = a.shape
    n = b.shape[1]
    out = np.zeros((m, n), np.uint16)
    ga, gb = ko.mk_global(np.ascontiguousarray(a).view(np.uint16), m, k, k, 1, ko.F16), ko.mk_global(np.ascontiguousarray(b).view(np.uint16), k, n, n, 1, ko.F16)
    gc = ko.mk_global(np.ascontiguousarray(acc).view(np.uint16), m, n, n, 1, ko.F16) if acc is not None else None
    go = ko.mk_global(out, m, n, n, 1, ko.F16)
    if wide:
        assert ko.lib().ko_matmul(C.byref(ga), C.byref(gb), C.byref(gc) if gc is not None else None, C.byref(go), ko.RN) == 0
    else:
        assert ko.lib().ko_matmul_f16acc(C.byref(ga), C.byref(gb), C.byref(gc) if gc is not None else None, C.byref(go), k_step) == 0
    return out.view(np.float16)


def test_a_long_sum_of_ones_stalls_where_half_a_step_is_half_a_unit(ko):
    """40000 products of 1 x 1.  With 16 per step the f16 sum climbs exactly to 32768, where f16 values are 32 apart: 32768 + 16
    is a tie and goes to the even 32768, for ever.  With 8 per step the same happens at 16384 (16 apart).  One rounding at the
    end gives 40000 (= 1250 x 32, an f16 value)."""
    a, b = np.ones((1, 40000), np.float16), np.ones((40000, 1), np.float16)
    assert _run(ko, a, b, None, 16)[0, 0] == 32768.0
    assert _run(ko, a, b, None, 8)[0, 0] == 16384.0
    assert _run(ko, a, b, None, 0, wide=True)[0, 0] == 40000.0


def test_where_the_steps_end_decides_the_ties(ko):
    """lhs row: 2048 at column 0, ones at columns 1, 8 and 16, zeros elsewhere (K = 32), rhs all ones.  f16 values from 2048 on
    are 2 apart.  8 per step: 2048 + 1 = 2049 -> 2048 (tie to even), + 1 -> 2048, + 1 -> 2048.  16 per step: 2048 + 1 + 1 = 2050;
    2050 + 1 = 2051 -> 2052 (tie; 2050 = 1025 x 2 is odd).  One rounding: 2051 -> 2052."""
    a = np.zeros((1, 32), np.float16)
    a[0, 0], a[0, 1], a[0, 8], a[0, 16] = 2048, 1, 1, 1
    b = np.ones((32, 1), np.float16)
    assert _run(ko, a, b, None, 8)[0, 0] == 2048.0
    assert _run(ko, a, b, None, 16)[0, 0] == 2052.0
    assert _run(ko, a, b, None, 0, wide=True)[0, 0] == 2052.0
    # the accumulator operand is the register's first value: 2048 in, one product of 1 per step -> every step a lost tie
    ones = np.zeros((1, 48), np.float16)
    ones[0, ::16] = 1
    assert _run(ko, ones, np.ones((48, 1), np.float16), np.full((1, 1), 2048, np.float16), 16)[0, 0] == 2048.0
    assert _run(ko, ones, np.ones((48, 1), np.float16), np.full((1, 1), 2048, np.float16), 0, wide=True)[0, 0] == 2052.0   # 2051 -> 2052


@pytest.mark.parametrize("k_step", [8, 16])
@pytest.mark.parametrize("m,n,k", [(5, 7, 16), (16, 16, 72), (3, 9, 100), (33, 20, 256)])
def test_against_a_numpy_float16_walk(ko, m, n, k, k_step):
    rng = np.random.default_rng(m * 100 + k)
    a, b = rng.standard_normal((m, k)).astype(np.float16), rng.standard_normal((k, n)).astype(np.float16)
    acc = rng.standard_normal((m, n)).astype(np.float16)
    held = acc.copy()
    for k0 in range(0, k, k_step):
        held = (held.astype(np.float64) + a[:, k0:k0 + k_step].astype(np.float64) @ b[k0:k0 + k_step].astype(np.float64)).astype(np.float16)
    assert np.array_equal(_run(ko, a, b, acc, k_step), held)


def test_refusals(ko):
    a = np.zeros((16, 16), np.uint16)
    g16, gbf, out = ko.mk_global(a, 16, 16, 16, 1, ko.F16), ko.mk_global(a, 16, 16, 16, 1, ko.BF16), ko.mk_global(a.copy(), 16, 16, 16, 1, ko.F16)
    assert ko.lib().ko_matmul_f16acc(C.byref(gbf), C.byref(gbf), None, C.byref(out), 16) != 0      # bf16 operands have no f16-accumulate instruction
    assert ko.lib().ko_matmul_f16acc(C.byref(g16), C.byref(g16), None, C.byref(out), 4) != 0        # no instruction of 4 columns
