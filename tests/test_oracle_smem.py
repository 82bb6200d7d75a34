"""The shared-memory planner and the barrier analysis: the oracle (oracle/ko_smem.py) against closed forms,
invariants and brute force, and the library's kapy_smem_plan / kapy_smem_barriers against the oracle."""
import ctypes as C
import itertools
import random

import pytest

import kapy_hip as kh
import ko_smem


def _check_plan(buffers, offsets, total, alignment):
    for (s, a, b), o in zip(buffers, offsets):
        assert o % alignment == 0 and o >= 0
    for i, j in itertools.combinations(range(len(buffers)), 2):
        (si, ai, bi), (sj, aj, bj) = buffers[i], buffers[j]
        if ai < bj and aj < bi:                               # live together: bytes must be disjoint
            assert not (offsets[i] < offsets[j] + sj and offsets[j] < offsets[i] + si), (i, j, buffers, offsets)
    assert total == max([o + s for (s, _, _), o in zip(buffers, offsets)], default=0)
    times = sorted({t for _, a, b in buffers for t in (a, b)})
    lower = max([sum(s for s, a, b in buffers if a <= t < b) for t in times], default=0)
    assert total >= lower


def _lib_plan(buffers, alignment):
    arr = (kh.SmemBuffer * max(len(buffers), 1))()
    for k, (s, a, b) in enumerate(buffers):
        arr[k].size, arr[k].live_start, arr[k].live_end, arr[k].offset = s, a, b, -7
    total = kh.lib().kapy_smem_plan(arr, len(buffers), alignment)
    assert total >= 0, kh.last_error()
    return [arr[k].offset for k in range(len(buffers))], total


def test_plan_closed_forms():
    sizes = [16384, 100, 4096, 130, 1]
    together = [(s, 0, 10) for s in sizes]
    off, total = ko_smem.plan(together, 128)
    want, at = [], 0
    for s in sizes:                                           # largest first: end to end in order, each start rounded up
        want.append(at)
        at = (at + s + 127) // 128 * 128
    assert off == want and total == want[-1] + sizes[-1]
    apart = [(s, 2 * k, 2 * k + 2) for k, s in enumerate(sizes)]
    assert ko_smem.plan(apart, 128) == ([0] * 5, max(sizes))
    assert ko_smem.plan([], 128) == ([], 0)
    # the fixture's four 128x64 f16 tiles, alive over the whole function: 64 KiB
    assert ko_smem.plan([(16384, 0, 200)] * 4, 128) == ([0, 16384, 32768, 49152], 65536)


def test_plan_ends_where_the_loop_as_written_would_not():
    # B overlaps A and C in time, A and C do not meet, C is larger than A: returning first-colour buffers to
    # offset 0 on every pass alternates between two placements for ever
    buffers = [(128, 0, 2), (256, 1, 4), (512, 3, 5)]
    off, total = ko_smem.plan(buffers, 128)
    _check_plan(buffers, off, total, 128)
    assert _lib_plan(buffers, 128) == (off, total)


def test_plan_invariants_and_library_agreement_on_random_inputs():
    rng = random.Random(5)
    for trial in range(300):
        n = rng.randint(1, 9)
        alignment = rng.choice([1, 16, 128])
        buffers = []
        for _ in range(n):
            a = rng.randint(0, 12)
            buffers.append((rng.choice([1, 48, 128, 200, 1024, 4096]), a, a + rng.randint(0, 6)))
        off, total = ko_smem.plan(buffers, alignment)
        _check_plan(buffers, off, total, alignment)
        assert _lib_plan(buffers, alignment) == (off, total), buffers


def test_plan_against_brute_force_minimum_on_tiny_inputs():
    # with unit alignment and sizes from a small set the minimum footprint is found by trying every offset;
    # the heuristic may not reach it (a buffer goes behind the farthest end of its neighbours, placed or not:
    # sizes 1, 1, 2 all live together end at 5) but can never beat it, and reaches it when the buffers are all
    # live together and come in descending size
    rng = random.Random(9)
    for trial in range(60):
        n = rng.randint(2, 4)
        buffers = [(rng.randint(1, 4), a, a + rng.randint(1, 3)) for a in (rng.randint(0, 4) for _ in range(n))]
        best = None
        for offs in itertools.product(range(0, 13), repeat=n):
            ok = all(not (buffers[i][1] < buffers[j][2] and buffers[j][1] < buffers[i][2] and
                          offs[i] < offs[j] + buffers[j][0] and offs[j] < offs[i] + buffers[i][0])
                     for i, j in itertools.combinations(range(n), 2))
            if ok:
                t = max(o + b[0] for o, b in zip(offs, buffers))
                best = t if best is None else min(best, t)
        off, total = ko_smem.plan(buffers, 1)
        _check_plan(buffers, off, total, 1)
        assert total >= best
        together = sorted(((b[0], 0, 1) for b in buffers), reverse=True)
        assert ko_smem.plan(together, 1)[1] == sum(b[0] for b in buffers)
    assert ko_smem.plan([(1, 4, 6), (1, 4, 7), (2, 3, 6)], 1) == ([0, 2, 3], 5)


def test_plan_rejects_bad_arguments():
    arr = (kh.SmemBuffer * 1)()
    arr[0].size, arr[0].live_start, arr[0].live_end = -1, 0, 1
    assert kh.lib().kapy_smem_plan(arr, 1, 128) == -1
    arr[0].size = 4
    assert kh.lib().kapy_smem_plan(arr, 1, 96) == -1
    assert kh.lib().kapy_smem_plan(None, 0, 0) == 0


# ---------------------------------------------------------------------------------------------------------
def _paths(successors, length):
    """Every path of `length` blocks from the entry."""
    out = [[0]]
    for _ in range(length - 1):
        out = [p + [s] for p in out for s in successors[p[-1]]] + [p for p in out if not successors[p[-1]]]
    return out


def _race_free(blocks, successors, flags, length=5):
    """No path carries two conflicting accesses of different ops without a barrier between them."""
    for path in _paths(successors, length):
        pending = []                                          # (begin, end, is_write)
        for b in path:
            for i, (kind, accesses) in enumerate(blocks[b]):
                if flags[b][i] & 1 or kind == ko_smem.BARRIER:
                    pending = []
                if kind == ko_smem.ACCESS:
                    for a in accesses:
                        for p in pending:
                            if (a[2] or p[2]) and a[0] < p[1] and p[0] < a[1] and a[1] > a[0]:
                                return False
                    pending += [a for a in accesses if a[1] > a[0]]
                if kind == ko_smem.WAIT_GROUP or flags[b][i] & 2:
                    pending = []
    return True


def _lib_barriers(blocks, successors):
    ops, accesses = [], []
    for b, block in enumerate(blocks):
        for kind, acc in block:
            ops.append((b, kind, len(accesses), len(acc)))
            accesses += acc
    o = (kh.SmemOp * max(len(ops), 1))(*[kh.SmemOp(*x) for x in ops])
    a = (kh.SmemAccess * max(len(accesses), 1))(*[kh.SmemAccess(x[0], x[1], int(x[2]), 0) for x in accesses])
    sb, flat = [0], []
    for s in successors:
        flat += s
        sb.append(len(flat))
    out = (C.c_int32 * max(len(ops), 1))()
    n = kh.lib().kapy_smem_barriers(o, len(ops), a, len(accesses), (C.c_int32 * len(sb))(*sb), (C.c_int32 * max(len(flat), 1))(*flat),
                                    len(blocks), out)
    assert n >= 0, kh.last_error()
    flags, k = [], 0
    for block in blocks:
        flags.append([out[k + i] for i in range(len(block))])
        k += len(block)
    assert n == sum((f & 1) + (f >> 1 & 1) for fl in flags for f in fl)
    return flags


R = lambda b, e: (b, e, False)
W = lambda b, e: (b, e, True)
A = ko_smem.ACCESS


def test_barriers_straight_line_cases():
    one = lambda ops: ko_smem.barriers([ops], [[]])[0]
    assert one([(A, [W(0, 64)]), (A, [R(0, 64)])]) == [0, 1]                       # read after write
    assert one([(A, [R(0, 64)]), (A, [W(32, 96)])]) == [0, 1]                      # write after read, partial overlap
    assert one([(A, [W(0, 64)]), (A, [W(0, 64)])]) == [0, 1]                       # write after write
    assert one([(A, [R(0, 64)]), (A, [R(0, 64)])]) == [0, 0]                       # reads never conflict
    assert one([(A, [W(0, 64)]), (A, [R(64, 128)])]) == [0, 0]                     # touching ranges do not meet
    assert one([(A, [W(0, 64)]), (ko_smem.BARRIER, []), (A, [R(0, 64)])]) == [0, 0, 0]
    assert one([(A, [W(0, 64)]), (ko_smem.WAIT_GROUP, []), (A, [R(0, 64)])]) == [0, 2, 0]
    assert one([(ko_smem.WAIT_GROUP, []), (ko_smem.BARRIER, [])]) == [0, 0]         # already followed by a barrier
    # one barrier serves every access pending before it
    assert one([(A, [W(0, 64)]), (A, [W(64, 128)]), (A, [R(0, 64)]), (A, [R(64, 128)])]) == [0, 0, 1, 0]


def test_barriers_loop_carried_hazard_is_found_through_the_back_edge():
    # entry -> header -> body -> header, header -> exit; the body reads a buffer at its top and overwrites it at
    # its bottom: the write of one trip meets the read of the next only across the back edge
    blocks = [[(A, [W(0, 64)])], [], [(A, [R(0, 64)]), (A, [R(64, 128)]), (A, [W(0, 64)])], [(A, [R(64, 128)])]]
    successors = [[1], [2, 3], [1], []]
    flags = ko_smem.barriers(blocks, successors)
    assert flags == [[0], [], [1, 0, 1], [0]]
    assert _race_free(blocks, successors, flags)
    assert _lib_barriers(blocks, successors) == flags


def test_barriers_are_sufficient_and_match_the_library_on_random_graphs():
    rng = random.Random(3)
    for trial in range(200):
        nb = rng.randint(1, 4)
        blocks = []
        for _ in range(nb):
            ops = []
            for _ in range(rng.randint(0, 4)):
                kind = rng.choice([A, A, A, A, ko_smem.BARRIER, ko_smem.WAIT_GROUP])
                acc = []
                if kind == A:
                    for _ in range(rng.randint(0, 2)):
                        b = rng.choice([0, 64, 128, 192])
                        acc.append((b, b + rng.choice([64, 128]), rng.random() < 0.5))
                ops.append((kind, acc))
            blocks.append(ops)
        successors = [sorted(set(rng.sample(range(nb), rng.randint(0, min(2, nb))))) for _ in range(nb)]
        flags = ko_smem.barriers(blocks, successors)
        assert _race_free(blocks, successors, flags, length=6), (blocks, successors, flags)
        assert _lib_barriers(blocks, successors) == flags, (blocks, successors)


def test_barriers_before_an_op_are_each_necessary_in_a_straight_line():
    rng = random.Random(4)
    for trial in range(200):
        ops = []
        for _ in range(rng.randint(1, 7)):
            b = rng.choice([0, 64, 128])
            ops.append((A, [(b, b + 64, rng.random() < 0.5)]))
        flags = ko_smem.barriers([ops], [[]])
        assert _race_free([ops], [[]], flags, 1)
        for i, f in enumerate(flags[0]):
            if f & 1:                                          # dropping any one barrier leaves a race
                fewer = [list(flags[0])]
                fewer[0][i] = 0
                assert not _race_free([ops], [[]], fewer, 1)


def test_barriers_reject_bad_arguments():
    ops = (kh.SmemOp * 2)(kh.SmemOp(0, 0, 0, 1), kh.SmemOp(0, 5, 0, 0))
    acc = (kh.SmemAccess * 1)(kh.SmemAccess(0, 64, 1, 0))
    out = (C.c_int32 * 2)()
    sb = (C.c_int32 * 2)(0, 0)
    assert kh.lib().kapy_smem_barriers(ops, 2, acc, 1, sb, None, 1, out) == -1 and "unknown kind" in kh.last_error()
    ops[1].kind, ops[1].first_access, ops[1].n_accesses = 0, 1, 1
    assert kh.lib().kapy_smem_barriers(ops, 2, acc, 1, sb, None, 1, out) == -1
    ops[1].n_accesses, ops[1].block = 0, 3
    assert kh.lib().kapy_smem_barriers(ops, 2, acc, 1, sb, None, 1, out) == -1
