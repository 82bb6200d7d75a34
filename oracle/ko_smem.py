"""CPU restatement of the reference's shared-memory allocator and barrier analysis, in plain Python for
small cases.  Test infrastructure only: tests/ import it as the checker of kapy_smem_plan and
kapy_smem_barriers; nothing in the product does.

plan()      lib/Analysis/AllocAnalysis.cpp:187-270 (interference graph, first-fit colouring, bumping,
            repeat until nothing interferes).  Pinned by tests/test_oracle_smem.py: closed forms (buffers all
            live together sit end to end in order; buffers never live together all sit at 0), the invariant
            that live-overlapping buffers never share bytes, the lower bound max over time of the live
            bytes, and exhaustive comparison with a brute-force minimal packing on tiny inputs.
barriers()  lib/Analysis/BlockAnalysis.cpp:37-88, :114-169.  Pinned by a brute-force checker that walks
            every path of bounded length through the control-flow graph and demands a barrier between any
            two conflicting accesses, and that no barrier can be dropped without breaking that.
"""


def _meets(a0, a1, b0, b1):
    return a0 < b1 and b0 < a1


def plan(buffers, alignment=128):
    """buffers: list of (size, live_start, live_end).  Returns (offsets, allocated_size)."""
    n = len(buffers)
    size = [b[0] for b in buffers]
    live = [(b[1], b[2]) for b in buffers]
    off = [0] * n
    up = lambda x: (x + alignment - 1) // alignment * alignment

    def graph_of():
        g = [[] for _ in range(n)]
        for i in range(n):
            for j in range(n):
                if i != j and _meets(*live[i], *live[j]) and _meets(off[i], off[i] + size[i], off[j], off[j] + size[j]):
                    g[i].append(j)
        return g

    def place(g, to_zero):
        colour = [-1] * n
        for i in range(n):
            taken = {colour[j] for j in g[i] if colour[j] >= 0}
            c = 0
            while c in taken:
                c += 1
            colour[i] = c
        for i in range(n):
            if colour[i] == 0:
                if to_zero:
                    off[i] = 0
            else:
                off[i] = up(max([off[j] + size[j] for j in g[i]], default=0))

    seen, as_written, passes = set(), True, 0
    g = graph_of()
    while True:
        place(g, as_written)
        g = graph_of()
        if not any(g):
            break
        if as_written:
            state = tuple(off)
            if state in seen:
                as_written = False      # the loop as written would repeat this placement for ever
            seen.add(state)
        passes += 1
        if passes > 64 + 8 * n:
            at = 0
            for i in range(n):
                off[i] = at
                at = up(at + size[i])
            break
    return off, max([off[i] + size[i] for i in range(n)], default=0)


ACCESS, BARRIER, WAIT_GROUP = 0, 1, 2


def barriers(blocks, successors):
    """blocks: list of blocks, a block a list of ops; an op is (kind, [(begin, end, is_write), ...]).
    successors: list of successor lists.  Returns a list of blocks of flags (bit 0: barrier before the op,
    bit 1: after it)."""
    flags = [[0] * len(b) for b in blocks]
    incoming = [(set(), set()) for _ in blocks]
    joined = [None] * len(blocks)
    hit = lambda xs, ys: any(_meets(a[0], a[1], b[0], b[1]) for a in xs for b in ys)
    work = [0]
    while work:
        b = work.pop(0)
        reads, writes = set(incoming[b][0]), set(incoming[b][1])
        for i, (kind, accesses) in enumerate(blocks[b]):
            if flags[b][i] & 1:
                reads, writes = set(), set()
            if kind == BARRIER:
                reads, writes = set(), set()
                continue
            if kind == WAIT_GROUP:
                nxt = blocks[b][i + 1][0] if i + 1 < len(blocks[b]) else None
                if nxt != BARRIER:
                    flags[b][i] |= 2
                reads, writes = set(), set()
                continue
            r = {(a[0], a[1]) for a in accesses if not a[2] and a[1] > a[0]}
            w = {(a[0], a[1]) for a in accesses if a[2] and a[1] > a[0]}
            if hit(writes, r) or hit(reads, w) or hit(writes, w):
                flags[b][i] |= 1
                reads, writes = set(), set()
            reads |= r
            writes |= w
        if joined[b] is not None and reads <= joined[b][0] and writes <= joined[b][1]:
            continue
        if joined[b] is None:
            joined[b] = (set(), set())
        joined[b][0].update(reads)
        joined[b][1].update(writes)
        for s in successors[b]:
            incoming[s][0].update(joined[b][0])
            incoming[s][1].update(joined[b][1])
            work.append(s)
    return flags
