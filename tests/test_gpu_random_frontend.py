"""Seeded random kapy.func bodies for the textual front-end: a random DAG of elementwise ops (arith / math on tensors, casts
between f16 and f32, splats, fma), row maxima broadcast back, values used more than once, one or two stores, over two to ten
loaded tensors.  The front-end defers such chains and runs each as one program (cut where a program's limits are reached); with
KAPY_MLIR_FUSE=0 every op is a call of its own, each of which the elementwise tests hold to the oracle.  The two runs execute the
same instructions on the same values, so they must agree bit for bit."""
import numpy as np
import pytest

import kapy_hip as kh
import kapy_programs as kp
from gpu_util import dev_zeros, sync, to_dev, to_host

pytestmark = pytest.mark.gpu

BINARY = ["arith.addf", "arith.subf", "arith.mulf", "arith.maximumf", "arith.minimumf", "arith.maxnumf", "arith.minnumf"]
UNARY = ["arith.negf", "math.absf", "math.tanh", "math.tanh", "math.erf", "math.sin", "math.cos", "math.floor", "math.ceil"]   # bounded, so that long chains stay finite


def random_program(rng, rows_per_warp, cols, warps):
    """(text, number of inputs, dtypes of the outputs) of a random function over [rows x cols] f16 tensors."""
    n_in = int(rng.randint(2, 11))
    n_ops = int(rng.randint(4, 45))
    t = {"f16": "tensor<%dx%dxf16" % (rows_per_warp, cols), "f32": "tensor<%dx%dxf32" % (rows_per_warp, cols)}
    c = {"f16": "tensor<%dx1xf16" % rows_per_warp, "f32": "tensor<%dx1xf32" % rows_per_warp}
    dyn = "tensor<?x?xf16, #global>"
    lines = [kp._consts([0, 1, rows_per_warp, rows_per_warp * warps, cols]),
             "    %half = arith.constant 0.5 : f32\n",
             "    %pid = kapy.program_id {axis = 0 : i32} : i32\n    %warp = kapy.warp_id : i32\n",
             "    %p0 = arith.muli %pid, %c{0}_i32 : i32\n    %w0 = arith.muli %warp, %c{1}_i32 : i32\n".format(rows_per_warp * warps, rows_per_warp),
             "    %row0 = arith.addi %p0, %w0 : i32\n    %row1 = arith.addi %row0, %c{0}_i32 : i32\n".format(rows_per_warp)]

    def view(name):
        return ("    %g{n} = kapy.mk_global %{n}[%c0_i32] [%rows, %c{cols}_i32] [%c{cols}_i32, %c1_i32] : !kapy.ptr<1> -> {dyn}\n"
                "    %s{n} = kapy.sv_global %g{n}[%row0 : %row1, %c0_i32 : %c{cols}_i32] : {dyn} -> {t}, #global>\n").format(
                    n=name, cols=cols, dyn=dyn, t=t["f16"])

    pool = {"f16": [], "f32": []}
    for k in range(n_in):
        lines.append(view("in%d" % k))
        lines.append("    %v{k} = kapy.ld_global %sin{k} : {t}, #global> -> {t}, #values>\n".format(k=k, t=t["f16"]))
        pool["f16"].append("%%v%d" % k)
    fresh = [0]

    def new():
        fresh[0] += 1
        return "%%t%d" % fresh[0]

    def pick(dt):
        """A value of type dt: an existing one, or a cast of one of the other type."""
        other = "f32" if dt == "f16" else "f16"
        if pool[dt] and (not pool[other] or rng.randint(4)):
            return pool[dt][rng.randint(len(pool[dt]))]
        src, r = pool[other][rng.randint(len(pool[other]))], new()
        if dt == "f32":
            lines.append("    {r} = kapy.fptofp {s} : {a}, #values> to {b}, #values>\n".format(r=r, s=src, a=t["f16"], b=t["f32"]))
        else:
            lines.append("    {r} = kapy.fptofp {s} {{rounding_mode = {m} : i32}} : {a}, #values> to {b}, #values>\n".format(
                r=r, s=src, m=int(rng.randint(2)), a=t["f32"], b=t["f16"]))
        pool[dt].append(r)
        return r

    for _ in range(n_ops):
        dt = ["f16", "f32", "f32"][rng.randint(3)]
        kind, r = rng.randint(10), new()
        if kind < 4:
            lines.append("    {r} = {op} {a}, {b} : {t}, #values>\n".format(r=r, op=BINARY[rng.randint(len(BINARY))], a=pick(dt), b=pick(dt), t=t[dt]))
        elif kind < 7:
            lines.append("    {r} = {op} {a} : {t}, #values>\n".format(r=r, op=UNARY[rng.randint(len(UNARY))], a=pick(dt), t=t[dt]))
        elif kind == 7:
            lines.append("    {r} = math.fma {a}, {b}, {c} : {t}, #values>\n".format(r=r, a=pick(dt), b=pick(dt), c=pick(dt), t=t[dt]))
        elif kind == 8:
            s = new()
            lines.append("    {s} = kapy.splat %half : f32 -> {t}, #values>\n    {r} = arith.mulf {a}, {s} : {t}, #values>\n".format(
                s=s, r=r, a=pick("f32"), t=t["f32"]))
            dt = "f32"
        else:                                             # the row maximum, optionally negated, broadcast back and subtracted
            m, mb, a = new(), new(), pick(dt)
            lines.append("    {m} = kapy.reduce {a} {{axis = 1 : i32}} lambda(%lhs: {e}, %rhs: {e}) {{\n      %r = arith.maximumf %lhs, %rhs : {e}\n"
                         "      kapy.return %r : {e}\n    }} : {t}, #values> -> {c}, #values>\n".format(m=m, a=a, e=dt, t=t[dt], c=c[dt]))
            if rng.randint(2):
                m2 = new()
                lines.append("    {m2} = math.absf {m} : {c}, #values>\n".format(m2=m2, m=m, c=c[dt]))
                m = m2
            lines.append("    {mb} = kapy.broadcast {m} : {c}, #values> -> {t}, #values>\n".format(mb=mb, m=m, c=c[dt], t=t[dt]))
            lines.append("    {r} = arith.subf {a}, {mb} : {t}, #values>\n".format(r=r, a=a, mb=mb, t=t[dt]))
        pool[dt].append(r)
    n_out = int(rng.randint(1, 3))
    for k in range(n_out):
        # the last value made, and for a second store any earlier one: a value with other uses
        src = pick("f16") if k else (pool["f16"][-1] if pool["f16"] and rng.randint(2) else pick("f16"))
        lines.append(view("out%d" % k))
        lines.append("    kapy.st_global {s}, %sout{k} : {t}, #values>, {t}, #global>\n".format(s=src, k=k, t=t["f16"]))
    lines.append("    kapy.return\n")
    args = ", ".join(["%%in%d: !kapy.ptr<1>" % k for k in range(n_in)] + ["%%out%d: !kapy.ptr<1>" % k for k in range(n_out)] + ["%rows: i32"])
    text = (kp.HEADER + "module attributes {kapy.num_warps = %d : i64} {\n  kapy.func public @random_kernel(%s) {\n" % (warps, args) +
            "".join(lines) + "  }\n}\n")
    return text, n_in, n_out


@pytest.mark.parametrize("seed", range(40))
def test_random_function_fused_equals_op_by_op(ko, monkeypatch, seed):
    rng = np.random.RandomState(11000 + seed)
    rows_per_warp, cols = [(2, 256), (4, 128), (1, 1024), (3, 72), (2, 100)][rng.randint(5)]
    warps, programs = int(rng.randint(1, 3)), int(rng.randint(1, 3))
    rows = rows_per_warp * warps * programs
    text, n_in, n_out = random_program(rng, rows_per_warp, cols, warps)
    n_args, _, _ = kh.parse_mlir(text)
    assert n_args == n_in + n_out + 1
    ins = [to_dev(ko.fill_normal(rows * cols, ko.F16, 11000 + seed, k)) for k in range(n_in)]
    results = []
    for fuse in ("1", "0"):
        monkeypatch.setenv("KAPY_MLIR_FUSE", fuse)
        outs = [dev_zeros(rows * cols, 2, fill=0x7e00) for _ in range(n_out)]
        kh.run_mlir(text, ins + outs + [rows], [programs])
        sync()
        results.append([to_host(o, np.uint16) for o in outs])
    for k in range(n_out):
        f, u = results[0][k], results[1][k]
        nan = lambda a: (a & 0x7fff) > 0x7c00
        same = (f == u) | (nan(f) & nan(u))
        bad = np.flatnonzero(~same)
        assert np.isfinite(f.view(np.float16)).mean() > 0.5, "seed %d, output %d: the program's values are not finite" % (seed, k)
        assert len(bad) == 0, "seed %d, output %d: %d of %d elements differ, first at %d (fused %#x, op by op %#x)\n%s" % (
            seed, k, len(bad), f.size, bad[0], f[bad[0]], u[bad[0]], text)
