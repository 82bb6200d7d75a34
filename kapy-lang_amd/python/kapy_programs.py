"""Kapy-dialect programs in textual form, written for the tests and the benchmark in the op syntax of the reference's
fixtures (test/Conversion/KapyToKgpu/{elementwise_add,reduce_sum,matmul}.mlir; Ops.td): the same ops and
the same program structure (per-warp sub-views, a shared-memory double buffer filled with
cp_async_global_to_shared, ld_matrix fragments, an scf.for carrying the accumulator, arith.select choosing
the buffer), with shapes and tilings of their own."""

HEADER = """#global = #kapy.encoding<global_memory>
#shared = #kapy.encoding<shared_memory>
#values = #kapy.encoding<register_file>
"""


def _consts(values):
    return "".join("    %%c%d_i32 = arith.constant %d : i32\n" % (v, v) for v in sorted(set(values)))


def binary_program(op="arith.addf", rows_per_warp=4, cols=128, num_warps=4, dtype="f16"):
    """out[r, :] = x[r, :] <op> y[r, :]; a program covers num_warps*rows_per_warp rows of `cols` columns."""
    t = "tensor<%dx%dx%s" % (rows_per_warp, cols, dtype)
    dyn = "tensor<?x?x%s, #global>" % dtype
    body = _consts([0, 1, rows_per_warp, rows_per_warp * num_warps, cols])
    body += """    %pid = kapy.program_id {{axis = 0 : i32}} : i32
    %warp = kapy.warp_id : i32
    %p0 = arith.muli %pid, %c{rpp}_i32 : i32
    %w0 = arith.muli %warp, %c{rpw}_i32 : i32
    %row0 = arith.addi %p0, %w0 : i32
    %row1 = arith.addi %row0, %c{rpw}_i32 : i32
    %gx = kapy.mk_global %x[%c0_i32] [%rows, %c{cols}_i32] [%c{cols}_i32, %c1_i32] : !kapy.ptr<1> -> {dyn}
    %gy = kapy.mk_global %y[%c0_i32] [%rows, %c{cols}_i32] [%c{cols}_i32, %c1_i32] : !kapy.ptr<1> -> {dyn}
    %go = kapy.mk_global %out[%c0_i32] [%rows, %c{cols}_i32] [%c{cols}_i32, %c1_i32] : !kapy.ptr<1> -> {dyn}
    %sx = kapy.sv_global %gx[%row0 : %row1, %c0_i32 : %c{cols}_i32] : {dyn} -> {t}, #global>
    %sy = kapy.sv_global %gy[%row0 : %row1, %c0_i32 : %c{cols}_i32] : {dyn} -> {t}, #global>
    %so = kapy.sv_global %go[%row0 : %row1, %c0_i32 : %c{cols}_i32] : {dyn} -> {t}, #global>
    %vx = kapy.ld_global %sx : {t}, #global> -> {t}, #values>
    %vy = kapy.ld_global %sy : {t}, #global> -> {t}, #values>
    %vo = {op} %vx, %vy : {t}, #values>
    kapy.st_global %vo, %so : {t}, #values>, {t}, #global>
    kapy.return
""".format(rpp=rows_per_warp * num_warps, rpw=rows_per_warp, cols=cols, dyn=dyn, t=t, op=op)
    return (HEADER + "module attributes {kapy.num_warps = %d : i64} {\n" % num_warps +
            "  kapy.func public @binary_kernel(%x: !kapy.ptr<1> {kapy.alignment = 128 : i64}, %y: !kapy.ptr<1> {kapy.alignment = 128 : i64}, "
            "%out: !kapy.ptr<1> {kapy.alignment = 128 : i64}, %rows: i32 {kapy.alignment = 4 : i64}) {\n" + body + "  }\n}\n")


def reduce_program(combiner="arith.addf", rows_per_warp=2, cols=512, num_warps=2, dtype="f16"):
    """out[r] = reduce over the columns of x[r, :]; out is a column vector stored with stride (1, rows)."""
    src = "tensor<%dx%dx%s" % (rows_per_warp, cols, dtype)
    dst = "tensor<%dx1x%s" % (rows_per_warp, dtype)
    dyn = "tensor<?x?x%s, #global>" % dtype
    body = _consts([0, 1, rows_per_warp, rows_per_warp * num_warps, cols])
    body += """    %0 = kapy.mk_global %arg0[%c0_i32] [%arg2, %c{cols}_i32] [%c{cols}_i32, %c1_i32] : !kapy.ptr<1> -> {dyn}
    %1 = kapy.program_id {{axis = 0 : i32}} : i32
    %2 = kapy.warp_id : i32
    %3 = arith.muli %1, %c{rpp}_i32 : i32
    %4 = arith.muli %2, %c{rpw}_i32 : i32
    %5 = arith.addi %3, %4 : i32
    %6 = arith.addi %5, %c{rpw}_i32 : i32
    %7 = kapy.sv_global %0[%5 : %6, %c0_i32 : %c{cols}_i32] : {dyn} -> {src}, #global>
    %8 = kapy.ld_global %7 : {src}, #global> -> {src}, #values>
    %9 = kapy.reduce %8 {{axis = 1 : i32}} lambda(%lhs: {dtype}, %rhs: {dtype}) {{
      %12 = {comb} %lhs, %rhs : {dtype}
      kapy.return %12 : {dtype}
    }} : {src}, #values> -> {dst}, #values>
    %10 = kapy.mk_global %arg1[%c0_i32] [%arg2, %c1_i32] [%c1_i32, %arg2] : !kapy.ptr<1> -> {dyn}
    %11 = kapy.sv_global %10[%5 : %6, %c0_i32 : %c1_i32] : {dyn} -> {dst}, #global>
    kapy.st_global %9, %11 : {dst}, #values>, {dst}, #global>
    kapy.return
""".format(rpp=rows_per_warp * num_warps, rpw=rows_per_warp, cols=cols, dyn=dyn, src=src, dst=dst, dtype=dtype, comb=combiner)
    return (HEADER + "module attributes {kapy.num_warps = %d : i64, kapy.nvidia_cc = 89 : i64} {\n" % num_warps +
            "  kapy.func public @reduce_kernel(%arg0: !kapy.ptr<1>, %arg1: !kapy.ptr<1>, %arg2: i32) {\n" + body + "  }\n}\n")


def matmul_program(bm=64, bn=64, bk=32, way="mma_m16n8k16_f16", acc="f16", dtype="f16"):
    """C[M,N] = A[M,K] . B[K,N], row-major.  A program owns a (2*bm)x(2*bn) tile of C, its four warps a bm x bn
    quarter each.  K advances in steps of bk through two shared-memory buffers per operand: the loop body
    multiplies the tile that the previous step loaded while cp_async fills the other buffer, which
    arith.select picks by the parity of the step, and the accumulator is carried in iter_args."""
    ga, gb, gc = ("tensor<%dx%dx%s, #global>" % s for s in ((bm, bk, dtype), (bk, bn, dtype), (bm, bn, acc)))
    sa_full, sb_full = "tensor<%dx%dx%s, #shared>" % (2 * bm, bk, dtype), "tensor<%dx%dx%s, #shared>" % (bk, 2 * bn, dtype)
    sa, sb = "tensor<%dx%dx%s, #shared>" % (bm, bk, dtype), "tensor<%dx%dx%s, #shared>" % (bk, bn, dtype)
    va, vb, vc = ("tensor<%dx%dx%s, #values>" % s for s in ((bm, bk, dtype), (bk, bn, dtype), (bm, bn, acc)))
    dyn, dync = "tensor<?x?x%s, #global>" % dtype, "tensor<?x?x%s, #global>" % acc
    body = _consts([0, 1, 2, bm, bn, bk, 2 * bm, 2 * bn])
    body += """    %zero = arith.constant dense<0.000000e+00> : {vc}
    %pad_a = arith.constant dense<0.000000e+00> : {va}
    %pad_b = arith.constant dense<0.000000e+00> : {vb}
    %A = kapy.mk_global %a[%c0_i32] [%m, %k] [%k, %c1_i32] : !kapy.ptr<1> -> {dyn}
    %B = kapy.mk_global %b[%c0_i32] [%k, %n] [%n, %c1_i32] : !kapy.ptr<1> -> {dyn}
    %C = kapy.mk_global %c[%c0_i32] [%m, %n] [%n, %c1_i32] : !kapy.ptr<1> -> {dync}
    %a_buf0 = kapy.mk_shared {{kapy.row_major = true}} : {sa_full}
    %b_buf0 = kapy.mk_shared {{kapy.row_major = true}} : {sb_full}
    %a_buf1 = kapy.mk_shared {{kapy.row_major = true}} : {sa_full}
    %b_buf1 = kapy.mk_shared {{kapy.row_major = true}} : {sb_full}
    %pid = kapy.program_id {{axis = 0 : i32}} : i32
    %warp = kapy.warp_id : i32
    %tiles_n = arith.divui %n, %c{bn2}_i32 : i32
    %tile_m = arith.divui %pid, %tiles_n : i32
    %tile_n = arith.remui %pid, %tiles_n : i32
    %warp_m = arith.divui %warp, %c2_i32 : i32
    %warp_n = arith.remui %warp, %c2_i32 : i32
    %sm0 = arith.muli %warp_m, %c{bm}_i32 : i32
    %sm1 = arith.addi %sm0, %c{bm}_i32 : i32
    %sn0 = arith.muli %warp_n, %c{bn}_i32 : i32
    %sn1 = arith.addi %sn0, %c{bn}_i32 : i32
    %tm = arith.muli %tile_m, %c{bm2}_i32 : i32
    %tn = arith.muli %tile_n, %c{bn2}_i32 : i32
    %row0 = arith.addi %tm, %sm0 : i32
    %row1 = arith.addi %row0, %c{bm}_i32 : i32
    %col0 = arith.addi %tn, %sn0 : i32
    %col1 = arith.addi %col0, %c{bn}_i32 : i32
    %a_sh0 = kapy.sv_shared %a_buf0[%sm0 : %sm1, %c0_i32 : %c{bk}_i32] : {sa_full} -> {sa}
    %b_sh0 = kapy.sv_shared %b_buf0[%c0_i32 : %c{bk}_i32, %sn0 : %sn1] : {sb_full} -> {sb}
    %a_sh1 = kapy.sv_shared %a_buf1[%sm0 : %sm1, %c0_i32 : %c{bk}_i32] : {sa_full} -> {sa}
    %b_sh1 = kapy.sv_shared %b_buf1[%c0_i32 : %c{bk}_i32, %sn0 : %sn1] : {sb_full} -> {sb}
    %a_g0 = kapy.sv_global %A[%row0 : %row1, %c0_i32 : %c{bk}_i32] : {dyn} -> {ga}
    %b_g0 = kapy.sv_global %B[%c0_i32 : %c{bk}_i32, %col0 : %col1] : {dyn} -> {gb}
    kapy.cp_async_global_to_shared %a_g0, %a_sh0, %pad_a : {ga}, {sa}, {va}
    kapy.cp_async_global_to_shared %b_g0, %b_sh0, %pad_b : {gb}, {sb}, {vb}
    kapy.cp_async_wait_group {{num_pending = 0 : i32}}
    %steps = arith.divui %k, %c{bk}_i32 : i32
    %loop:2 = scf.for %step = %c1_i32 to %steps step %c1_i32 iter_args(%acc = %zero, %unused = %c0_i32) -> ({vc}, i32)  : i32 {{
      %parity = arith.remui %step, %c2_i32 : i32
      %odd = arith.cmpi eq, %parity, %c1_i32 : i32
      %a_cur = arith.select %odd, %a_sh0, %a_sh1 : {sa}
      %b_cur = arith.select %odd, %b_sh0, %b_sh1 : {sb}
      %a_nxt = arith.select %odd, %a_sh1, %a_sh0 : {sa}
      %b_nxt = arith.select %odd, %b_sh1, %b_sh0 : {sb}
      %k0 = arith.muli %step, %c{bk}_i32 : i32
      %k1 = arith.addi %k0, %c{bk}_i32 : i32
      %a_g = kapy.sv_global %A[%row0 : %row1, %k0 : %k1] : {dyn} -> {ga}
      %b_g = kapy.sv_global %B[%k0 : %k1, %col0 : %col1] : {dyn} -> {gb}
      kapy.cp_async_global_to_shared %a_g, %a_nxt, %pad_a : {ga}, {sa}, {va}
      kapy.cp_async_global_to_shared %b_g, %b_nxt, %pad_b : {gb}, {sb}, {vb}
      %a_frag = kapy.ld_matrix %a_cur, %pad_a : {sa}, {va} -> {va}
      %b_frag = kapy.ld_matrix %b_cur, %pad_b : {sb}, {vb} -> {vb}
      %next = kapy.matmul {way} %a_frag, %b_frag, %acc : {va}, {vb} -> {vc}
      kapy.cp_async_wait_group {{num_pending = 0 : i32}}
      scf.yield %next, %step : {vc}, i32
    }}
    %last = arith.remui %loop#1, %c2_i32 : i32
    %last_odd = arith.cmpi eq, %last, %c1_i32 : i32
    %a_fin = arith.select %last_odd, %a_sh1, %a_sh0 : {sa}
    %b_fin = arith.select %last_odd, %b_sh1, %b_sh0 : {sb}
    %a_ff = kapy.ld_matrix %a_fin, %pad_a : {sa}, {va} -> {va}
    %b_ff = kapy.ld_matrix %b_fin, %pad_b : {sb}, {vb} -> {vb}
    %result = kapy.matmul {way} %a_ff, %b_ff, %loop#0 : {va}, {vb} -> {vc}
    %c_g = kapy.sv_global %C[%row0 : %row1, %col0 : %col1] : {dync} -> {gc}
    kapy.st_global %result, %c_g : {vc}, {gc}
    kapy.return
""".format(bm=bm, bn=bn, bk=bk, bm2=2 * bm, bn2=2 * bn, ga=ga, gb=gb, gc=gc, sa=sa, sb=sb, sa_full=sa_full, sb_full=sb_full,
           va=va, vb=vb, vc=vc, dyn=dyn, dync=dync, way=way)
    return (HEADER + "module attributes {kapy.num_warps = 4 : i64, kapy.nvidia_cc = 89 : i64} {\n"
            "  kapy.func public @matmul_kernel(%a: !kapy.ptr<1> {kapy.alignment = 128 : i64}, %b: !kapy.ptr<1> {kapy.alignment = 128 : i64}, "
            "%c: !kapy.ptr<1> {kapy.alignment = 128 : i64}, %m: i32, %n: i32, %k: i32) {\n" + body + "  }\n}\n")


def phases_program():
    """p[64,64] <- 2*p through shared memory in two phases: a buffer filled by cp_async and read by ld_matrix, then,
    once that one is dead, two more buffers (one of them only read) written by st_shared and read by ld_shared."""
    return HEADER + """module attributes {kapy.num_warps = 1 : i64} {
  kapy.func public @phases(%p: !kapy.ptr<1>) {
    %c0_i32 = arith.constant 0 : i32
    %c1_i32 = arith.constant 1 : i32
    %c64_i32 = arith.constant 64 : i32
    %pad = arith.constant dense<0.000000e+00> : tensor<64x64xf16, #values>
    %g = kapy.mk_global %p[%c0_i32] [%c64_i32, %c64_i32] [%c64_i32, %c1_i32] : !kapy.ptr<1> -> tensor<?x?xf16, #global>
    %gs = kapy.sv_global %g[%c0_i32 : %c64_i32, %c0_i32 : %c64_i32] : tensor<?x?xf16, #global> -> tensor<64x64xf16, #global>
    %first = kapy.mk_shared {kapy.row_major = true} : tensor<64x64xf16, #shared>
    kapy.cp_async_global_to_shared %gs, %first, %pad : tensor<64x64xf16, #global>, tensor<64x64xf16, #shared>, tensor<64x64xf16, #values>
    kapy.cp_async_wait_group {num_pending = 0 : i32}
    %v = kapy.ld_matrix %first, %pad : tensor<64x64xf16, #shared>, tensor<64x64xf16, #values> -> tensor<64x64xf16, #values>
    %w = arith.addf %v, %v : tensor<64x64xf16, #values>
    %second = kapy.mk_shared {kapy.row_major = true} : tensor<64x32xf16, #shared>
    %third = kapy.mk_shared {kapy.row_major = true} : tensor<64x64xf16, #shared>
    kapy.st_shared %w, %third : tensor<64x64xf16, #values>, tensor<64x64xf16, #shared>
    %u = kapy.ld_shared %third : tensor<64x64xf16, #shared> -> tensor<64x64xf16, #values>
    %x = kapy.ld_shared %second : tensor<64x32xf16, #shared> -> tensor<64x32xf16, #values>
    kapy.st_global %u, %gs : tensor<64x64xf16, #values>, tensor<64x64xf16, #global>
    kapy.return
  }
}
"""


def softmax_program(rows_per_warp=2, cols=256, num_warps=2, dtype="f16"):
    """out[r, :] = softmax(x[r, :]) computed in f32: fptofp up, reduce max, broadcast, subf, math.exp, reduce add,
    broadcast, divf, fptofp down with round-to-nearest."""
    t16, t32 = "tensor<%dx%dx%s" % (rows_per_warp, cols, dtype), "tensor<%dx%dxf32" % (rows_per_warp, cols)
    c32 = "tensor<%dx1xf32, #values>" % rows_per_warp
    dyn = "tensor<?x?x%s, #global>" % dtype
    body = _consts([0, 1, rows_per_warp, rows_per_warp * num_warps, cols])
    body += """    %pid = kapy.program_id {{axis = 0 : i32}} : i32
    %warp = kapy.warp_id : i32
    %p0 = arith.muli %pid, %c{rpp}_i32 : i32
    %w0 = arith.muli %warp, %c{rpw}_i32 : i32
    %row0 = arith.addi %p0, %w0 : i32
    %row1 = arith.addi %row0, %c{rpw}_i32 : i32
    %gx = kapy.mk_global %x[%c0_i32] [%rows, %c{cols}_i32] [%c{cols}_i32, %c1_i32] : !kapy.ptr<1> -> {dyn}
    %go = kapy.mk_global %out[%c0_i32] [%rows, %c{cols}_i32] [%c{cols}_i32, %c1_i32] : !kapy.ptr<1> -> {dyn}
    %sx = kapy.sv_global %gx[%row0 : %row1, %c0_i32 : %c{cols}_i32] : {dyn} -> {t16}, #global>
    %so = kapy.sv_global %go[%row0 : %row1, %c0_i32 : %c{cols}_i32] : {dyn} -> {t16}, #global>
    %x16 = kapy.ld_global %sx : {t16}, #global> -> {t16}, #values>
    %xf = kapy.fptofp %x16 : {t16}, #values> to {t32}, #values>
    %m = kapy.reduce %xf {{axis = 1 : i32}} lambda(%lhs: f32, %rhs: f32) {{
      %r = arith.maximumf %lhs, %rhs : f32
      kapy.return %r : f32
    }} : {t32}, #values> -> {c32}
    %mb = kapy.broadcast %m : {c32} -> {t32}, #values>
    %d = arith.subf %xf, %mb : {t32}, #values>
    %e = math.exp %d : {t32}, #values>
    %s = kapy.reduce %e {{axis = 1 : i32}} lambda(%lhs: f32, %rhs: f32) {{
      %r = arith.addf %lhs, %rhs : f32
      kapy.return %r : f32
    }} : {t32}, #values> -> {c32}
    %sb = kapy.broadcast %s : {c32} -> {t32}, #values>
    %q = arith.divf %e, %sb : {t32}, #values>
    %y = kapy.fptofp %q {{rounding_mode = 1 : i32}} : {t32}, #values> to {t16}, #values>
    kapy.st_global %y, %so : {t16}, #values>, {t16}, #global>
    kapy.return
""".format(rpp=rows_per_warp * num_warps, rpw=rows_per_warp, cols=cols, dyn=dyn, t16=t16, t32=t32, c32=c32)
    return (HEADER + "module attributes {kapy.num_warps = %d : i64} {\n" % num_warps +
            "  kapy.func public @softmax_kernel(%x: !kapy.ptr<1>, %out: !kapy.ptr<1>, %rows: i32) {\n" + body + "  }\n}\n")


def causal_softmax_program(rows_per_warp=2, cols=256, num_warps=2, dtype="f16"):
    """out[r, :] = softmax over the columns c <= r of x[r, :] (zero elsewhere), in f32: the row index is kapy.arange along
    axis 0 plus the tile's first row (an integer splat), the column index kapy.arange along axis 1, arith.cmpi sle makes the
    i1 mask and arith.select puts -inf where it is false; then the softmax chain."""
    t16, t32 = "tensor<%dx%dx%s" % (rows_per_warp, cols, dtype), "tensor<%dx%dxf32" % (rows_per_warp, cols)
    ti, tb = "tensor<%dx%dxi32, #values>" % (rows_per_warp, cols), "tensor<%dx%dxi1, #values>" % (rows_per_warp, cols)
    ri, ci = "tensor<%dx1xi32, #values>" % rows_per_warp, "tensor<1x%dxi32, #values>" % cols
    c32 = "tensor<%dx1xf32, #values>" % rows_per_warp
    dyn = "tensor<?x?x%s, #global>" % dtype
    body = _consts([0, 1, rows_per_warp, rows_per_warp * num_warps, cols])
    body += """    %pid = kapy.program_id {{axis = 0 : i32}} : i32
    %warp = kapy.warp_id : i32
    %p0 = arith.muli %pid, %c{rpp}_i32 : i32
    %w0 = arith.muli %warp, %c{rpw}_i32 : i32
    %row0 = arith.addi %p0, %w0 : i32
    %row1 = arith.addi %row0, %c{rpw}_i32 : i32
    %gx = kapy.mk_global %x[%c0_i32] [%rows, %c{cols}_i32] [%c{cols}_i32, %c1_i32] : !kapy.ptr<1> -> {dyn}
    %go = kapy.mk_global %out[%c0_i32] [%rows, %c{cols}_i32] [%c{cols}_i32, %c1_i32] : !kapy.ptr<1> -> {dyn}
    %sx = kapy.sv_global %gx[%row0 : %row1, %c0_i32 : %c{cols}_i32] : {dyn} -> {t16}, #global>
    %so = kapy.sv_global %go[%row0 : %row1, %c0_i32 : %c{cols}_i32] : {dyn} -> {t16}, #global>
    %x16 = kapy.ld_global %sx : {t16}, #global> -> {t16}, #values>
    %xf = kapy.fptofp %x16 : {t16}, #values> to {t32}, #values>
    %rl = kapy.arange {{axis = 0 : i32, start = 0 : i32, end = {rpw} : i32}} : {ri}
    %rb = kapy.splat %row0 : i32 -> {ri}
    %rg = arith.addi %rl, %rb : {ri}
    %rr = kapy.broadcast %rg : {ri} -> {ti}
    %cl = kapy.arange {{axis = 1 : i32, start = 0 : i32, end = {cols} : i32}} : {ci}
    %cc = kapy.broadcast %cl : {ci} -> {ti}
    %keep = arith.cmpi sle, %cc, %rr : {ti}
    %ninf = arith.constant dense<0xFF800000> : {t32}, #values>
    %xm = arith.select %keep, %xf, %ninf : {tb}, {t32}, #values>
    %m = kapy.reduce %xm {{axis = 1 : i32}} lambda(%lhs: f32, %rhs: f32) {{
      %r = arith.maximumf %lhs, %rhs : f32
      kapy.return %r : f32
    }} : {t32}, #values> -> {c32}
    %mb = kapy.broadcast %m : {c32} -> {t32}, #values>
    %d = arith.subf %xm, %mb : {t32}, #values>
    %e = math.exp %d : {t32}, #values>
    %s = kapy.reduce %e {{axis = 1 : i32}} lambda(%lhs: f32, %rhs: f32) {{
      %r = arith.addf %lhs, %rhs : f32
      kapy.return %r : f32
    }} : {t32}, #values> -> {c32}
    %sb = kapy.broadcast %s : {c32} -> {t32}, #values>
    %q = arith.divf %e, %sb : {t32}, #values>
    %y = kapy.fptofp %q {{rounding_mode = 1 : i32}} : {t32}, #values> to {t16}, #values>
    kapy.st_global %y, %so : {t16}, #values>, {t16}, #global>
    kapy.return
""".format(rpp=rows_per_warp * num_warps, rpw=rows_per_warp, cols=cols, dyn=dyn, t16=t16, t32=t32, c32=c32, ti=ti, tb=tb, ri=ri, ci=ci)
    return (HEADER + "module attributes {kapy.num_warps = %d : i64} {\n" % num_warps +
            "  kapy.func public @causal_softmax_kernel(%x: !kapy.ptr<1>, %out: !kapy.ptr<1>, %rows: i32) {\n" + body + "  }\n}\n")


def gated_program(rows_per_warp=4, cols=256, num_warps=2, dtype="f16"):
    """out[r, :] = silu(x[r, :]) * y[r, :] * g[r] in f32, rounded once: two casts up, negf, math.exp, a splat of 1.0, addf,
    divf, mulf, a broadcast of the per-row gate g ([rows x 1]), mulf, a cast down.  Eleven elementwise ops between the loads
    and the store."""
    t16, t32 = "tensor<%dx%dx%s" % (rows_per_warp, cols, dtype), "tensor<%dx%dxf32" % (rows_per_warp, cols)
    c32 = "tensor<%dx1xf32" % rows_per_warp
    dyn, dyn32 = "tensor<?x?x%s, #global>" % dtype, "tensor<?x?xf32, #global>"
    body = _consts([0, 1, rows_per_warp, rows_per_warp * num_warps, cols])
    body += """    %one = arith.constant 1.0 : f32
    %pid = kapy.program_id {{axis = 0 : i32}} : i32
    %warp = kapy.warp_id : i32
    %p0 = arith.muli %pid, %c{rpp}_i32 : i32
    %w0 = arith.muli %warp, %c{rpw}_i32 : i32
    %row0 = arith.addi %p0, %w0 : i32
    %row1 = arith.addi %row0, %c{rpw}_i32 : i32
    %gx = kapy.mk_global %x[%c0_i32] [%rows, %c{cols}_i32] [%c{cols}_i32, %c1_i32] : !kapy.ptr<1> -> {dyn}
    %gy = kapy.mk_global %y[%c0_i32] [%rows, %c{cols}_i32] [%c{cols}_i32, %c1_i32] : !kapy.ptr<1> -> {dyn}
    %gg = kapy.mk_global %gate[%c0_i32] [%rows, %c1_i32] [%c1_i32, %c1_i32] : !kapy.ptr<1> -> {dyn32}
    %go = kapy.mk_global %out[%c0_i32] [%rows, %c{cols}_i32] [%c{cols}_i32, %c1_i32] : !kapy.ptr<1> -> {dyn}
    %sx = kapy.sv_global %gx[%row0 : %row1, %c0_i32 : %c{cols}_i32] : {dyn} -> {t16}, #global>
    %sy = kapy.sv_global %gy[%row0 : %row1, %c0_i32 : %c{cols}_i32] : {dyn} -> {t16}, #global>
    %sg = kapy.sv_global %gg[%row0 : %row1, %c0_i32 : %c1_i32] : {dyn32} -> {c32}, #global>
    %so = kapy.sv_global %go[%row0 : %row1, %c0_i32 : %c{cols}_i32] : {dyn} -> {t16}, #global>
    %x16 = kapy.ld_global %sx : {t16}, #global> -> {t16}, #values>
    %y16 = kapy.ld_global %sy : {t16}, #global> -> {t16}, #values>
    %gv = kapy.ld_global %sg : {c32}, #global> -> {c32}, #values>
    %xf = kapy.fptofp %x16 : {t16}, #values> to {t32}, #values>
    %yf = kapy.fptofp %y16 : {t16}, #values> to {t32}, #values>
    %nx = arith.negf %xf : {t32}, #values>
    %ex = math.exp %nx : {t32}, #values>
    %ones = kapy.splat %one : f32 -> {t32}, #values>
    %den = arith.addf %ex, %ones : {t32}, #values>
    %sig = arith.divf %xf, %den : {t32}, #values>
    %prod = arith.mulf %sig, %yf : {t32}, #values>
    %gb = kapy.broadcast %gv : {c32}, #values> -> {t32}, #values>
    %scaled = arith.mulf %prod, %gb : {t32}, #values>
    %r = kapy.fptofp %scaled {{rounding_mode = 1 : i32}} : {t32}, #values> to {t16}, #values>
    kapy.st_global %r, %so : {t16}, #values>, {t16}, #global>
    kapy.return
""".format(rpp=rows_per_warp * num_warps, rpw=rows_per_warp, cols=cols, dyn=dyn, dyn32=dyn32, t16=t16, t32=t32, c32=c32)
    return (HEADER + "module attributes {kapy.num_warps = %d : i64} {\n" % num_warps +
            "  kapy.func public @gated_kernel(%x: !kapy.ptr<1>, %y: !kapy.ptr<1>, %gate: !kapy.ptr<1>, %out: !kapy.ptr<1>, %rows: i32) {\n" +
            body + "  }\n}\n")


def aliasing_program(rows_per_warp=4, cols=128, num_warps=2, dtype="f16"):
    """Stores into memory that earlier loads read: out = (x + y) * x with the values x had on entry, although x is overwritten
    with y between the loads and the arithmetic's use; then x <- x + x in place (x now holding y)."""
    t = "tensor<%dx%dx%s" % (rows_per_warp, cols, dtype)
    dyn = "tensor<?x?x%s, #global>" % dtype
    body = _consts([0, 1, rows_per_warp, rows_per_warp * num_warps, cols])
    body += """    %pid = kapy.program_id {{axis = 0 : i32}} : i32
    %warp = kapy.warp_id : i32
    %p0 = arith.muli %pid, %c{rpp}_i32 : i32
    %w0 = arith.muli %warp, %c{rpw}_i32 : i32
    %row0 = arith.addi %p0, %w0 : i32
    %row1 = arith.addi %row0, %c{rpw}_i32 : i32
    %gx = kapy.mk_global %x[%c0_i32] [%rows, %c{cols}_i32] [%c{cols}_i32, %c1_i32] : !kapy.ptr<1> -> {dyn}
    %gy = kapy.mk_global %y[%c0_i32] [%rows, %c{cols}_i32] [%c{cols}_i32, %c1_i32] : !kapy.ptr<1> -> {dyn}
    %go = kapy.mk_global %out[%c0_i32] [%rows, %c{cols}_i32] [%c{cols}_i32, %c1_i32] : !kapy.ptr<1> -> {dyn}
    %sx = kapy.sv_global %gx[%row0 : %row1, %c0_i32 : %c{cols}_i32] : {dyn} -> {t}, #global>
    %sy = kapy.sv_global %gy[%row0 : %row1, %c0_i32 : %c{cols}_i32] : {dyn} -> {t}, #global>
    %so = kapy.sv_global %go[%row0 : %row1, %c0_i32 : %c{cols}_i32] : {dyn} -> {t}, #global>
    %vx = kapy.ld_global %sx : {t}, #global> -> {t}, #values>
    %vy = kapy.ld_global %sy : {t}, #global> -> {t}, #values>
    %a = arith.addf %vx, %vy : {t}, #values>
    kapy.st_global %vy, %sx : {t}, #values>, {t}, #global>
    %b = arith.mulf %a, %vx : {t}, #values>
    kapy.st_global %b, %so : {t}, #values>, {t}, #global>
    %x2 = kapy.ld_global %sx : {t}, #global> -> {t}, #values>
    %d = arith.addf %x2, %x2 : {t}, #values>
    kapy.st_global %d, %sx : {t}, #values>, {t}, #global>
    kapy.return
""".format(rpp=rows_per_warp * num_warps, rpw=rows_per_warp, cols=cols, dyn=dyn, t=t)
    return (HEADER + "module attributes {kapy.num_warps = %d : i64} {\n" % num_warps +
            "  kapy.func public @aliasing_kernel(%x: !kapy.ptr<1>, %y: !kapy.ptr<1>, %out: !kapy.ptr<1>, %rows: i32) {\n" + body + "  }\n}\n")


def block_sum_program(rows_per_warp=4, block_cols=64, num_warps=2, dtype="f16"):
    """out[r, 0:block_cols] = 0.25 + sum over the column blocks j of tanh(x[r, j*block_cols:(j+1)*block_cols]) * 0.5, accumulated
    in f32 by an scf.for that carries the accumulator, rounded once at the end.  %cols is a run-time argument."""
    t16, t32 = "tensor<%dx%dx%s" % (rows_per_warp, block_cols, dtype), "tensor<%dx%dxf32" % (rows_per_warp, block_cols)
    dyn = "tensor<?x?x%s, #global>" % dtype
    body = _consts([0, 1, rows_per_warp, rows_per_warp * num_warps, block_cols])
    body += """    %half = arith.constant 0.5 : f32
    %start = arith.constant dense<2.500000e-01> : {t32}, #values>
    %pid = kapy.program_id {{axis = 0 : i32}} : i32
    %warp = kapy.warp_id : i32
    %p0 = arith.muli %pid, %c{rpp}_i32 : i32
    %w0 = arith.muli %warp, %c{rpw}_i32 : i32
    %row0 = arith.addi %p0, %w0 : i32
    %row1 = arith.addi %row0, %c{rpw}_i32 : i32
    %gx = kapy.mk_global %x[%c0_i32] [%rows, %cols] [%cols, %c1_i32] : !kapy.ptr<1> -> {dyn}
    %go = kapy.mk_global %out[%c0_i32] [%rows, %c{bc}_i32] [%c{bc}_i32, %c1_i32] : !kapy.ptr<1> -> {dyn}
    %so = kapy.sv_global %go[%row0 : %row1, %c0_i32 : %c{bc}_i32] : {dyn} -> {t16}, #global>
    %halves = kapy.splat %half : f32 -> {t32}, #values>
    %blocks = arith.divui %cols, %c{bc}_i32 : i32
    %sum = scf.for %j = %c0_i32 to %blocks step %c1_i32 iter_args(%acc = %start) -> ({t32}, #values>)  : i32 {{
      %c0 = arith.muli %j, %c{bc}_i32 : i32
      %c1 = arith.addi %c0, %c{bc}_i32 : i32
      %sx = kapy.sv_global %gx[%row0 : %row1, %c0 : %c1] : {dyn} -> {t16}, #global>
      %v = kapy.ld_global %sx : {t16}, #global> -> {t16}, #values>
      %vf = kapy.fptofp %v : {t16}, #values> to {t32}, #values>
      %th = math.tanh %vf : {t32}, #values>
      %sc = arith.mulf %th, %halves : {t32}, #values>
      %next = arith.addf %acc, %sc : {t32}, #values>
      scf.yield %next : {t32}, #values>
    }}
    %r = kapy.fptofp %sum {{rounding_mode = 1 : i32}} : {t32}, #values> to {t16}, #values>
    kapy.st_global %r, %so : {t16}, #values>, {t16}, #global>
    kapy.return
""".format(rpp=rows_per_warp * num_warps, rpw=rows_per_warp, bc=block_cols, dyn=dyn, t16=t16, t32=t32)
    return (HEADER + "module attributes {kapy.num_warps = %d : i64} {\n" % num_warps +
            "  kapy.func public @block_sum_kernel(%x: !kapy.ptr<1>, %out: !kapy.ptr<1>, %rows: i32, %cols: i32) {\n" + body + "  }\n}\n")


def scaled_transpose_program(tile=32, scale=0.5, dtype="f16"):
    """out[j, i] = x[i, j] * scale over tile x tile blocks, one block per program: ld_global, kapy.transpose, kapy.splat of
    a scalar constant, mulf, st_global."""
    t = "tensor<%dx%dx%s" % (tile, tile, dtype)
    dyn = "tensor<?x?x%s, #global>" % dtype
    body = _consts([0, 1, tile])
    body += """    %scale = arith.constant {scale:e} : {dtype}
    %pi = kapy.program_id {{axis = 0 : i32}} : i32
    %pj = kapy.program_id {{axis = 1 : i32}} : i32
    %i0 = arith.muli %pi, %c{tile}_i32 : i32
    %i1 = arith.addi %i0, %c{tile}_i32 : i32
    %j0 = arith.muli %pj, %c{tile}_i32 : i32
    %j1 = arith.addi %j0, %c{tile}_i32 : i32
    %gx = kapy.mk_global %x[%c0_i32] [%m, %n] [%n, %c1_i32] : !kapy.ptr<1> -> {dyn}
    %go = kapy.mk_global %out[%c0_i32] [%n, %m] [%m, %c1_i32] : !kapy.ptr<1> -> {dyn}
    %sx = kapy.sv_global %gx[%i0 : %i1, %j0 : %j1] : {dyn} -> {t}, #global>
    %so = kapy.sv_global %go[%j0 : %j1, %i0 : %i1] : {dyn} -> {t}, #global>
    %v = kapy.ld_global %sx : {t}, #global> -> {t}, #values>
    %vt = kapy.transpose %v : {t}, #values> -> {t}, #values>
    %k = kapy.splat %scale : {dtype} -> {t}, #values>
    %y = arith.mulf %vt, %k : {t}, #values>
    kapy.st_global %y, %so : {t}, #values>, {t}, #global>
    kapy.return
""".format(tile=tile, scale=scale, dtype=dtype, dyn=dyn, t=t)
    return (HEADER + "module attributes {kapy.num_warps = 1 : i64} {\n"
            "  kapy.func public @scaled_transpose_kernel(%x: !kapy.ptr<1>, %out: !kapy.ptr<1>, %m: i32, %n: i32) {\n" + body + "  }\n}\n")


def exchange_program(rows_per_warp=16, cols=64, num_warps=4, dtype="f16", barrier=True):
    """A program whose warps exchange data through shared memory: warp w stores its rows of x, scaled by 2, into its slot
    of one shared buffer; after the barrier it reads the slot of warp (w + 1) % num_warps and stores that to its rows of out.
    So out[block w] = 2 * x[block (w + 1) % num_warps] within every program's group of num_warps row blocks - which only
    comes out right if every warp has stored before any warp loads."""
    t = "tensor<%dx%dx%s" % (rows_per_warp, cols, dtype)
    full = "tensor<%dx%dx%s, #shared>" % (rows_per_warp * num_warps, cols, dtype)
    dyn = "tensor<?x?x%s, #global>" % dtype
    body = _consts([0, 1, rows_per_warp, rows_per_warp * num_warps, cols, num_warps])
    body += """    %two = arith.constant dense<2.000000e+00> : {t}, #values>
    %pid = kapy.program_id {{axis = 0 : i32}} : i32
    %warp = kapy.warp_id : i32
    %p0 = arith.muli %pid, %c{rpp}_i32 : i32
    %w0 = arith.muli %warp, %c{rpw}_i32 : i32
    %w1 = arith.addi %w0, %c{rpw}_i32 : i32
    %row0 = arith.addi %p0, %w0 : i32
    %row1 = arith.addi %row0, %c{rpw}_i32 : i32
    %next = arith.addi %warp, %c1_i32 : i32
    %peer = arith.remui %next, %c{nw}_i32 : i32
    %q0 = arith.muli %peer, %c{rpw}_i32 : i32
    %q1 = arith.addi %q0, %c{rpw}_i32 : i32
    %gx = kapy.mk_global %x[%c0_i32] [%rows, %c{cols}_i32] [%c{cols}_i32, %c1_i32] : !kapy.ptr<1> -> {dyn}
    %go = kapy.mk_global %out[%c0_i32] [%rows, %c{cols}_i32] [%c{cols}_i32, %c1_i32] : !kapy.ptr<1> -> {dyn}
    %sx = kapy.sv_global %gx[%row0 : %row1, %c0_i32 : %c{cols}_i32] : {dyn} -> {t}, #global>
    %so = kapy.sv_global %go[%row0 : %row1, %c0_i32 : %c{cols}_i32] : {dyn} -> {t}, #global>
    %buf = kapy.mk_shared {{kapy.row_major = true}} : {full}
    %mine = kapy.sv_shared %buf[%w0 : %w1, %c0_i32 : %c{cols}_i32] : {full} -> {t}, #shared>
    %theirs = kapy.sv_shared %buf[%q0 : %q1, %c0_i32 : %c{cols}_i32] : {full} -> {t}, #shared>
    %vx = kapy.ld_global %sx : {t}, #global> -> {t}, #values>
    %v2 = arith.mulf %vx, %two : {t}, #values>
    kapy.st_shared %v2, %mine : {t}, #values>, {t}, #shared>
{barrier}    %vy = kapy.ld_shared %theirs : {t}, #shared> -> {t}, #values>
    kapy.st_global %vy, %so : {t}, #values>, {t}, #global>
    kapy.return
""".format(rpp=rows_per_warp * num_warps, rpw=rows_per_warp, cols=cols, dyn=dyn, t=t, full=full, nw=num_warps,
           barrier="    nvvm.barrier0\n" if barrier else "")
    return (HEADER + "module attributes {kapy.num_warps = %d : i64} {\n" % num_warps +
            "  kapy.func public @exchange_kernel(%x: !kapy.ptr<1> {kapy.alignment = 128 : i64}, %out: !kapy.ptr<1> {kapy.alignment = 128 : i64}, "
            "%rows: i32 {kapy.alignment = 4 : i64}) {\n" + body + "  }\n}\n")


def exchange_loop_program(rows_per_warp=8, cols=64, num_warps=4, steps=3, dtype="f16"):
    """The same exchange inside an scf.for that carries the tile: every step each warp adds 1 to its tile, parks it in its slot,
    and continues with the tile of warp (w + 1) % num_warps; after `steps` steps block w of out is x[block (w + steps) % num_warps]
    + steps.  Every step reuses the one shared buffer, so it needs a barrier before the stores as well as before the loads."""
    t = "tensor<%dx%dx%s" % (rows_per_warp, cols, dtype)
    full = "tensor<%dx%dx%s, #shared>" % (rows_per_warp * num_warps, cols, dtype)
    dyn = "tensor<?x?x%s, #global>" % dtype
    body = _consts([0, 1, rows_per_warp, rows_per_warp * num_warps, cols, num_warps, steps])
    body += """    %one = arith.constant dense<1.000000e+00> : {t}, #values>
    %pid = kapy.program_id {{axis = 0 : i32}} : i32
    %warp = kapy.warp_id : i32
    %p0 = arith.muli %pid, %c{rpp}_i32 : i32
    %w0 = arith.muli %warp, %c{rpw}_i32 : i32
    %w1 = arith.addi %w0, %c{rpw}_i32 : i32
    %row0 = arith.addi %p0, %w0 : i32
    %row1 = arith.addi %row0, %c{rpw}_i32 : i32
    %next = arith.addi %warp, %c1_i32 : i32
    %peer = arith.remui %next, %c{nw}_i32 : i32
    %q0 = arith.muli %peer, %c{rpw}_i32 : i32
    %q1 = arith.addi %q0, %c{rpw}_i32 : i32
    %gx = kapy.mk_global %x[%c0_i32] [%rows, %c{cols}_i32] [%c{cols}_i32, %c1_i32] : !kapy.ptr<1> -> {dyn}
    %go = kapy.mk_global %out[%c0_i32] [%rows, %c{cols}_i32] [%c{cols}_i32, %c1_i32] : !kapy.ptr<1> -> {dyn}
    %sx = kapy.sv_global %gx[%row0 : %row1, %c0_i32 : %c{cols}_i32] : {dyn} -> {t}, #global>
    %so = kapy.sv_global %go[%row0 : %row1, %c0_i32 : %c{cols}_i32] : {dyn} -> {t}, #global>
    %buf = kapy.mk_shared {{kapy.row_major = true}} : {full}
    %mine = kapy.sv_shared %buf[%w0 : %w1, %c0_i32 : %c{cols}_i32] : {full} -> {t}, #shared>
    %theirs = kapy.sv_shared %buf[%q0 : %q1, %c0_i32 : %c{cols}_i32] : {full} -> {t}, #shared>
    %v0 = kapy.ld_global %sx : {t}, #global> -> {t}, #values>
    %last = scf.for %i = %c0_i32 to %c{steps}_i32 step %c1_i32 iter_args(%v = %v0) -> ({t}, #values>) : i32 {{
      %v1 = arith.addf %v, %one : {t}, #values>
      nvvm.barrier0
      kapy.st_shared %v1, %mine : {t}, #values>, {t}, #shared>
      nvvm.barrier0
      %vn = kapy.ld_shared %theirs : {t}, #shared> -> {t}, #values>
      scf.yield %vn : {t}, #values>
    }}
    kapy.st_global %last, %so : {t}, #values>, {t}, #global>
    kapy.return
""".format(rpp=rows_per_warp * num_warps, rpw=rows_per_warp, cols=cols, dyn=dyn, t=t, full=full, nw=num_warps, steps=steps)
    return (HEADER + "module attributes {kapy.num_warps = %d : i64} {\n" % num_warps +
            "  kapy.func public @exchange_loop_kernel(%x: !kapy.ptr<1> {kapy.alignment = 128 : i64}, %out: !kapy.ptr<1> {kapy.alignment = 128 : i64}, "
            "%rows: i32 {kapy.alignment = 4 : i64}) {\n" + body + "  }\n}\n")


def column_softmax_program(rows=64, cols_per_warp=64, num_warps=2, dtype="f16"):
    """out[:, c] = softmax(x[:, c]) over the `rows` rows of the matrix, in f32: the reduces run along axis 0 and their [1 x cols]
    results are broadcast back down the columns.  A program instance owns cols_per_warp * num_warps columns."""
    t16, t32 = "tensor<%dx%dx%s" % (rows, cols_per_warp, dtype), "tensor<%dx%dxf32" % (rows, cols_per_warp)
    c32 = "tensor<1x%dxf32, #values>" % cols_per_warp
    dyn = "tensor<?x?x%s, #global>" % dtype
    body = _consts([0, 1, rows, cols_per_warp, cols_per_warp * num_warps])
    body += """    %pid = kapy.program_id {{axis = 0 : i32}} : i32
    %warp = kapy.warp_id : i32
    %p0 = arith.muli %pid, %c{cpp}_i32 : i32
    %w0 = arith.muli %warp, %c{cpw}_i32 : i32
    %col0 = arith.addi %p0, %w0 : i32
    %col1 = arith.addi %col0, %c{cpw}_i32 : i32
    %gx = kapy.mk_global %x[%c0_i32] [%c{rows}_i32, %cols] [%cols, %c1_i32] : !kapy.ptr<1> -> {dyn}
    %go = kapy.mk_global %out[%c0_i32] [%c{rows}_i32, %cols] [%cols, %c1_i32] : !kapy.ptr<1> -> {dyn}
    %sx = kapy.sv_global %gx[%c0_i32 : %c{rows}_i32, %col0 : %col1] : {dyn} -> {t16}, #global>
    %so = kapy.sv_global %go[%c0_i32 : %c{rows}_i32, %col0 : %col1] : {dyn} -> {t16}, #global>
    %x16 = kapy.ld_global %sx : {t16}, #global> -> {t16}, #values>
    %xf = kapy.fptofp %x16 : {t16}, #values> to {t32}, #values>
    %m = kapy.reduce %xf {{axis = 0 : i32}} lambda(%lhs: f32, %rhs: f32) {{
      %r = arith.maximumf %lhs, %rhs : f32
      kapy.return %r : f32
    }} : {t32}, #values> -> {c32}
    %mb = kapy.broadcast %m : {c32} -> {t32}, #values>
    %d = arith.subf %xf, %mb : {t32}, #values>
    %e = math.exp %d : {t32}, #values>
    %s = kapy.reduce %e {{axis = 0 : i32}} lambda(%lhs: f32, %rhs: f32) {{
      %r = arith.addf %lhs, %rhs : f32
      kapy.return %r : f32
    }} : {t32}, #values> -> {c32}
    %sb = kapy.broadcast %s : {c32} -> {t32}, #values>
    %q = arith.divf %e, %sb : {t32}, #values>
    %y = kapy.fptofp %q {{rounding_mode = 1 : i32}} : {t32}, #values> to {t16}, #values>
    kapy.st_global %y, %so : {t16}, #values>, {t16}, #global>
    kapy.return
""".format(cpp=cols_per_warp * num_warps, cpw=cols_per_warp, rows=rows, dyn=dyn, t16=t16, t32=t32, c32=c32)
    return (HEADER + "module attributes {kapy.num_warps = %d : i64} {\n" % num_warps +
            "  kapy.func public @column_softmax_kernel(%x: !kapy.ptr<1>, %out: !kapy.ptr<1>, %cols: i32) {\n" + body + "  }\n}\n")
