"""CPU checks of the textual front-end: the programs of kapy_programs.py (the reference fixtures' op set and
structure) parse, and malformed or unsupported text is rejected with the line it occurs on."""
import pytest

import kapy_hip as kh
import kapy_programs as kp


def test_fixture_shaped_programs_parse():
    assert kh.parse_mlir(kp.binary_program()) == (4, 22, 4)
    n_args, n_ops, warps = kh.parse_mlir(kp.reduce_program(num_warps=2))
    assert (n_args, warps) == (3, 2) and n_ops == 21    # 19 ops and the two of the combiner region
    n_args, n_ops, warps = kh.parse_mlir(kp.matmul_program(), "matmul_kernel")
    assert (n_args, warps) == (6, 4) and n_ops > 60


def test_programs_with_casts_math_broadcast_transpose_and_splat_parse():
    assert kh.parse_mlir(kp.softmax_program())[0] == 3
    assert kh.parse_mlir(kp.scaled_transpose_program())[0] == 4


def test_function_is_found_by_name():
    two = kp.binary_program().rstrip()[:-1] + kp.reduce_program().split("{\n", 1)[1]
    assert kh.parse_mlir(two, "reduce_kernel")[0] == 3
    assert kh.parse_mlir(two, "binary_kernel")[0] == 4
    assert kh.parse_mlir(two)[0] == 4
    with pytest.raises(kh.KapyError) as e:
        kh.parse_mlir(two, "absent")
    assert e.value.status == -1 and "absent" in e.value.message


def test_unsupported_op_is_named_with_its_line():
    text = kp.binary_program().replace("arith.addf", "math.atan")
    with pytest.raises(kh.KapyError) as e:
        kh.parse_mlir(text)
    assert e.value.status == -3 and "math.atan" in e.value.message and "line " in e.value.message


@pytest.mark.parametrize("damage", [
    lambda t: t.replace("tensor<4x128xf16, #values>", "tensor<4x128xq7, #values>"),   # unknown element type
    lambda t: t.replace("%vo = arith.addf", "%vo arith.addf"),                        # missing '='
    lambda t: t[:t.rindex("kapy.return")],                                            # unterminated region
])
def test_malformed_text_is_rejected(damage):
    with pytest.raises(kh.KapyError) as e:
        kh.parse_mlir(damage(kp.binary_program()))
    assert e.value.status == -1


def test_run_needs_a_device_and_matching_arguments():
    import ctypes as C
    text = kp.binary_program().encode()
    args = (kh.MlirArg * 4)()
    grid = (C.c_int32 * 3)(1, 1, 1)
    assert kh.lib().kapy_run_mlir(text, None, args, 3, grid, None) == -1     # wrong argument count
    assert "takes 4 arguments" in kh.last_error()
    assert kh.lib().kapy_run_mlir(text, None, args, 4, (C.c_int32 * 3)(0, 1, 1), None) == -1


REFERENCE_FIXTURES = "/root/reference/test/Conversion/KapyToKgpu"


@pytest.mark.skipif(not __import__("os").path.isdir(REFERENCE_FIXTURES), reason="the reference tree is not present")
@pytest.mark.parametrize("name,n_args,n_ops,warps", [
    ("elementwise_add", 4, 21, 2), ("reduce_sum", 3, 21, 2), ("matmul", 6, 126, 4)])
def test_reference_fixtures_parse_unchanged(name, n_args, n_ops, warps):
    text = open("%s/%s.mlir" % (REFERENCE_FIXTURES, name)).read()
    assert kh.parse_mlir(text, name + "_kernel") == (n_args, n_ops, warps)


def _lines(text, needle):
    return [k + 1 for k, line in enumerate(text.split("\n")) if needle in line]


def test_analysis_of_programs_without_shared_memory_is_empty():
    assert kh.analyze_mlir(kp.binary_program()) == (0, [], [])
    assert kh.analyze_mlir(kp.reduce_program()) == (0, [], [])


def test_analysis_places_the_double_buffers_and_finds_the_barriers():
    text = kp.matmul_program(64, 64, 32)
    total, offsets, barriers = kh.analyze_mlir(text)
    # four buffers of 128x32 f16, all live from their mk_shared to the last ld_matrix: end to end
    assert (total, offsets) == (4 * 8192, [0, 8192, 16384, 24576])
    waits = _lines(text, "kapy.cp_async_wait_group")
    # every wait_group gets a barrier after it; inside the loop the first ld_matrix reads through a select that may
    # point at the buffer the cp_async just before it is filling, so it needs one before it
    first_ld_in_loop = [l for l in _lines(text, "kapy.ld_matrix") if l > _lines(text, "scf.for")[0]][0]
    assert sorted(barriers) == sorted([-w for w in waits] + [first_ld_in_loop])


def test_analysis_shares_memory_between_buffers_that_are_never_live_together():
    # two phases, each with a buffer of its own: the second buffer is made after the last use of the first
    text = kp.phases_program()
    total, offsets, barriers = kh.analyze_mlir(text)
    # %first is dead when %second and %third are made: they start at 0 again; %second and %third live together
    assert offsets == [0, 0, 4096] and total == 4096 + 8192
    # the wait_group's own barrier; st_shared into %third writes bytes that ld_matrix has read as %first (the reuse
    # is a write after read); ld_shared of %third after the st_shared is a read after write
    assert sorted(barriers) == sorted([-_lines(text, "cp_async_wait_group")[0], _lines(text, "kapy.st_shared")[0],
                                       _lines(text, "%u = kapy.ld_shared")[0]])


@pytest.mark.skipif(not __import__("os").path.isdir(REFERENCE_FIXTURES), reason="the reference tree is not present")
def test_analysis_of_the_reference_matmul_fixture():
    text = open(REFERENCE_FIXTURES + "/matmul.mlir").read()
    total, offsets, barriers = kh.analyze_mlir(text)
    assert (total, offsets) == (65536, [0, 16384, 32768, 49152])          # four 128x64 f16 tiles
    waits = _lines(text, "kapy.cp_async_wait_group")
    loop = _lines(text, "scf.for")[0]
    refill = [l for l in _lines(text, "kapy.cp_async_global_to_shared") if l > loop][0]
    # a barrier after each wait_group, and one before the loop's refill of the buffer that ld_matrix has just read
    assert sorted(barriers) == sorted([-w for w in waits] + [refill])


def test_a_program_beyond_the_lds_is_refused_before_anything_runs():
    import ctypes as C
    text = kp.matmul_program(64, 64, 32).replace("tensor<128x32xf16, #shared>", "tensor<128x256xf16, #shared>") \
        .replace("tensor<32x128xf16, #shared>", "tensor<256x128xf16, #shared>")
    total, _, _ = kh.analyze_mlir(text)
    assert total == 4 * 65536
    args = (kh.MlirArg * 6)()
    assert kh.lib().kapy_run_mlir(text.encode(), None, args, 6, (C.c_int32 * 3)(1, 1, 1), None) == -3
    assert "shared memory" in kh.last_error() and "163840" in kh.last_error()


def test_analysis_finds_the_barrier_between_warps_that_exchange_tiles():
    # a store into one sub-view of a buffer and a load from another sub-view of it: the views' offsets depend on the warp id,
    # so the two accesses may touch the same bytes and the load needs a barrier; the program's own nvvm.barrier0 is honoured
    text = kp.exchange_program(barrier=False)
    total, offsets, barriers = kh.analyze_mlir(text)
    assert (total, offsets) == (4 * 16 * 64 * 2, [0])
    assert barriers == [_lines(text, "kapy.ld_shared")[0]]
    assert kh.analyze_mlir(kp.exchange_program(barrier=True))[2] == []
    # in the loop the program places both barriers itself (before the stores: the previous step's loads; before the loads)
    assert kh.analyze_mlir(kp.exchange_loop_program())[2] == []


@pytest.mark.parametrize("program,damage,named", [
    (kp.binary_program, lambda t: t.replace("%vo = arith.addf %vx, %vy", "%vo = arith.addf %vx"), "arith.addf"),                     # an operand short
    (kp.binary_program, lambda t: t.replace("%vo = arith.addf %vx, %vy", "arith.addf %vx, %vy"), "arith.addf"),                     # no result
    (kp.binary_program, lambda t: t.replace("kapy.st_global %vo, %so", "kapy.st_global %vo"), "kapy.st_global"),
    (kp.exchange_program, lambda t: t.replace("%mine = kapy.sv_shared %buf[%w0 : %w1, %c0_i32 : %c64_i32]", "%mine = kapy.sv_shared %buf[%w0 : %w1]"), "kapy.sv_shared"),
    (kp.exchange_loop_program, lambda t: t.replace("%last = scf.for", "%last, %more = scf.for"), "scf.for"),                       # more results than carried values
])
def test_an_op_written_with_too_few_operands_or_results_is_refused_before_it_runs(program, damage, named):
    text = program()
    broken = damage(text)
    assert broken != text
    with pytest.raises(kh.KapyError) as e:
        kh.parse_mlir(broken)
    assert e.value.status == -1 and named in e.value.message and "line " in e.value.message
    with pytest.raises(kh.KapyError):
        kh.analyze_mlir(broken)
