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


def test_function_is_found_by_name():
    two = kp.binary_program().rstrip()[:-1] + kp.reduce_program().split("{\n", 1)[1]
    assert kh.parse_mlir(two, "reduce_kernel")[0] == 3
    assert kh.parse_mlir(two, "binary_kernel")[0] == 4
    assert kh.parse_mlir(two)[0] == 4
    with pytest.raises(kh.KapyError) as e:
        kh.parse_mlir(two, "absent")
    assert e.value.status == -1 and "absent" in e.value.message


def test_unsupported_op_is_named_with_its_line():
    text = kp.binary_program().replace("arith.addf", "math.exp")
    with pytest.raises(kh.KapyError) as e:
        kh.parse_mlir(text)
    assert e.value.status == -3 and "math.exp" in e.value.message and "line " in e.value.message


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
