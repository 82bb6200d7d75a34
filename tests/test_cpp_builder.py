"""The C++ host side (include/kapy_hip.hpp: kapy::OpBuilder, the reference's create_* builder names over the C ABI),
exercised by tests/cpp/builder_test: lowering and error behaviour without a device, the same graphs on the GPU."""
import os
import subprocess

import pytest

HERE = os.path.join(os.path.dirname(os.path.abspath(__file__)), "cpp")
BINARY = os.path.join(HERE, "builder_test")


def _binary():
    if not os.path.exists(BINARY):      # built by __graft_entry__.build(); a source checkout builds it here (host code only)
        subprocess.check_call(["make", "-C", HERE, "-s"])
    return BINARY


def test_builder_lowers_and_refuses_without_a_device():
    out = subprocess.run([_binary(), "cpu"], capture_output=True, text=True, timeout=120)
    assert out.returncode == 0 and "builder cpu ok" in out.stdout, out.stdout + out.stderr


@pytest.mark.gpu
def test_builder_runs_the_graphs_on_the_gpu():
    out = subprocess.run([_binary(), "gpu"], capture_output=True, text=True, timeout=120)
    assert out.returncode == 0 and "builder gpu ok" in out.stdout, out.stdout + out.stderr


@pytest.mark.gpu
def test_the_full_lds_ring_kernel_runs_in_a_process_without_torch():
    """The 256 x 256 x 64 tiles address all 160 KiB of a CU's LDS, declared statically in the code object and checked against the
    runtime's own figures before the first launch; this C++ process links the system HIP runtime directly."""
    out = subprocess.run([_binary(), "gpu256"], capture_output=True, text=True, timeout=120)
    assert out.returncode == 0 and "builder gpu large tile ok" in out.stdout, out.stdout + out.stderr



@pytest.mark.gpu
def test_the_wide_row_major_kernel_runs_in_a_process_without_torch():
    """Row-major x row-major on 256-wide tiles (128 KiB of statically declared LDS, the runtime's figures checked before the first
    launch), picked by the library's own rule, from the C++ process."""
    out = subprocess.run([_binary(), "gpunn256"], capture_output=True, text=True, timeout=120)
    assert out.returncode == 0 and "builder gpu row-major wide ok" in out.stdout, out.stdout + out.stderr
