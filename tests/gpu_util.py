"""Helpers for the GPU parity tests: move numpy storage arrays to device memory and back through
torch (plumbing only), and build descriptors over them for both the oracle and the product."""
import numpy as np
import torch

import kapy_hip as kh

_TORCH_STORAGE = {1: torch.uint8, 2: torch.int16, 4: torch.int32}


def to_dev(arr):
    """numpy storage array (any dtype of 1/2/4 bytes) -> flat device tensor holding the same bits."""
    a = np.ascontiguousarray(arr)
    t = torch.from_numpy(a.view({1: np.uint8, 2: np.int16, 4: np.int32}[a.itemsize]).reshape(-1))
    return t.cuda()


def dev_zeros(n, itemsize, fill=0):
    return torch.full((n,), fill, dtype=_TORCH_STORAGE[itemsize], device="cuda")


def to_host(t, np_dtype, shape=None):
    a = t.cpu().numpy().view(np_dtype)
    return a.reshape(shape) if shape is not None else a


def dglobal(t, size0, size1, stride0, stride1, dtype, dynamic_offset=0):
    return kh.mk_global(t.data_ptr(), size0, size1, stride0, stride1, dtype, dynamic_offset)


def sync():
    torch.cuda.synchronize()


def ulp_diff_f16(a_bits, b_bits):
    """Distance in units of the last place between two uint16 arrays of f16 (or bf16) bit patterns,
    measured on the monotone integer line (sign-magnitude -> offset)."""
    def line(x):
        x = x.astype(np.int32)
        return np.where(x & 0x8000, -(x & 0x7FFF), x & 0x7FFF)
    return np.abs(line(a_bits) - line(b_bits))
