"""Shared helpers for the parity tests."""
import ctypes
import os

import numpy as np
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
NUM_TEST = int(os.environ.get("NUM_TEST", "3"))  # random shapes per axis, as in the reference's tests

# Tolerances against fp32 math (stated per dtype): one 16-bit rounding of the
# result is |ref| * 2^-11 (fp16) or |ref| * 2^-8 (bf16); atol covers the
# accumulated rounding of 16-bit inputs for O(1) data.
TOL = {
    torch.float16: dict(atol=1e-2, rtol=1e-3),
    torch.bfloat16: dict(atol=6e-2, rtol=8e-3),
    torch.float32: dict(atol=1e-4, rtol=1e-5),
}


def rel_l2(a, b):
    a, b = a.detach().float().cpu(), b.detach().float().cpu()
    return ((a - b).norm() / (b.norm() + 1e-30)).item()


def assert_close(got, ref, dtype=torch.float16, name="", atol=None, rtol=None):
    got, ref = got.detach().float().cpu(), ref.detach().float().cpu()
    assert got.shape == ref.shape, f"{name}: shape {tuple(got.shape)} vs {tuple(ref.shape)}"
    tol = TOL[dtype]
    atol = tol["atol"] if atol is None else atol
    rtol = tol["rtol"] if rtol is None else rtol
    err = (got - ref).abs()
    bound = atol + rtol * ref.abs()
    bad = err > bound
    assert not bad.any(), (
        f"{name}: {int(bad.sum())} of {bad.numel()} elements outside atol={atol} rtol={rtol}; "
        f"max abs err {err.max().item():.4e}, rel-L2 {rel_l2(got, ref):.3e}"
    )


class RefOps:
    """ctypes view of oracle/libref_ops.so (brute-force C restatement)."""

    def __init__(self):
        self.lib = ctypes.CDLL(os.path.join(ROOT, "oracle", "libref_ops.so"))

    @staticmethod
    def _p(a):
        return a.ctypes.data_as(ctypes.c_void_p)

    def call(self, name, *args):
        conv = []
        for a in args:
            if isinstance(a, np.ndarray):
                conv.append(self._p(a))
            elif a is None:
                conv.append(None)
            elif isinstance(a, float):
                conv.append(ctypes.c_double(a))
            else:
                conv.append(ctypes.c_int(int(a)))
        fn = getattr(self.lib, name)
        fn.restype = None
        fn(*conv)


def f32(t):
    return np.ascontiguousarray(t.detach().float().cpu().numpy())
