"""GPU parity of the Softmax Function against the fp32 oracle; mirrors the
reference's tritonformer/test_softmax.py (fp32 input, dy = 0.1*randn, atol 1e-4)
and adds the 16-bit dtypes."""
import numpy as np
import pytest
import torch

import tritonformer_amd as T
from oracle import ref_torch as R
from tests.util import NUM_TEST, assert_close

pytestmark = pytest.mark.gpu
rng = np.random.RandomState(0)
DIMS = [(int(b), int(r), int(c)) for b in rng.randint(1, 8, size=NUM_TEST) for r in rng.randint(256, 512, size=1)
        for c in rng.randint(64, 1024, size=NUM_TEST)]
EDGE = [(1, 1, 1), (1, 3, 5), (2, 64, 1024), (1, 17, 2048), (1, 9, 2052), (1, 4, 9000)]


@pytest.mark.parametrize("dims", DIMS + EDGE)
def test_softmax_fp32_fwd_bwd(dims, dev):
    g = torch.Generator().manual_seed(sum(dims))
    x = torch.randn(*dims, generator=g)
    dy = 0.1 * torch.randn(*dims, generator=g)
    xd = x.to(dev).requires_grad_(True)
    y = T.Softmax.apply(xd)
    assert y.dtype == torch.float32          # dtype preserved, no autocast hook (reference softmax.py:9-10)
    y.backward(dy.to(dev))
    y_ref = R.softmax(x)
    assert_close(y, y_ref, torch.float32, f"y {dims}")          # atol 1e-4 as test_softmax.py:44
    assert_close(xd.grad, R.softmax_bwd(y_ref, dy), torch.float32, f"dx {dims}")
    assert (y.sum(-1) - 1).abs().max() < 1e-5
    assert xd.grad.sum(-1).abs().max() < 1e-5


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("dims", [(2, 100, 777), (3, 64, 1024)])
def test_softmax_16bit(dims, dtype, dev):
    g = torch.Generator().manual_seed(1)
    x = torch.randn(*dims, generator=g).to(dtype)
    dy = (0.1 * torch.randn(*dims, generator=g)).to(dtype)
    xd = x.to(dev).requires_grad_(True)
    y = T.Softmax.apply(xd)
    keep = dy.to(dev)
    before = keep.clone()
    y.backward(keep)
    assert torch.equal(keep, before)          # grad_out is not overwritten (the reference does, softmax.py:101-111)
    assert_close(y, R.softmax(x), dtype, "y", atol=2e-3)
    assert_close(xd.grad, R.softmax_bwd(y.detach().cpu(), dy), dtype, "dx", atol=2e-3)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16, torch.float32])
@pytest.mark.parametrize("dims", [(1, 5, 50304), (2, 3, 4104), (1, 2, 33000), (1, 2, 65536), (1, 2, 65544), (1, 3, 50301)])
def test_softmax_long_rows(dims, dtype, dev):
    """Rows beyond what one wave holds in registers (4096 16-bit / 2048 fp32 elements): a workgroup per
    row, 4 / 8 / 16 chunks per thread (the fp32 row of 65536 re-reads dy in the backward pass), up to
    65536 elements; longer or unaligned rows (65544, 50301) take the scalar kernels.  Against the fp32
    oracle; rows sum to one, gradients to zero."""
    g = torch.Generator().manual_seed(3)
    x = (torch.randn(*dims, generator=g) * 2).to(dtype)
    dy = torch.randn(*dims, generator=g).to(dtype)
    xd = x.to(dev).requires_grad_(True)
    y = T.Softmax.apply(xd)
    y.backward(dy.to(dev))
    y_ref = R.softmax(x.float())
    tol = dict(atol=1e-6, rtol=1e-4) if dtype == torch.float32 else dict(atol=1e-5, rtol=4e-3 if dtype == torch.float16 else 2e-2)
    assert_close(y, y_ref, dtype, f"y {dims}", **tol)
    assert_close(xd.grad, R.softmax_bwd(y.detach().float().cpu(), dy.float()), dtype, f"dx {dims}",
                 atol=tol["atol"] * 10, rtol=tol["rtol"])
    assert (y.float().sum(-1) - 1).abs().max() < (1e-4 if dtype == torch.float32 else 2e-2)
