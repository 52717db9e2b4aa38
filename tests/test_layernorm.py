"""GPU parity of LayerNorm (forward, dx, dgamma, dbeta) against the fp32 oracle;
mirrors the reference's tritonformer/test_layernorm.py (x = 3.14 + 0.4*randn so the
mean matters, gamma, beta, dy ~ N(0,1); B in [1,32), S, d in [64,1024) arbitrary).
Tolerance: forward and dx atol 1e-2 (+1e-3 relative); dgamma, dbeta relative L2
< 1e-3, as test_layernorm.py:52, 87, 125, 161."""
import numpy as np
import pytest
import torch

import tritonformer_amd as T
from oracle import ref_torch as R
from tests.util import NUM_TEST, assert_close, rel_l2

pytestmark = pytest.mark.gpu
rng = np.random.RandomState(0)
DIMS = [(int(b), int(s), int(d)) for b in rng.randint(1, 16, size=NUM_TEST) for s in rng.randint(64, 512, size=1)
        for d in rng.randint(64, 1024, size=NUM_TEST)]
EDGE = [(1, 1, 8), (1, 3, 7), (2, 64, 768), (3, 77, 333), (1, 130, 1024), (2, 33, 2048), (1, 17, 4096), (1, 9, 5000),
        (1, 5, 8192)]


def run_case(dims, dtype, dev):
    b, s, d = dims
    g = torch.Generator().manual_seed(b * 1000 + d)
    x = (3.14 + 0.4 * torch.randn(b, s, d, generator=g)).to(dtype)
    gamma, beta = torch.randn(d, generator=g).to(dtype), torch.randn(d, generator=g).to(dtype)
    dy = torch.randn(b, s, d, generator=g).to(dtype)
    xd, gd, bd = (t.to(dev).requires_grad_(True) for t in (x, gamma, beta))
    y = T.layer_norm.apply(xd, gd, bd, 1e-5)
    y.backward(dy.to(dev))
    assert_close(y, R.layer_norm(x, gamma, beta, 1e-5), dtype, f"y {dims}")
    dx, dg, db = R.layer_norm_bwd(x, gamma, dy, 1e-5)
    assert_close(xd.grad, dx, dtype, f"dx {dims}", atol=2e-2 if dtype == torch.float16 else 1.5e-1)
    lim = 1e-3 if dtype == torch.float16 else 8e-3
    assert gd.grad.shape == (d,) and bd.grad.shape == (d,)
    assert rel_l2(gd.grad, dg) < lim and rel_l2(bd.grad, db) < lim
    return xd, y


@pytest.mark.parametrize("dims", DIMS + EDGE)
def test_layernorm_fwd_bwd(dims, dev):
    run_case(dims, torch.float16, dev)


@pytest.mark.parametrize("dims", [(2, 64, 768), (3, 77, 333)])
def test_layernorm_bf16(dims, dev):
    run_case(dims, torch.bfloat16, dev)


def test_layernorm_invariants(dev):
    x, y = run_case((2, 128, 1024), torch.float16, dev)
    assert x.grad.float().sum(-1).abs().max() < 0.25          # dx rows sum to ~0 (fp16 rounding of 1024 terms)
    const = torch.full((1, 4, 512), 3.0, dtype=torch.float16, device=dev)
    g = torch.randn(512, device=dev).half()
    b = torch.randn(512, device=dev).half()
    assert torch.equal(T.layer_norm.apply(const, g, b, 1e-5), b.expand(1, 4, 512))   # constant row -> beta


def test_layernorm_headline_shape_and_autocast(dev):
    """(4, 2048, 1024) as in the 410M model, fp32 parameters under autocast."""
    g = torch.Generator().manual_seed(0)
    x = (torch.randn(4, 2048, 1024, generator=g) * 0.5).to(dev).requires_grad_(True)
    gamma = torch.ones(1024, device=dev, requires_grad=True)
    beta = torch.zeros(1024, device=dev, requires_grad=True)
    with torch.autocast("cuda", dtype=torch.float16):
        y = T.layer_norm.apply(x, gamma, beta, 1e-5)
    assert y.dtype == torch.float16
    dy = torch.randn(4, 2048, 1024, generator=g).half().to(dev)
    y.backward(dy)
    assert gamma.grad.dtype == torch.float32 and x.grad.dtype == torch.float32
    xr = x.detach().half()
    assert_close(y, R.layer_norm(xr, gamma.detach(), beta.detach()), name="y")
    dx, dg, db = R.layer_norm_bwd(xr, gamma.detach(), dy)
    assert rel_l2(gamma.grad, dg) < 1e-3 and rel_l2(beta.grad, db) < 1e-3
    assert_close(x.grad, dx, name="dx", atol=2e-2)


def test_layernorm_fp32_parameters_direct(dev):
    """fp32 gamma / beta with 16-bit activations (master parameters under autocast) are
    read by the kernel as they are; their gradients come back in fp32."""
    g = torch.Generator().manual_seed(5)
    x = (1.0 + torch.randn(2, 70, 333, generator=g)).half()
    gamma, beta = torch.randn(333, generator=g), torch.randn(333, generator=g)
    dy = torch.randn(2, 70, 333, generator=g).half()
    xd = x.to(dev).requires_grad_(True)
    gd, bd = gamma.to(dev).requires_grad_(True), beta.to(dev).requires_grad_(True)
    y = T.layer_norm.apply(xd, gd, bd, 1e-5)
    y.backward(dy.to(dev))
    assert y.dtype == torch.float16 and gd.grad.dtype == torch.float32
    assert_close(y, R.layer_norm(x, gamma, beta), name="y")
    dx, dg, db = R.layer_norm_bwd(x, gamma, dy)
    assert_close(xd.grad, dx, name="dx", atol=2e-2)
    assert rel_l2(gd.grad, dg) < 1e-3 and rel_l2(bd.grad, db) < 1e-3


def test_layernorm_rejects_fp32_and_2d(dev):
    with pytest.raises(TypeError):   # reference kernels/layernorm.py:71 asserts fp16
        T.layer_norm.apply(torch.zeros(1, 4, 8, device=dev), torch.ones(8, device=dev), torch.zeros(8, device=dev), 1e-5)
    h = torch.float16
    with pytest.raises(ValueError):
        T.layer_norm.apply(torch.zeros(4, 8, device=dev, dtype=h), torch.ones(8, device=dev, dtype=h),
                           torch.zeros(8, device=dev, dtype=h), 1e-5)
