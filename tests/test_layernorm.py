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
        (1, 5, 8192),
        (31, 1023, 1021), (31, 64, 1016)]  # upper end of the reference's draws (test_layernorm.py:35-37)


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
    xr = x.detach().half().cpu()    # the oracle runs on the CPU
    assert_close(y, R.layer_norm(xr, gamma.detach().cpu(), beta.detach().cpu()), name="y")
    dx, dg, db = R.layer_norm_bwd(xr, gamma.detach().cpu(), dy.cpu())
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


@pytest.mark.parametrize("dims", [(2, 64, 768), (3, 77, 333), (1, 9, 5000), (4, 2048, 1024), (1, 3, 7)])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_add_layernorm_equals_add_then_layernorm(dims, dtype, dev):
    """The fused residual-add + LayerNorm node: forward results are bit-identical to an
    elementwise addition followed by layer_norm (the sum is rounded to the 16-bit type
    before the statistics); the backward adds the residual-stream gradient in fp32
    before one rounding, so dx is compared with the fp32 oracle (atol 2e-2 fp16) and
    with the two-node path."""
    b, s, d = dims
    g = torch.Generator().manual_seed(d)
    x = torch.randn(b, s, d, generator=g).to(dtype)
    br = (0.5 * torch.randn(b, s, d, generator=g)).to(dtype)
    gamma, beta = torch.randn(d, generator=g), torch.randn(d, generator=g)   # fp32 master parameters
    d_total = (0.5 * torch.randn(b, s, d, generator=g)).to(dtype)
    d_y = torch.randn(b, s, d, generator=g).to(dtype)

    def leaves():
        return [t.to(dev).requires_grad_(True) for t in (x, br, gamma, beta)]

    xd, bd, gd, btd = leaves()
    total, y = T.add_layer_norm.apply(xd, bd, gd, btd, 1e-5)
    torch.autograd.backward([total, y], [d_total.to(dev), d_y.to(dev)])
    x2, b2, g2, bt2 = leaves()
    total2 = x2 + b2
    y2 = T.layer_norm.apply(total2, g2, bt2, 1e-5)
    torch.autograd.backward([total2, y2], [d_total.to(dev), d_y.to(dev)])
    assert torch.equal(total, total2) and torch.equal(y, y2)
    assert xd.grad is not None and torch.equal(xd.grad, bd.grad)
    # oracle: d(sum) = layernorm backward at the rounded sum + upstream gradient of the sum
    dx, dg, db = R.layer_norm_bwd(total2.detach().cpu(), gamma, d_y, 1e-5)
    want = dx.float() + d_total.float()
    atol = 2e-2 if dtype == torch.float16 else 1.5e-1
    assert_close(xd.grad, want, dtype, f"dx {dims}", atol=atol)
    assert_close(xd.grad, x2.grad, dtype, f"dx vs two nodes {dims}", atol=atol)
    lim = 1e-3 if dtype == torch.float16 else 8e-3
    assert rel_l2(gd.grad, dg) < lim and rel_l2(btd.grad, db) < lim
    assert torch.equal(gd.grad, g2.grad) and torch.equal(btd.grad, bt2.grad)


def test_add_layernorm_unused_outputs(dev):
    """Only one of the two outputs used downstream: the other's gradient arrives as None."""
    g = torch.Generator().manual_seed(3)
    x = torch.randn(2, 10, 256, generator=g).half().to(dev).requires_grad_(True)
    br = torch.randn(2, 10, 256, generator=g).half().to(dev).requires_grad_(True)
    gamma = torch.randn(256, generator=g).half().to(dev).requires_grad_(True)
    beta = torch.randn(256, generator=g).half().to(dev).requires_grad_(True)
    dy = torch.randn(2, 10, 256, generator=g).half().to(dev)
    _, y = T.add_layer_norm.apply(x, br, gamma, beta, 1e-5)
    y.backward(dy)
    x2 = (x.detach() + br.detach()).requires_grad_(True)
    g2, b2 = gamma.detach().clone().requires_grad_(True), beta.detach().clone().requires_grad_(True)
    T.layer_norm.apply(x2, g2, b2, 1e-5).backward(dy)
    assert torch.equal(x.grad, x2.grad) and torch.equal(br.grad, x2.grad) and torch.equal(gamma.grad, g2.grad)
    x.grad = br.grad = gamma.grad = beta.grad = None
    total, _ = T.add_layer_norm.apply(x, br, gamma, beta, 1e-5)
    total.backward(dy)
    assert torch.equal(x.grad, dy) and torch.equal(br.grad, dy) and gamma.grad is None
    with pytest.raises(ValueError):
        T.add_layer_norm.apply(x, br[:, :5], gamma, beta, 1e-5)


@pytest.mark.gpu
@pytest.mark.parametrize("pdtype", [torch.float32, torch.float16])
def test_param_grads_of_many_layernorms_in_one_launch(pdtype, dev):
    """Row passes that leave their partial sums in place, then ONE second stage for all of them
    (tf_layernorm_param_grads, 70 LayerNorms: a launch of 64 and one of 6) against the one-call
    form that the reference's structure has (kernels/layernorm.py:226-259): same dx, same bits in
    dgamma / dbeta; plain and residual-adding row passes, different row counts."""
    from tritonformer_amd import kernels as K

    g = torch.Generator().manual_seed(5)
    d = 256
    want, partials = [], []
    for i in range(70):
        rows = (3, 64 + 7 * i)
        x = torch.randn(*rows, d, generator=g).half().to(dev)
        dy = torch.randn(*rows, d, generator=g).half().to(dev)
        gamma = torch.randn(d, generator=g).to(pdtype).to(dev)
        mean = x.float().mean(-1).reshape(-1)
        rstd = (x.float().var(-1, unbiased=False) + 1e-5).rsqrt().reshape(-1)
        if i % 2:
            ds = torch.randn(*rows, d, generator=g).half().to(dev)
            dx, da, db = K.add_layernorm_bwd(dy, ds, x, gamma, mean, rstd)
            dx2, part = K.add_layernorm_bwd(dy, ds, x, gamma, mean, rstd, leave_partials=True)
        else:
            dx, da, db = K.layernorm_bwd(dy, x, gamma, mean, rstd)
            dx2, part = K.layernorm_bwd(dy, x, gamma, mean, rstd, leave_partials=True)
        assert torch.equal(dx, dx2)
        want.append((da, db))
        partials.append(part)
    out = K.layernorm_param_grads(partials, d, pdtype)
    assert out.shape == (70, 2, d) and out.dtype == pdtype
    for i, (da, db) in enumerate(want):
        assert torch.equal(out[i, 0], da) and torch.equal(out[i, 1], db), i
