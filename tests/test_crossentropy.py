"""GPU parity of the cross-entropy Function against the fp32 oracle.  The
contract is the one the model uses (reference transformer.py:336-343): a loss
per row, mean taken by the caller; reference test shapes N in [1,32), V in
[256,64000) (tritonformer/test_crossentropy.py).  Tolerance: loss atol 1e-2 as
the reference's test; gradient atol 1e-3 on probabilities in [0,1]."""
import math

import numpy as np
import pytest
import torch

import tritonformer_amd as T
from oracle import ref_torch as R
from tests.util import NUM_TEST, assert_close, rel_l2

pytestmark = pytest.mark.gpu
rng = np.random.RandomState(0)
DIMS = [(int(n), int(v)) for n in rng.randint(1, 32, size=NUM_TEST) for v in rng.randint(256, 64000, size=NUM_TEST)]
EDGE = [(1, 8), (3, 7), (5, 50304), (64, 50304), (2, 131072)]


@pytest.mark.parametrize("dims", DIMS + EDGE)
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_cross_entropy_fwd_bwd(dims, dtype, dev):
    n, v = dims
    g = torch.Generator().manual_seed(n + v)
    x = torch.randn(n, v, generator=g).to(dtype)
    lab = torch.randint(0, v, (n,), generator=g)
    gout = torch.randn(n, generator=g).to(dtype)
    xd = x.to(dev).requires_grad_(True)
    loss = T.cross_entropy_loss.apply(xd, lab.to(dev))
    assert loss.shape == (n,) and loss.dtype == dtype
    loss.backward(gout.to(dev))
    assert_close(loss, R.cross_entropy(x, lab), dtype, f"loss {dims}", atol=1e-2 if dtype == torch.float16 else 6e-2)
    assert_close(xd.grad, R.cross_entropy_bwd(x, lab, gout), dtype, f"grad {dims}", atol=1e-3, rtol=1e-2)


def test_uniform_logits_and_mean_reduction(dev):
    n, v = 16, 50304
    x = torch.zeros(n, v, dtype=torch.float16, device=dev, requires_grad=True)
    lab = torch.randint(0, v, (n,), device=dev)
    loss = T.cross_entropy_loss.apply(x, lab)
    assert (loss.float() - math.log(v)).abs().max() < 5e-3          # ln(50304) = 10.8258
    loss.float().mean().backward()                                   # the caller's reduction
    grad = x.grad.float()
    assert (grad.sum(-1)).abs().max() < 1e-3                         # softmax - onehot sums to zero
    assert torch.equal(grad.argmin(-1), lab)


def test_row_stride_and_labels_edge(dev):
    """Logits that are a column slice of a wider buffer (row stride > V) and labels at both ends."""
    g = torch.Generator().manual_seed(3)
    wide = torch.randn(9, 1000, generator=g).half()
    x = wide[:, :904]
    lab = torch.tensor([0, 903, 5, 17, 903, 0, 450, 1, 902])
    loss = T.cross_entropy_loss.apply(x.to(dev), lab.to(dev))
    assert_close(loss, R.cross_entropy(x, lab), name="strided rows")


def test_headline_rows(dev):
    """Rows of the 410M configuration (V = 50304) with unit-variance logits; fp32 oracle on the CPU."""
    n, v = 2047, 50304
    g = torch.Generator().manual_seed(0)
    x = torch.randn(n, v, generator=g).half().to(dev).requires_grad_(True)
    lab = torch.randint(0, v, (n,), generator=g).to(dev)
    loss = T.cross_entropy_loss.apply(x, lab)
    loss.float().sum().backward()
    ref = R.cross_entropy(x.detach().cpu(), lab.cpu())
    assert_close(loss, ref, name="loss")
    assert abs(loss.float().mean().item() - ref.mean().item()) <= 1e-3 * ref.mean().item()
    assert rel_l2(x.grad, R.cross_entropy_bwd(x.detach().cpu(), lab.cpu(), torch.ones(n))) < 2e-3


def test_argument_checks(dev):
    with pytest.raises(TypeError):
        T.cross_entropy_loss.apply(torch.zeros(4, 8, device=dev, dtype=torch.float16), torch.zeros(4, device=dev, dtype=torch.int32))
    with pytest.raises(ValueError):
        T.cross_entropy_loss.apply(torch.zeros(4, 8, device=dev, dtype=torch.float16), torch.zeros(5, device=dev, dtype=torch.int64))


@pytest.mark.parametrize("dims", [(2, 5, 904), (3, 64, 1000), (4, 256, 50304)])
def test_shifted_cross_entropy_equals_copy_then_cross_entropy(dims, dev):
    """The in-place shifted variant must give exactly what the reference's
    shift-copy followed by the plain Function gives (transformer.py:333-341)."""
    b, s, v = dims
    g = torch.Generator().manual_seed(7)
    x = torch.randn(b, s, v, generator=g).half().to(dev)
    lab = torch.randint(0, v, (b, s), generator=g).to(dev)
    xa = x.clone().requires_grad_(True)
    xb = x.clone().requires_grad_(True)
    fused = T.shifted_cross_entropy_loss.apply(xa, lab)
    plain = T.cross_entropy_loss.apply(xb[:, :-1].contiguous().view(-1, v), lab[:, 1:].contiguous().view(-1))
    assert fused.shape == (b * (s - 1),) and torch.equal(fused, plain)
    gout = torch.randn(b * (s - 1), generator=g).half().to(dev)
    fused.backward(gout)
    plain.backward(gout)
    assert torch.equal(xa.grad, xb.grad)
    assert (xa.grad[:, -1] == 0).all()
    ref = R.cross_entropy(x[:, :-1].reshape(-1, v).cpu(), lab[:, 1:].reshape(-1).cpu())
    assert_close(fused, ref, name="shifted loss")


@pytest.mark.parametrize("dims,dtype,scale", [((2, 5, 904), torch.float16, 1024.0), ((3, 64, 50304), torch.float16, 1024.0),
                                              ((2, 9, 1000), torch.bfloat16, 1.0), ((1, 3, 60000), torch.float16, 1024.0),
                                              ((2, 7, 333), torch.float16, 1024.0)])
def test_forward_that_also_writes_the_gradient(dims, dtype, scale, dev):
    """tf_cross_entropy_fwd_grad: loss and log-sum-exp of the plain forward, and (softmax - onehot) *
    scale equal, bit for bit, to the backward kernel run with every upstream gradient = scale --
    whether one kernel does both (rows that fit the registers), or the pair runs (60000 columns;
    333 columns: no 16-byte chunks)."""
    from tritonformer_amd import kernels as K

    b, s, v = dims
    g = torch.Generator().manual_seed(5)
    x = (torch.randn(b, s, v, generator=g) * 2).to(dtype).to(dev)
    lab = torch.randint(0, v, (b, s), generator=g).to(dev)
    loss, lse, dl = K.shifted_cross_entropy_fwd_grad(x, lab, scale)
    loss0, lse0, _, shift = K.shifted_cross_entropy_fwd(x, lab)
    assert torch.equal(loss, loss0) and torch.equal(lse, lse0)
    gout = torch.full((b * (s - 1),), scale, dtype=dtype, device=dev)
    assert torch.equal(dl, K.shifted_cross_entropy_bwd(gout, x, shift, lse0))
    assert (dl[:, -1] == 0).all()
    ref = R.cross_entropy_bwd(x[:, :-1].reshape(-1, v).float().cpu(), lab[:, 1:].reshape(-1).cpu(),
                              torch.full((b * (s - 1),), scale))
    assert rel_l2(dl[:, :-1].reshape(-1, v), ref) < (2e-3 if dtype == torch.float16 else 1e-2)


@pytest.mark.parametrize("master", [True, False])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_lm_head_loss_node(master, dtype, dev):
    """lm_head_loss = linear_no_bias + shifted_cross_entropy_loss + mean as one node: logits and loss
    equal those of the three calls bit for bit; the gradients are compared with the fp32 oracle --
    with an UNSCALED loss, where the separate calls lose the logits gradient to fp16 underflow
    ((softmax - onehot) / N with N = 2046 rows) and the fused node does not."""
    b, s, d, v = 2, 1024, 256, 50304
    g = torch.Generator().manual_seed(19)
    h = torch.randn(b, s, d, generator=g)
    w = torch.randn(d, v, generator=g) * 0.05
    lab = torch.randint(0, v, (b, s), generator=g)
    if not master:
        h, w = h.to(dtype), w.to(dtype)

    hr, wr = h.float().clone().requires_grad_(True), w.float().clone().requires_grad_(True)
    hq = hr.to(dtype).float() if master else hr          # what the kernels see after autocast's cast
    wq = wr.to(dtype).float() if master else wr
    logits_ref = hq @ wq
    loss_ref = R.cross_entropy(logits_ref[:, :-1].reshape(-1, v), lab[:, 1:].reshape(-1)).mean()
    loss_ref.backward()

    def run(fused):
        hd, wd = h.to(dev).requires_grad_(True), w.to(dev).requires_grad_(True)
        with torch.autocast("cuda", dtype=dtype, enabled=master):
            if fused:
                logits, loss = T.lm_head_loss.apply(hd, wd, lab.to(dev))
            else:
                logits = T.linear_no_bias.apply(hd, wd)
                loss = T.shifted_cross_entropy_loss.apply(logits, lab.to(dev)).mean()
        loss.backward()
        return logits, loss, hd.grad, wd.grad

    lf, lossf, dhf, dwf = run(True)
    ls, losss, dhs, dws = run(False)
    assert torch.equal(lf, ls) and torch.equal(lossf, losss)
    assert abs(lossf.item() - loss_ref.item()) <= (1e-3 if dtype == torch.float16 else 4e-3) * loss_ref.item()
    assert dwf.dtype == (torch.float32 if master else dtype) and dwf.shape == (d, v) and dhf.shape == (b, s, d)
    tol_w = 3e-3 if dtype == torch.float16 else 1.5e-2
    assert rel_l2(dwf, wr.grad) < tol_w, rel_l2(dwf, wr.grad)
    if master:    # fp32 gradient of the fp32 hidden state (autograd casts the 16-bit result up)
        assert rel_l2(dhf, hr.grad) < (2e-2 if dtype == torch.float16 else 3e-2), rel_l2(dhf, hr.grad)
    if dtype == torch.float16:
        # the separate calls, unscaled: most of the gradient is gone
        assert rel_l2(dws, wr.grad) > 10 * rel_l2(dwf, wr.grad)


def test_lm_head_loss_when_the_logits_are_used_too(dev):
    """A gradient arriving through the returned logits is added to the loss gradient."""
    b, s, d, v = 2, 33, 64, 1000
    g = torch.Generator().manual_seed(23)
    h = torch.randn(b, s, d, generator=g).half()
    w = (torch.randn(d, v, generator=g) * 0.1).half()
    lab = torch.randint(0, v, (b, s), generator=g)
    extra = torch.randn(b, s, v, generator=g).half() * 1e-2
    hd, wd = h.to(dev).requires_grad_(True), w.to(dev).requires_grad_(True)
    logits, loss = T.lm_head_loss.apply(hd, wd, lab.to(dev))
    (loss.float() * 64 + (logits.float() * extra.to(dev).float()).sum()).backward()
    hr, wr = h.float().requires_grad_(True), w.float().requires_grad_(True)
    lr = hr @ wr
    (R.cross_entropy(lr[:, :-1].reshape(-1, v), lab[:, 1:].reshape(-1)).mean() * 64 + (lr * extra.float()).sum()).backward()
    assert rel_l2(wd.grad, wr.grad) < 5e-3 and rel_l2(hd.grad, hr.grad) < 5e-3
    # no gradient needed: no gradient buffer is written, same outputs
    with torch.no_grad():
        l2, loss2 = T.lm_head_loss.apply(h.to(dev), w.to(dev), lab.to(dev))
    assert torch.equal(l2, logits) and torch.equal(loss2, loss)
