"""GPU parity of the fused AdamW step against the fp32 oracle (itself pinned against
torch.optim.AdamW on the CPU in tests/test_oracle.py).  The reference ships no optimizer;
the expectations are the library's.  Tolerance: the update is a handful of fp32 operations
per element, compared at 2e-6 relative after six steps; the 16-bit copies must be the
rounded parameters exactly."""
import pytest
import torch

from oracle import ref_torch as R
from tritonformer_amd.optim import AdamW

pytestmark = pytest.mark.gpu

SHAPES = [(1,), (7,), (1024,), (3, 5), (333, 77), (1024, 4096), (50304, 64)]   # unaligned tails, several launches' worth


@pytest.mark.parametrize("shadow_dtype", [None, torch.float16, torch.bfloat16])
def test_adamw_steps_match_oracle(shadow_dtype, dev):
    hyper = dict(lr=3e-3, betas=(0.9, 0.95), eps=1e-8, weight_decay=0.1)
    g = torch.Generator().manual_seed(0)
    cpu = [torch.randn(s, generator=g) for s in SHAPES] + [torch.randn(64, generator=g) for _ in range(30)]
    params = [t.clone().to(dev).requires_grad_(True) for t in cpu]
    opt = AdamW(params, shadow_dtype=shadow_dtype, **hyper)
    ms, vs = [torch.zeros_like(t) for t in cpu], [torch.zeros_like(t) for t in cpu]
    for step in range(1, 7):
        grads = [torch.randn(t.shape, generator=g) * (0.05 * step) for t in cpu]
        for p, gr in zip(params, grads):
            p.grad = gr.to(dev)
        opt.step()
        for i, gr in enumerate(grads):
            cpu[i], ms[i], vs[i] = R.adamw_step(cpu[i], gr, ms[i], vs[i], step, **hyper)
    for p, want, m, v in zip(params, cpu, ms, vs):
        assert torch.allclose(p.detach().cpu(), want, rtol=2e-6, atol=1e-7)
        st = opt.state[p]
        assert st["step"] == 6
        assert torch.allclose(st["exp_avg"].cpu(), m, rtol=2e-6, atol=1e-7)   # sums that cancel: absolute, one ulp of the terms
        assert torch.allclose(st["exp_avg_sq"].cpu(), v, rtol=2e-6, atol=1e-9)
        if shadow_dtype is None:
            assert opt.shadow(p) is None
        else:
            assert torch.equal(opt.shadow(p), p.detach().to(shadow_dtype))


def test_adamw_skips_parameters_without_gradient_and_checks_dtypes(dev):
    a = torch.randn(100, device=dev, requires_grad=True)
    b = torch.randn(100, device=dev, requires_grad=True)
    before = b.detach().clone()
    opt = AdamW([a, b], lr=1e-2)
    a.grad = torch.randn(100, device=dev)
    opt.step()
    assert torch.equal(b.detach(), before) and not opt.state[b]
    h = torch.randn(8, device=dev, dtype=torch.float16, requires_grad=True)
    h.grad = torch.randn(8, device=dev, dtype=torch.float16)
    with pytest.raises(TypeError):
        AdamW([h]).step()
    with pytest.raises(ValueError):
        AdamW([a], lr=-1.0)


def test_training_steps_reduce_the_loss(dev):
    """Forward + backward through the HIP kernels and this optimizer: a tiny model overfits
    one batch (loss falls from ln(vocab) by more than half within 30 steps)."""
    from tritonformer_amd.transformer import Transformer, TransformerConfig

    cfg = TransformerConfig(512, 128, 128, 2, 64, 256, 2, True, False)
    torch.manual_seed(0)
    model = Transformer(cfg, device=dev, param_dtype=torch.float32)
    opt = AdamW(model.parameters(), lr=3e-3, weight_decay=0.0)
    ids = torch.randint(0, cfg.vocab_size, (2, 128), device=dev)
    losses = []
    for _ in range(30):
        opt.zero_grad(set_to_none=True)
        with torch.autocast("cuda", dtype=torch.float16):
            _, loss = model(ids, ids)
        loss.backward()
        opt.step()
        losses.append(loss.item())
    assert abs(losses[0] - 6.2383) < 2e-2          # zero-initialised LM head: ln(512)
    assert losses[-1] < 0.5 * losses[0]
