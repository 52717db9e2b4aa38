"""GPU parity of the token + position embedding kernels against the fp32 oracle.  The
reference leaves this part of the model to nn.Embedding (transformer.py:259-272, 311-323),
so the expectations are the library's: forward exact (one fp32 addition, one rounding);
gradients are sums of fp32 terms in a fixed order, compared at 1e-6 relative (fp32
parameters) -- exact where no id repeats more than once -- and at fp16 resolution for
16-bit tables."""
import pytest
import torch

import tritonformer_amd as T
from oracle import ref_torch as R
from tritonformer_amd.transformer import Transformer, TransformerConfig
import tritonformer_amd.transformer as TM

pytestmark = pytest.mark.gpu

# (B, S, d, V, P, with_pos): repeats everywhere (tiny vocabulary), rows that are no multiple of
# a workgroup, widths that are no multiple of 8 (element path), long sequences (several LDS
# chunks in the chain scan), the headline shape
CASES = [(1, 1, 8, 4, 4, True), (2, 5, 3, 4, 7, True), (3, 64, 40, 11, 64, True), (2, 300, 256, 50, 512, False),
         (1, 4500, 64, 7, 4500, True), (2, 2500, 72, 3000, 2600, True), (4, 2048, 1024, 50304, 2048, True)]


def run_case(case, param_dtype, out_dtype, dev):
    b, s, d, v, p, with_pos = case
    g = torch.Generator().manual_seed(b * 131 + s)
    ids = torch.randint(0, v, (b, s), generator=g)
    tok = torch.randn(v, d, generator=g).to(param_dtype)
    pos = torch.randn(p, d, generator=g).to(param_dtype) if with_pos else None
    dy = torch.randn(b, s, d, generator=g).to(out_dtype)
    tok_d = tok.to(dev).requires_grad_(True)
    pos_d = pos.to(dev).requires_grad_(True) if with_pos else None
    out = T.embedding_sum.apply(ids.to(dev), tok_d, pos_d, out_dtype)
    out.backward(dy.to(dev))
    want = R.embedding(ids, tok, pos).to(out_dtype)
    assert out.dtype == out_dtype and torch.equal(out.cpu(), want), f"forward {case}"
    d_tok, d_pos = R.embedding_bwd(ids, dy, v, p if with_pos else None)
    tol = dict(rtol=1e-6, atol=1e-6) if param_dtype == torch.float32 else dict(rtol=2e-3, atol=2e-3)
    assert tok_d.grad.dtype == param_dtype
    assert torch.allclose(tok_d.grad.float().cpu(), d_tok, **tol), f"d_tok {case}"
    if with_pos:
        assert torch.allclose(pos_d.grad.float().cpu(), d_pos, **tol), f"d_pos {case}"
        assert torch.count_nonzero(pos_d.grad[s:]) == 0
    return ids, tok_d


@pytest.mark.parametrize("case", CASES)
def test_embedding_fp32_tables_fp16_stream(case, dev):
    run_case(case, torch.float32, torch.float16, dev)


@pytest.mark.parametrize("case", CASES[:6])
def test_embedding_other_dtypes(case, dev):
    run_case(case, torch.float32, torch.float32, dev)
    run_case(case, torch.float32, torch.bfloat16, dev)
    run_case(case, torch.float16, torch.float16, dev)


def test_embedding_gradient_is_reproducible_and_exact_without_repeats(dev):
    """Two runs give the same bits; with every id used once the gradient is a permutation of
    the rows of dy, bit for bit; rows of unused ids are zero."""
    b, s, d, v = 2, 512, 128, 4096
    ids = torch.randperm(v)[: b * s].view(b, s)
    tok = torch.randn(v, d).to(dev).requires_grad_(True)
    dy = torch.randn(b, s, d).to(dev)
    grads = []
    for _ in range(2):
        tok.grad = None
        T.embedding_sum.apply(ids.to(dev), tok, None, None).backward(dy)
        grads.append(tok.grad.clone())
    assert torch.equal(grads[0], grads[1])
    assert torch.equal(grads[0][ids.reshape(-1).to(dev)], dy.view(b * s, d))
    unused = torch.ones(v, dtype=torch.bool)
    unused[ids.reshape(-1)] = False
    assert torch.count_nonzero(grads[0][unused.to(dev)]) == 0
    rep = torch.randint(0, 5, (4, 1000))  # heavy repeats: still the same bits on every run
    small = torch.randn(5, 64).to(dev).requires_grad_(True)
    dy2 = torch.randn(4, 1000, 64).to(dev)
    runs = []
    for _ in range(2):
        small.grad = None
        T.embedding_sum.apply(rep.to(dev), small, None, None).backward(dy2)
        runs.append(small.grad.clone())
    assert torch.equal(runs[0], runs[1])


def test_model_with_and_without_fused_embedding(dev):
    """The model's loss and table gradients with the embedding kernels against the
    nn.Embedding composition they stand for (fp32 parameters under fp16 autocast)."""
    cfg = TransformerConfig(512, 128, 128, 2, 64, 256, 2, True, False)
    torch.manual_seed(0)
    model = Transformer(cfg, device=dev, param_dtype=torch.float32)
    model.logits_out.weight.data.normal_(0.0, 0.02)
    ids = torch.randint(0, cfg.vocab_size, (2, 128), device=dev)
    results = []
    for fused in (True, False):
        TM.FUSE_EMBED = fused
        try:
            model.zero_grad(set_to_none=True)
            with torch.autocast("cuda", dtype=torch.float16):
                _, loss = model(ids, ids)
            loss.backward()
            results.append((loss.item(), model.embed_tokens.weight.grad.clone(), model.embed_positions.weight.grad.clone()))
        finally:
            TM.FUSE_EMBED = True
    assert results[0][0] == results[1][0]  # same forward bits: fp32 add, one rounding to fp16
    for a, b_ in zip(results[0][1:], results[1][1:]):
        assert torch.allclose(a, b_, rtol=1e-5, atol=1e-7)
