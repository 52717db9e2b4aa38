"""GPU parity of causal attention with an additive bias against the fp32 oracle;
mirrors the reference's tritonformer/test_biased_attention.py (ALiBi bias from the
model's mask builder, passed as (nh, S', S') with -inf above the diagonal)."""
import numpy as np
import pytest
import torch

import tritonformer_amd as T
from oracle import ref_torch as R
from tests.test_attention import make_qkv, run_case
from tests.util import NUM_TEST, assert_close

pytestmark = pytest.mark.gpu
rng = np.random.RandomState(1)

DIMS = [(int(b), int(nh), int(sq), int(hd))
        for b in rng.randint(1, 4, size=NUM_TEST)
        for nh in rng.randint(4, 12, size=1)
        for sq in 64 * rng.randint(1, 10, size=NUM_TEST)
        for hd in rng.choice([32, 64], size=1)]


@pytest.mark.parametrize("dims", DIMS + [(1, 2, 64, 64), (1, 3, 192, 128), (2, 24, 256, 64)])
def test_biased_attn_fwd_bwd(dims, dev):
    b, nh, s, hd = dims
    run_case(dims, torch.float16, dev, bias=R.alibi_mask(s, nh))


def test_bias_larger_than_sequence(dev):
    """The model passes the full max_position_embeddings mask for any seq_len
    (reference transformer.py:297-302, 326): only the top-left S x S block is read."""
    run_case((2, 4, 128, 64), torch.float16, dev, bias=R.alibi_mask(320, 4))


def test_zero_bias_equals_unbiased(dev):
    q, k, v, _ = make_qkv((1, 4, 256, 64), torch.float16, dev)
    qd, kd, vd = q.to(dev), k.to(dev), v.to(dev)
    zero = torch.zeros(4, 256, 256, dtype=torch.float16, device=dev)
    a = T.fast_causal_attention_with_bias.apply(qd, kd, vd, zero)
    b = T.fast_causal_attention.apply(qd, kd, vd)
    assert (a.float() - b.float()).abs().max() < 1e-3


def test_random_dense_bias_and_no_bias_gradient(dev):
    g = torch.Generator().manual_seed(4)
    bias = torch.randn(3, 128, 128, generator=g).half()
    run_case((2, 3, 128, 64), torch.float16, dev, bias=bias)
    q, k, v, do = make_qkv((1, 3, 128, 64), torch.float16, dev)
    bd = bias.to(dev).requires_grad_(True)
    o = T.fast_causal_attention_with_bias.apply(q.to(dev).requires_grad_(True), k.to(dev), v.to(dev), bd)
    o.backward(do.to(dev))
    assert bd.grad is None   # reference attention.py:60 returns None for the bias


def test_bf16_bias(dev):
    run_case((1, 4, 128, 64), torch.bfloat16, dev, bias=R.alibi_mask(128, 4, dtype=torch.bfloat16))


def test_long_context_alibi_shape(dev):
    """840M ALiBi configuration (24 heads x 64, ctx 4096) on a reduced head count."""
    b, nh, s, hd = 1, 4, 4096, 64
    bias = R.alibi_mask(s, 24)[:nh].contiguous().to(dev)
    g = torch.Generator().manual_seed(0)
    raw = [torch.randn(b, s, nh * hd, generator=g).half().to(dev) for _ in range(4)]
    q, k, v, do = (t.view(b, s, nh, hd).permute(0, 2, 1, 3) for t in raw)
    q, k, v = (t.requires_grad_(True) for t in (q, k, v))
    o = T.fast_causal_attention_with_bias.apply(q, k, v, bias)
    o.backward(do)
    qr, kr, vr = (t.detach().float().requires_grad_(True) for t in (q, k, v))
    orf = R.causal_attention(qr, kr, vr, bias)
    orf.backward(do.float())
    assert_close(o, orf, name="o")
    assert_close(q.grad, qr.grad, name="dq")
    assert_close(k.grad, kr.grad, name="dk")
    assert_close(v.grad, vr.grad, name="dv")
