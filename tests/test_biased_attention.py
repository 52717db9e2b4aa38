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


# ---- ALiBi in closed form: (nh,) float16 slopes in place of the dense matrix built from them
from tritonformer_amd.transformer import generate_alibi_mask, get_slopes  # noqa: E402


def _closed_form_vs_dense(dims, dtype, dev, packed_slopes=None):
    b, nh, s, hd = dims
    g = torch.Generator().manual_seed(s + hd)
    raw = [torch.randn(b, s, nh * hd, generator=g).to(dtype).to(dev) for _ in range(4)]
    slopes = torch.tensor(get_slopes(nh), dtype=torch.float16, device=dev)
    dense = generate_alibi_mask(s, nh, device=dev)[0].to(dtype)  # the fp16 matrix, cast as the model casts it
    outs = []
    for bias in (dense, slopes):
        q, k, v, do = (t.view(b, s, nh, hd).permute(0, 2, 1, 3) for t in raw)
        q, k, v = (t.detach().requires_grad_(True) for t in (q, k, v))
        o = T.fast_causal_attention_with_bias.apply(q, k, v, bias)
        o.backward(do)
        outs.append((o, q.grad, k.grad, v.grad))
    for name, a, c in zip(("o", "dq", "dk", "dv"), *outs):
        assert torch.equal(a, c), f"{name} differs between dense and closed-form ALiBi at {dims} {dtype}"
    return outs[1]


@pytest.mark.parametrize("dims", [(1, 2, 64, 64), (2, 4, 192, 32), (1, 3, 320, 128), (2, 8, 512, 64), (1, 24, 256, 64),
                                  (1, 12, 1024, 64)])
def test_alibi_closed_form_is_bit_identical_to_dense(dims, dev):
    """Forward, dQ, dK, dV from the slopes equal those from the dense matrix bit for bit: the
    kernels round distance, slope and product to fp16 exactly as the matrix holds them.
    Head counts that are powers of two and not (24, 12, 3: the interleaved slope rule)."""
    _closed_form_vs_dense(dims, torch.float16, dev)


def test_alibi_closed_form_bf16_and_long_distances(dev):
    """bf16 sees the fp16 matrix rounded to bf16; at 4096 keys the distances above 2048 are
    no longer exact in fp16 -- both reproduced (840M configuration: 24 heads x 64, ctx 4096,
    on four of its heads to bound the dense matrix)."""
    _closed_form_vs_dense((1, 4, 256, 64), torch.bfloat16, dev)
    b, nh, s, hd = 1, 4, 4096, 64
    g = torch.Generator().manual_seed(7)
    raw = [torch.randn(b, s, nh * hd, generator=g).half().to(dev) for _ in range(4)]
    slopes = torch.tensor(get_slopes(24), dtype=torch.float16, device=dev)[20:24].contiguous()
    dense = generate_alibi_mask(s, 24, device=dev)[0][20:24].contiguous()
    outs = []
    for bias in (dense, slopes):
        q, k, v, do = (t.view(b, s, nh, hd).permute(0, 2, 1, 3) for t in raw)
        q, k, v = (t.detach().requires_grad_(True) for t in (q, k, v))
        o = T.fast_causal_attention_with_bias.apply(q, k, v, bias)
        o.backward(do)
        outs.append((o, q.grad, k.grad, v.grad))
    for a, c in zip(*outs):
        assert torch.equal(a, c)


def test_alibi_closed_form_against_oracle_and_argument_checks(dev):
    run_case((2, 4, 256, 64), torch.float16, dev, bias=R.alibi_mask(256, 4),
             kernel_bias=torch.tensor(get_slopes(4), dtype=torch.float16))
    q, k, v, _ = make_qkv((1, 4, 128, 64), torch.float16, dev)
    with pytest.raises(ValueError):   # one slope per head
        T.fast_causal_attention_with_bias.apply(q.to(dev), k.to(dev), v.to(dev), torch.ones(3, dtype=torch.float16, device=dev))
    with pytest.raises(ValueError):   # float16 slopes, the precision the reference's matrix is built from
        T.fast_causal_attention_with_bias.apply(q.to(dev), k.to(dev), v.to(dev), torch.ones(4, dtype=torch.float32, device=dev))
