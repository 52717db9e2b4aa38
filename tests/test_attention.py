"""GPU parity of causal flash attention (forward, dQ, dK, dV) against the fp32
oracle; mirrors the reference's tritonformer/test_attention.py (q, k, v, dy ~
N(0,1) fp16; B in [1,4), nh in [4,32), S = 64*[1,32), hd in {32,64}) and adds
hd = 128, bf16, the strided (B,S,nh,hd)->(B,nh,S,hd) views the model feeds, and
the baseline configurations' shapes.

Tolerance: max-abs <= 1e-2 (+1e-3 relative), as test_attention.py:88 (atol=1e-2),
against fp32 math instead of the reference's fp16-rounded P.
"""
import math

import numpy as np
import pytest
import torch

import tritonformer_amd as T
from oracle import ref_torch as R
from tests.util import NUM_TEST, assert_close, rel_l2

pytestmark = pytest.mark.gpu
rng = np.random.RandomState(0)

DIMS = [(int(b), int(nh), int(sq), int(hd))
        for b in rng.randint(1, 4, size=NUM_TEST)
        for nh in rng.randint(4, 12, size=1)
        for sq in 64 * rng.randint(1, 12, size=NUM_TEST)
        for hd in rng.choice([32, 64], size=1)]
EDGE = [(1, 1, 64, 64), (1, 2, 64, 32), (2, 3, 128, 64), (1, 2, 192, 128), (1, 4, 320, 128), (2, 2, 1024, 64)]
# the upper ends of the reference's draws (test_attention.py:66-73: nh < 32, S = 64 * [1, 32), B < 4)
UPPER = [(1, 31, 1984, 64), (3, 5, 1984, 32)]
# head_dim 128 with S = 32 (mod 64): lengths the reference's 32-row blocks admit (kernels/attention.py:177-183)
HD128_S32 = [(1, 2, 32, 128), (2, 3, 96, 128), (1, 2, 160, 128)]


def make_qkv(dims, dtype, dev, seed=0, strided=True):
    b, nh, s, hd = dims
    g = torch.Generator().manual_seed(seed)
    if strided:  # views of (B, S, nh*hd) buffers, strides (S*d, hd, d, 1), as transformer.py:158-175
        raw = [torch.randn(b, s, nh * hd, generator=g).to(dtype) for _ in range(4)]
        q, k, v, do = (t.view(b, s, nh, hd).permute(0, 2, 1, 3) for t in raw)
    else:
        q, k, v, do = (torch.randn(b, nh, s, hd, generator=g).to(dtype) for _ in range(4))
    return q, k, v, do


def run_case(dims, dtype, dev, bias=None, strided=True, seed=0, kernel_bias=None):
    """``bias``: what the oracle adds; ``kernel_bias``: what the kernels are given for it when that
    differs (the ALiBi slopes instead of the dense matrix)."""
    q, k, v, do = make_qkv(dims, dtype, dev, seed, strided)
    qd, kd, vd = (t.to(dev).requires_grad_(True) for t in (q, k, v))  # .to keeps the strides
    if bias is None:
        o = T.fast_causal_attention.apply(qd, kd, vd)
    else:
        o = T.fast_causal_attention_with_bias.apply(qd, kd, vd, (bias if kernel_bias is None else kernel_bias).to(dev))
    assert o.stride() == qd.stride() and o.dtype == dtype
    o.backward(do.to(dev))
    qr, kr, vr = (t.float().requires_grad_(True) for t in (q, k, v))
    o_ref = R.causal_attention(qr, kr, vr, bias)
    o_ref.backward(do.float())
    tag = f"{dims} {dtype}"
    assert_close(o, o_ref, dtype, "o " + tag)
    assert_close(qd.grad, qr.grad, dtype, "dq " + tag)
    assert_close(kd.grad, kr.grad, dtype, "dk " + tag)
    assert_close(vd.grad, vr.grad, dtype, "dv " + tag)
    return o, qd, kd, vd


@pytest.mark.parametrize("dims", DIMS + EDGE + UPPER)
def test_attn_fwd_bwd(dims, dev):
    run_case(dims, torch.float16, dev)


@pytest.mark.parametrize("dims", HD128_S32)
@pytest.mark.parametrize("strided", [True, False])
def test_attn_head_dim_128_takes_multiples_of_32(dims, strided, dev):
    run_case(dims, torch.float16, dev, strided=strided)
    run_case(dims, torch.bfloat16, dev, strided=strided, seed=1)
    with pytest.raises(ValueError):     # 64-wide heads keep the reference's multiple-of-64 rule
        q = torch.zeros(1, 2, dims[2], 64, dtype=torch.float16, device=dev)
        T.fast_causal_attention.apply(q, q, q)


@pytest.mark.parametrize("dims", [(1, 2, 128, 64), (2, 3, 256, 32), (1, 2, 192, 128)])
def test_attn_bf16(dims, dev):
    run_case(dims, torch.bfloat16, dev)


def test_attn_contiguous_layout(dev):
    run_case((2, 4, 256, 64), torch.float16, dev, strided=False)


def test_attn_mismatched_strides_are_normalised(dev):
    """The reference silently uses q's strides for k, v and o (kernels/attention.py:202-205)."""
    q, k, v, do = make_qkv((1, 2, 128, 64), torch.float16, dev, strided=True)
    kc = k.contiguous()
    o = T.fast_causal_attention.apply(q.to(dev), kc.to(dev), v.to(dev))
    assert_close(o, R.causal_attention(q, k, v), name="mixed layouts")


def test_attn_invariants(dev):
    o, q, k, v = run_case((2, 4, 512, 64), torch.float16, dev, seed=7)
    assert torch.equal(o[:, :, 0], v.detach()[:, :, 0])        # query 0 attends to key 0 only
    # a constant V makes every output row that constant, and dQ = dK = 0
    vc = torch.ones_like(v.detach()) * 0.5
    qd, kd = q.detach().clone().requires_grad_(True), k.detach().clone().requires_grad_(True)
    oc = T.fast_causal_attention.apply(qd, kd, vc)
    assert (oc.float() - 0.5).abs().max() < 2e-3
    oc.backward(torch.randn_like(oc))
    assert qd.grad.abs().max() < 2e-3 and kd.grad.abs().max() < 2e-3
    # bitwise reproducible
    assert torch.equal(T.fast_causal_attention.apply(q, k, v), o)


def test_attn_large_magnitude_scores(dev):
    """Scores far from zero exercise the thresholded running-max update."""
    q, k, v, do = make_qkv((1, 2, 256, 64), torch.float16, dev, seed=3)
    q = q * 6.0
    o = T.fast_causal_attention.apply(q.to(dev), k.to(dev), v.to(dev))
    assert_close(o, R.causal_attention(q, k, v), name="peaked softmax")


@pytest.mark.parametrize("dims", [(4, 16, 2048, 64), (2, 16, 2048, 128)])
def test_baseline_config_shapes(dims, dev):
    """410M (hd 64) and 1.4B (hd 128) attention shapes at full size, one batch element at a time
    (keeps the S x S fp32 score matrices small): the first against the fp32 oracle on the CPU, the
    others against the same oracle expressions evaluated in fp32 on the GPU."""
    b, nh, s, hd = dims
    g = torch.Generator().manual_seed(0)
    raw = [torch.randn(b, s, nh * hd, generator=g).half().to(dev) for _ in range(4)]
    q, k, v, do = (t.view(b, s, nh, hd).permute(0, 2, 1, 3) for t in raw)
    q, k, v = (t.requires_grad_(True) for t in (q, k, v))
    o = T.fast_causal_attention.apply(q, k, v)
    o.backward(do)
    grads = [t.grad.clone() for t in (q, k, v)]
    for t in (q, k, v):
        t.grad = None
    worst = 0.0
    for bi in range(b):
        where = "cpu" if bi == 0 else dev
        qr, kr, vr = (t[bi:bi + 1].detach().float().to(where).requires_grad_(True) for t in (q, k, v))
        orf = R.causal_attention(qr, kr, vr)
        orf.backward(do[bi:bi + 1].float().to(where))
        assert_close(o[bi:bi + 1], orf, name="o")
        for got, ref, nm in zip(grads, (qr, kr, vr), "qkv"):
            assert_close(got[bi:bi + 1], ref.grad, name="d" + nm)


@pytest.mark.parametrize("use_bias", [False, True])
def test_packed_qkv_equals_three_slices(use_bias, dev):
    """The packed Function runs the same kernels on strided slices of one buffer:
    results must equal the three-tensor Function bit for bit, gradient included."""
    b, s, nh, hd = 2, 256, 4, 64
    g = torch.Generator().manual_seed(11)
    qkv = torch.randn(b, s, 3, nh, hd, generator=g).half().to(dev)
    do = torch.randn(b, s, nh * hd, generator=g).half().to(dev)
    bias = R.alibi_mask(s, nh).to(dev) if use_bias else None
    a = qkv.clone().requires_grad_(True)
    out_p = T.fast_causal_attention_qkvpacked.apply(a, bias)
    out_p.backward(do)
    parts = [qkv[:, :, i].permute(0, 2, 1, 3).contiguous().requires_grad_(True) for i in range(3)]
    if use_bias:
        out_s = T.fast_causal_attention_with_bias.apply(*parts, bias)
    else:
        out_s = T.fast_causal_attention.apply(*parts)
    out_s.backward(do.view(b, s, nh, hd).permute(0, 2, 1, 3))
    assert out_p.shape == (b, s, nh * hd)
    assert torch.equal(out_p.view(b, s, nh, hd).permute(0, 2, 1, 3), out_s)
    for i in range(3):
        assert torch.equal(a.grad[:, :, i].permute(0, 2, 1, 3), parts[i].grad)
    o_ref = R.causal_attention(*[p_.detach().cpu() for p_ in parts], bias.cpu() if use_bias else None)
    assert_close(out_s, o_ref, name="packed vs oracle")


@pytest.mark.parametrize("use_bias", [False, True])
def test_attention_block_equals_separate_functions(use_bias, dev):
    """attention_block (projections + attention + output projection as one node) against
    linear_no_bias_packed -> fast_causal_attention_qkvpacked -> linear_no_bias: the forward is
    the same kernels in the same order (bitwise equal); gradients agree up to the fp32
    summation order of the weight-gradient contraction (relative L2 < 1e-3 in fp16)."""
    from tritonformer_amd.transformer import generate_alibi_mask

    b, s, nh, hd = 2, 256, 4, 64
    d = nh * hd
    g = torch.Generator().manual_seed(21)
    x = torch.randn(b, s, d, generator=g).half()
    ws = [(torch.randn(d, d, generator=g) / d ** 0.5).half() for _ in range(4)]
    dy = torch.randn(b, s, d, generator=g).half().to(dev)
    bias = generate_alibi_mask(s, nh, device=dev)[0] if use_bias else None

    def run(block):
        xd = x.to(dev).requires_grad_(True)
        wd = [w.to(dev).requires_grad_(True) for w in ws]
        if block:
            y = T.attention_block.apply(xd, *wd, nh, bias)
        else:
            qkv = T.linear_no_bias_packed.apply(xd, *wd[:3]).view(b, s, 3, nh, hd)
            y = T.linear_no_bias.apply(T.fast_causal_attention_qkvpacked.apply(qkv, bias), wd[3])
        y.backward(dy)
        return y, xd.grad, [w.grad for w in wd]

    y1, dx1, dw1 = run(True)
    y0, dx0, dw0 = run(False)
    assert torch.equal(y1, y0) and torch.equal(dx1, dx0)
    for a, c in zip(dw1, dw0):
        assert a.shape == (d, d) and a.is_contiguous() and rel_l2(a, c) < 1e-3


@pytest.mark.parametrize("dims", [(2, 3, 96, 64), (1, 2, 160, 32), (1, 4, 32, 64), (2, 2, 224, 128), (1, 2, 1056, 64)])
@pytest.mark.parametrize("bias_kind", ["none", "dense", "alibi"])
def test_half_used_last_block_through_the_c_abi(dims, bias_kind, dev):
    """S = 32 (mod 64) at every head_dim: the kernels walk 64-row blocks and use half of the last one.  The
    operator keeps the reference's rule (multiples of 64 below head_dim 128), so these go through the C
    ABI directly.  q, k, v, o, dO, lse and the dense bias lie in buffers whose every element beyond the
    sequence is NaN: a row of the unused half that took part in anything would show in the results."""
    import math
    from tritonformer_amd import _lib
    from tritonformer_amd.transformer import get_slopes

    lib = _lib.load()
    b, nh, s, hd = dims
    g = torch.Generator().manual_seed(5)
    nan = float("nan")

    def poisoned(*shape):
        """(B, S, nh, hd)-shaped random data at the front of a NaN buffer with 64 spare rows behind every sequence"""
        buf = torch.full((b, s + 64, nh, hd), nan, dtype=torch.float16)
        buf[:, :s] = torch.randn(b, s, nh, hd, generator=g).half()
        return buf.to(dev)

    qb, kb, vb, dob = poisoned(), poisoned(), poisoned(), poisoned()
    ob, dqb, dkb, dvb = (torch.full((b, s + 64, nh, hd), nan, dtype=torch.float16, device=dev) for _ in range(4))
    lse = torch.full((b * nh * s + 64,), nan, dtype=torch.float32, device=dev)
    delta = torch.full((b * nh * s + 64,), nan, dtype=torch.float32, device=dev)
    sb, sh, ss = (s + 64) * nh * hd, hd, nh * hd
    bias_t = slopes = None
    bias_ref = None
    if bias_kind == "dense":
        sp = s  # exactly the sequence: nothing to spare behind the last row or column
        bias_full = torch.full((nh, sp + 8, sp + 8), nan, dtype=torch.float16)
        bias_ref = (torch.randn(nh, sp, sp, generator=g) * 0.5).half()
        bias_full[:, :sp, :sp] = bias_ref
        bias_t = bias_full.to(dev)
    elif bias_kind == "alibi":
        slopes = torch.tensor(get_slopes(nh), dtype=torch.float16, device=dev)
        bias_ref = R.alibi_mask(s, nh)
    stream = torch.cuda.current_stream().cuda_stream
    scale = 1.0 / math.sqrt(hd)
    if slopes is not None:
        _lib.check(lib.tf_attn_alibi_fwd(stream, 0, b, nh, s, hd, qb.data_ptr(), kb.data_ptr(), vb.data_ptr(), ob.data_ptr(),
                                         sb, sh, ss, sb, sh, ss, lse.data_ptr(), slopes.data_ptr(), scale))
        _lib.check(lib.tf_attn_alibi_bwd(stream, 0, b, nh, s, hd, qb.data_ptr(), kb.data_ptr(), vb.data_ptr(), ob.data_ptr(),
                                         dob.data_ptr(), dqb.data_ptr(), dkb.data_ptr(), dvb.data_ptr(), sb, sh, ss, sb, sh, ss,
                                         lse.data_ptr(), delta.data_ptr(), slopes.data_ptr(), scale))
    else:
        bargs = (bias_t.data_ptr(), bias_t.stride(0), bias_t.stride(1)) if bias_t is not None else (None, 0, 0)
        _lib.check(lib.tf_attn_fwd(stream, 0, b, nh, s, hd, qb.data_ptr(), kb.data_ptr(), vb.data_ptr(), ob.data_ptr(),
                                   sb, sh, ss, sb, sh, ss, lse.data_ptr(), *bargs, scale))
        _lib.check(lib.tf_attn_bwd(stream, 0, b, nh, s, hd, qb.data_ptr(), kb.data_ptr(), vb.data_ptr(), ob.data_ptr(),
                                   dob.data_ptr(), dqb.data_ptr(), dkb.data_ptr(), dvb.data_ptr(), sb, sh, ss, sb, sh, ss,
                                   lse.data_ptr(), delta.data_ptr(), *bargs, scale))
    torch.cuda.synchronize()
    view = lambda t: t[:, :s].permute(0, 2, 1, 3)
    qr, kr, vr = (view(t).float().cpu().requires_grad_(True) for t in (qb, kb, vb))
    o_ref = R.causal_attention(qr, kr, vr, bias_ref)
    o_ref.backward(view(dob).float().cpu())
    tag = f"{dims} {bias_kind}"
    assert_close(view(ob), o_ref, name="o " + tag)
    assert_close(view(dqb), qr.grad, name="dq " + tag)
    assert_close(view(dkb), kr.grad, name="dk " + tag)
    assert_close(view(dvb), vr.grad, name="dv " + tag)
    # nothing was written behind the sequences
    for t in (ob, dqb, dkb, dvb):
        assert torch.isnan(t[:, s:]).all()
    assert torch.isnan(lse[b * nh * s:]).all() and torch.isnan(delta[b * nh * s:]).all()
    assert torch.isfinite(lse[: b * nh * s]).all()
