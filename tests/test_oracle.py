"""Pins the PyTorch fp32 oracle (oracle/ref_torch.py) before anything is compared
with it: against the brute-force C restatement (oracle/ref_ops.c, explicit
closed-form backward passes), against library routines, and against what the
mathematics fixes.  CPU only."""
import math

import numpy as np
import pytest
import torch
import torch.nn.functional as F

from oracle import ref_torch as R
from tests.util import RefOps, f32

torch.manual_seed(0)
np.random.seed(0)
ref = RefOps()


def close(a, b, tol=2e-5):
    a = torch.as_tensor(a).float()
    b = torch.as_tensor(b).float()
    assert a.shape == b.shape
    assert (a - b).abs().max().item() <= tol * (1 + b.abs().max().item()), (a - b).abs().max().item()


@pytest.mark.parametrize("m,k,n,bias,relu", [(7, 13, 5, False, False), (16, 33, 24, True, False),
                                             (9, 17, 31, False, True), (12, 8, 40, True, True)])
def test_linear_vs_bruteforce(m, k, n, bias, relu):
    x, w = torch.randn(1, m, k), torch.randn(k, n) / k ** 0.5
    b = torch.randn(n) if bias else None
    dy = torch.randn(1, m, n)
    y = R.linear(x, w, b, relu)
    yc = np.empty((m, n), np.float32)
    ref.call("ref_linear_fwd", m, n, k, f32(x), f32(w), f32(b) if bias else None, int(relu), yc)
    close(y[0], yc)
    dx, dw, db = R.linear_bwd(x, w, dy, act=y if relu else None, with_bias=bias)
    dxc, dwc, dbc = np.empty((m, k), np.float32), np.empty((k, n), np.float32), np.empty(n, np.float32)
    ref.call("ref_linear_bwd", m, n, k, f32(x), f32(w), f32(dy), f32(y) if relu else None, dxc, dwc,
             dbc if bias else None)
    close(dx[0], dxc)
    close(dw, dwc)
    if bias:
        close(db, dbc)
    # closed-form backward == autograd of the forward expression
    xa, wa = x.clone().requires_grad_(True), w.clone().requires_grad_(True)
    ba = b.clone().requires_grad_(True) if bias else None
    R.linear(xa, wa, ba, relu).backward(dy)
    close(dx, xa.grad)
    close(dw, wa.grad)
    if bias:
        close(db, ba.grad)


def test_linear_known_answers():
    x = torch.randn(2, 5, 6)
    close(R.linear(x, torch.eye(6)), x)                      # identity weight
    perm = torch.randperm(6)
    close(R.linear(x, torch.eye(6)[:, perm]), x[..., perm])  # permutation weight: W is (in, out)
    w = torch.randn(6, 4)
    close(R.linear(x, w, relu=True), torch.relu(R.linear(x, w)))
    # rows whose outputs are all <= 0 get a zero input gradient through the ReLU
    xn = -x.abs()
    wp = w.abs()
    y = R.linear(xn, wp, relu=True)
    assert (y == 0).all()
    dx, dw, _ = R.linear_bwd(xn, wp, torch.randn_like(y), act=y)
    assert (dx == 0).all() and (dw == 0).all()


@pytest.mark.parametrize("rows,d", [(5, 8), (11, 33), (4, 256)])
def test_layernorm_vs_bruteforce_and_library(rows, d):
    x = 3.14 + 0.4 * torch.randn(1, rows, d)
    g, b, dy = torch.randn(d), torch.randn(d), torch.randn(1, rows, d)
    y = R.layer_norm(x, g, b, 1e-5)
    yc = np.empty((rows, d), np.float32)
    ref.call("ref_layernorm_fwd", rows, d, f32(x), f32(g), f32(b), 1e-5, yc)
    close(y[0], yc, 1e-4)
    close(y, F.layer_norm(x, (d,), g, b, 1e-5), 1e-5)
    dx, dg, db = R.layer_norm_bwd(x, g, dy, 1e-5)
    dxc, dgc, dbc = np.empty((rows, d), np.float32), np.empty(d, np.float32), np.empty(d, np.float32)
    ref.call("ref_layernorm_bwd", rows, d, f32(x), f32(g), f32(dy), 1e-5, dxc, dgc, dbc)
    close(dx[0], dxc, 2e-4)
    close(dg, dgc, 2e-4)
    close(db, dbc, 2e-4)
    xa, ga, ba = (t.clone().requires_grad_(True) for t in (x, g, b))
    F.layer_norm(xa, (d,), ga, ba, 1e-5).backward(dy)
    close(dx, xa.grad, 1e-4)
    close(dg, ga.grad, 1e-4)
    close(db, ba.grad, 1e-4)
    # invariants: every dx row sums to zero; a constant row normalises to beta
    assert dx.sum(-1).abs().max() < 1e-3
    close(R.layer_norm(torch.full((1, 2, d), 7.0), g, b), b.expand(1, 2, d), 1e-3)


@pytest.mark.parametrize("rows,cols", [(3, 7), (8, 65), (2, 1000)])
def test_softmax_vs_bruteforce(rows, cols):
    x, dy = torch.randn(1, rows, cols), 0.1 * torch.randn(1, rows, cols)
    y = R.softmax(x)
    yc, dxc = np.empty((rows, cols), np.float32), np.empty((rows, cols), np.float32)
    ref.call("ref_softmax_fwd", rows, cols, f32(x), yc)
    close(y[0], yc)
    ref.call("ref_softmax_bwd", rows, cols, f32(y), f32(dy), dxc)
    dx = R.softmax_bwd(y, dy)
    close(dx[0], dxc)
    xa = x.clone().requires_grad_(True)
    R.softmax(xa).backward(dy)
    close(dx, xa.grad)
    close(y.sum(-1), torch.ones(1, rows), 1e-6)        # rows sum to one
    close(R.softmax(x + 3.0), y, 1e-6)                 # shift invariance
    assert dx.sum(-1).abs().max() < 1e-6               # gradient rows sum to zero


@pytest.mark.parametrize("rows,v", [(4, 11), (9, 300), (3, 50304)])
def test_cross_entropy_vs_bruteforce(rows, v):
    x = torch.randn(rows, v)
    lab = torch.randint(0, v, (rows,))
    g = torch.randn(rows)
    loss = R.cross_entropy(x, lab)
    lc, dc = np.empty(rows, np.float32), np.empty((rows, v), np.float32)
    ref.call("ref_cross_entropy_fwd", rows, v, f32(x), np.ascontiguousarray(lab.numpy()), lc)
    close(loss, lc)
    ref.call("ref_cross_entropy_bwd", rows, v, f32(x), np.ascontiguousarray(lab.numpy()), f32(g), dc)
    close(R.cross_entropy_bwd(x, lab, g), dc)
    xa = x.clone().requires_grad_(True)
    R.cross_entropy(xa, lab).backward(g)
    close(R.cross_entropy_bwd(x, lab, g), xa.grad)
    # uniform logits: loss = ln V exactly
    close(R.cross_entropy(torch.zeros(rows, v), lab), torch.full((rows,), math.log(v)), 1e-6)
    # numpy logsumexp restatement
    xn = x.double().numpy()
    lse = np.log(np.exp(xn - xn.max(1, keepdims=True)).sum(1)) + xn.max(1)
    close(loss, lse - xn[np.arange(rows), lab.numpy()], 1e-5)


@pytest.mark.parametrize("bh,nh,s,hd,bias", [(2, 2, 8, 4, False), (3, 3, 16, 8, True), (2, 1, 33, 16, False)])
def test_attention_vs_bruteforce(bh, nh, s, hd, bias):
    q, k, v, do = (torch.randn(bh // nh, nh, s, hd) for _ in range(4))
    b = None
    if bias:
        b = R.alibi_mask(s + 4, nh, dtype=torch.float32)   # bias larger than S: top-left block is used
    o = R.causal_attention(q, k, v, b)
    oc, dqc, dkc, dvc = (np.empty((bh, s, hd), np.float32) for _ in range(4))
    bias_np = None
    if bias:
        bias_np = f32(b).copy()
        bias_np[np.isinf(bias_np)] = 0.0  # the C loops never touch keys above the diagonal
    ref.call("ref_attention", bh, nh, s, hd, f32(q), f32(k), f32(v), bias_np, s + 4 if bias else 0, oc, f32(do),
             dqc, dkc, dvc)
    close(o.reshape(bh, s, hd), oc)
    qa, ka, va = (t.clone().requires_grad_(True) for t in (q, k, v))
    R.causal_attention(qa, ka, va, b).backward(do)
    close(qa.grad.reshape(bh, s, hd), dqc, 1e-4)
    close(ka.grad.reshape(bh, s, hd), dkc, 1e-4)
    close(va.grad.reshape(bh, s, hd), dvc, 1e-4)


def test_attention_invariants():
    q, k, v = (torch.randn(2, 3, 24, 16) for _ in range(3))
    o = R.causal_attention(q, k, v)
    close(o, F.scaled_dot_product_attention(q, k, v, is_causal=True), 1e-5)   # library routine
    close(o[:, :, 0], v[:, :, 0], 1e-6)                                       # first row sees only key 0
    causal_bias = torch.zeros(3, 24, 24).masked_fill(torch.triu(torch.ones(24, 24, dtype=torch.bool), 1),
                                                     float("-inf"))
    close(R.causal_attention(q, k, v, causal_bias), o, 1e-6)                  # 0 / -inf bias == no bias
    assert (o.amax(-2) <= v.amax(-2) + 1e-5).all() and (o.amin(-2) >= v.amin(-2) - 1e-5).all()  # convex combos


def test_alibi_closed_forms():
    assert R.get_slopes(8) == [2.0 ** -(i + 1) for i in range(8)]
    np.testing.assert_allclose(R.get_slopes(16), [2.0 ** (-0.5 * (i + 1)) for i in range(16)], rtol=1e-12)
    s24 = R.get_slopes(24)
    np.testing.assert_allclose(s24[:16], R.get_slopes(16), rtol=1e-12)
    np.testing.assert_allclose(s24[16:], [2.0 ** (-0.25 * (2 * j + 1)) for j in range(8)], rtol=1e-12)
    np.testing.assert_allclose(s24[-3:], [0.148651, 0.105112, 0.074325], rtol=1e-5)
    m = R.alibi_mask(6, 4)
    assert m.shape == (4, 6, 6) and m.dtype == torch.float16
    assert torch.isinf(m[:, 0, 1:]).all() and (m.diagonal(dim1=1, dim2=2) == 0).all()
    slopes = torch.tensor(R.get_slopes(4), dtype=torch.float16)
    assert torch.equal(m[:, 5, 2], (torch.tensor(-3.0, dtype=torch.float16) * slopes))


def test_embedding_vs_loops_and_library():
    """The oracle's embedding and its gradient against element loops, F.embedding's autograd
    and the one-hot matrix product (ids with repeats, so the scatter-add is exercised)."""
    torch.manual_seed(3)
    b, s, d, v, p = 2, 5, 3, 4, 7
    ids = torch.randint(0, v, (b, s))
    tok, pos = torch.randn(v, d), torch.randn(p, d)
    out = R.embedding(ids, tok, pos)
    for i in range(b):
        for j in range(s):
            for c in range(d):
                assert out[i, j, c].item() == (tok[ids[i, j], c] + pos[j, c]).item()
    assert torch.equal(R.embedding(ids, tok), tok[ids])
    g = torch.randn(b, s, d)
    d_tok, d_pos = R.embedding_bwd(ids, g, v, p)
    loop_tok, loop_pos = torch.zeros(v, d, dtype=torch.float64), torch.zeros(p, d, dtype=torch.float64)
    for i in range(b):
        for j in range(s):
            loop_tok[ids[i, j]] += g[i, j].double()
            loop_pos[j] += g[i, j].double()
    assert torch.allclose(d_tok.double(), loop_tok, atol=1e-6) and torch.allclose(d_pos.double(), loop_pos, atol=1e-6)
    assert torch.count_nonzero(d_pos[s:]) == 0
    tok_a, pos_a = tok.clone().requires_grad_(True), pos.clone().requires_grad_(True)
    lib = F.embedding(ids, tok_a) + F.embedding(torch.arange(s)[None].expand(b, -1), pos_a)
    assert torch.equal(lib, out)
    lib.backward(g)
    assert torch.allclose(tok_a.grad, d_tok, atol=1e-6) and torch.allclose(pos_a.grad, d_pos, atol=1e-6)
    onehot = F.one_hot(ids.reshape(-1), v).float()
    assert torch.allclose(onehot.T @ g.reshape(b * s, d), d_tok, atol=1e-6)


def test_adamw_vs_library_and_first_step_closed_form():
    torch.manual_seed(5)
    p0 = torch.randn(37, 11)
    hyper = dict(lr=3e-3, betas=(0.9, 0.95), eps=1e-8, weight_decay=0.1)
    lib_p = p0.clone().requires_grad_(True)
    opt = torch.optim.AdamW([lib_p], **hyper)
    p, m, v = p0.clone(), torch.zeros_like(p0), torch.zeros_like(p0)
    for step in range(1, 6):
        g = torch.randn_like(p0) * (0.1 * step)
        lib_p.grad = g.clone()
        opt.step()
        p, m, v = R.adamw_step(p, g, m, v, step, **hyper)
        assert torch.allclose(p, lib_p.detach(), rtol=1e-6, atol=1e-7), step
        if step == 1:  # m / sqrt(v) = sign(g) after bias correction: p1 = p0 (1 - lr wd) - lr sign(g)
            want = p0 * (1 - hyper["lr"] * hyper["weight_decay"]) - hyper["lr"] * torch.sign(g)
            assert torch.allclose(p, want, rtol=1e-5, atol=1e-6)
    st = opt.state[lib_p]
    assert torch.allclose(m, st["exp_avg"], rtol=1e-6, atol=1e-8) and torch.allclose(v, st["exp_avg_sq"], rtol=1e-6, atol=1e-10)


def test_model_known_answers():
    cfg = R.RefConfig(50304, 64, 32, 2, 32, 128, 2, True, False)
    torch.manual_seed(0)
    m = R.RefTransformer(cfg)
    ids = torch.randint(0, 50304, (2, 32))
    logits, loss = m(ids, ids)
    # zero-initialised LM head: uniform prediction, loss = ln(vocab), no gradient reaches the stack
    assert abs(loss.item() - math.log(50304)) < 1e-5
    loss.backward()
    for name, p in m.named_parameters():
        if not name.startswith("logits_out"):
            assert p.grad is None or p.grad.abs().max() == 0, name
    assert m.logits_out.weight.grad.abs().max() > 0
    assert logits.shape == (2, 32, 50304)
    assert abs(R.step_flops(cfg, 2, 32) - (6 * 64 * (2 * (4 * 64 * 64 + 2 * 64 * 128) + 64 * 50304)
                                           + 7 * 2 * 2 * 32 * 32 * 64)) < 1


def test_model_flops_table():
    # the five baseline configurations: total TFLOP per step as tabulated for the benchmark
    table = {(24, 1024, 4096, 2048, 4): 20.262, (12, 768, 3072, 2048, 8): 14.312, (4, 256, 1024, 256, 2): 0.0502,
             (24, 1536, 6144, 4096, 1): 22.927, (24, 2048, 8192, 2048, 2): 35.105}
    for (L, d, f, S, B), tf in table.items():
        cfg = R.RefConfig(50304, d, S, 16, d // 16, f, L, False, False)
        assert abs(R.step_flops(cfg, B, S) / 1e12 - tf) < 2e-3 * tf + 1e-4


def test_model_golden_fixture():
    """Config 1 of the baseline (seed 0): loss and per-parameter gradient norms
    committed under tests/golden/ by make_config1_fixture.py."""
    import json
    import os

    from tests.golden.make_config1_fixture import run_config1

    path = os.path.join(os.path.dirname(__file__), "golden", "config1_fixture.json")
    want = json.load(open(path))
    got = run_config1()
    assert abs(got["loss"] - want["loss"]) <= 1e-5 * abs(want["loss"])
    for name, norm in want["grad_norms"].items():
        assert abs(got["grad_norms"][name] - norm) <= 1e-3 * norm + 1e-9, name


# --------------------------------------------------------------------------- block wiring of the oracle model
def _random_norm_params(model):
    """LayerNorm gamma / beta away from (1, 0): with the initial values a LayerNorm applied
    twice equals one applied once, and a misplaced one would go unnoticed."""
    g = torch.Generator().manual_seed(5)
    for name, p in model.named_parameters():
        if "layernorm" in name:
            p.data = (torch.rand(p.shape, generator=g) + 0.5) if name.endswith("weight") else torch.randn(p.shape, generator=g) * 0.3


def _branch_outputs(model, ids):
    """logits plus what each attention / MLP module returned, in call order."""
    seen, hooks = [], []
    for layer in model.layer_list:
        hooks.append(layer.attention.register_forward_hook(lambda m, i, o: seen.append(("attn", o.detach()))))
        hooks.append(layer.mlp.register_forward_hook(lambda m, i, o: seen.append(("mlp", o.detach()))))
    with torch.no_grad():
        logits = model(ids, None)
    for h in hooks:
        h.remove()
    return logits, seen


@pytest.mark.parametrize("alibi", [False, True])
def test_model_wiring_is_pre_ln_with_both_residuals(alibi):
    """What reference transformer.py:238-251, 311-331 fixes, checked on quantities a wrong wiring
    changes: (a) the residual stream is the embedding plus every branch output, and the logits
    are final_layernorm(stream) @ W_out -- a dropped residual, a branch added to the normalised
    input or a LayerNorm on the stream (post-LN) fails it; (b) each branch reads a LayerNorm of
    the stream, so scaling the embeddings by c leaves the first attention output unchanged, and
    the first MLP output too once the attention output is silenced; (c) with both output
    projections zero the logits are LN_f(embedding) @ W_out in closed form."""
    cfg = R.RefConfig(97, 32, 24, 4, 8, 64, 3, True, alibi)
    torch.manual_seed(3)
    model = R.RefTransformer(cfg)
    model.logits_out.weight.data.normal_(0.0, 0.3)
    _random_norm_params(model)
    for name, p in model.named_parameters():   # biases away from zero as well
        if name.endswith("bias") and "layernorm" not in name:
            p.data.normal_(0.0, 0.1)
    ids = torch.randint(0, 97, (2, 24))

    def embed(m):
        x = m.embed_tokens.weight[ids]
        if m.embed_positions is not None:
            x = x + m.embed_positions.weight[torch.arange(24)][None]
        return x.detach()

    def head(m, x):
        f = m.final_layernorm
        return F.layer_norm(x, (32,), f.weight, f.bias, f.eps) @ m.logits_out.weight

    # (a) stream = embedding + all branch outputs
    logits, seen = _branch_outputs(model, ids)
    assert [k for k, _ in seen] == ["attn", "mlp"] * 3
    stream = embed(model) + sum(o for _, o in seen)
    close(logits, head(model, stream).detach())
    # the branch inputs are LayerNorms of the running stream: recompute branch by branch
    x = embed(model)
    bias = model.attn_bias
    for li, layer in enumerate(model.layer_list):
        ln1, ln2 = layer.input_layernorm, layer.post_attention_layernorm
        a = layer.attention(F.layer_norm(x, (32,), ln1.weight, ln1.bias, ln1.eps), bias).detach()
        close(a, seen[2 * li][1])
        x = x + a
        m = layer.mlp(F.layer_norm(x, (32,), ln2.weight, ln2.bias, ln2.eps)).detach()
        close(m, seen[2 * li + 1][1])
        x = x + m

    # (b) pre-LN: branches do not see the scale of the stream
    scaled = R.RefTransformer(cfg)
    scaled.load_state_dict(model.state_dict())
    scaled.embed_tokens.weight.data *= 7.0
    if scaled.embed_positions is not None:
        scaled.embed_positions.weight.data *= 7.0
    for m in (model, scaled):
        for layer in m.layer_list:
            layer.input_layernorm.eps = layer.post_attention_layernorm.eps = 0.0   # exact scale invariance
    _, seen1 = _branch_outputs(model, ids)
    _, seen7 = _branch_outputs(scaled, ids)
    close(seen7[0][1], seen1[0][1], tol=1e-4)                    # first attention output: unchanged
    assert (seen7[1][1] - seen1[1][1]).abs().max() > 1e-3        # first MLP saw stream = c x + a: changed
    for m in (model, scaled):
        m.layer_list[0].attention.out_proj.weight.data.zero_()
    _, seen1 = _branch_outputs(model, ids)
    _, seen7 = _branch_outputs(scaled, ids)
    assert seen1[0][1].abs().max() == 0
    close(seen7[1][1], seen1[1][1], tol=1e-4)                    # ... now the first MLP output is unchanged too

    # (c) both output projections zero: logits = LN_f(embedding) @ W_out
    for layer in model.layer_list:
        layer.attention.out_proj.weight.data.zero_()
        layer.mlp.dense_4h_to_h.weight.data.zero_()
        layer.mlp.dense_4h_to_h.bias.data.zero_()
    with torch.no_grad():
        logits0 = model(ids, None)
    close(logits0, head(model, embed(model)).detach())


def test_model_loss_is_the_shifted_mean():
    """reference transformer.py:332-343: row (b, s), s < S-1, is scored against labels[b, s+1];
    the loss is the mean over the B*(S-1) rows."""
    cfg = R.RefConfig(53, 16, 12, 2, 8, 32, 1, False, False)
    torch.manual_seed(4)
    model = R.RefTransformer(cfg)
    model.logits_out.weight.data.normal_(0.0, 0.5)
    ids, labels = torch.randint(0, 53, (3, 12)), torch.randint(0, 53, (3, 12))
    with torch.no_grad():
        logits, loss = model(ids, labels)
    lp = torch.log_softmax(logits.double(), -1)
    want = -sum(lp[b, s, labels[b, s + 1]] for b in range(3) for s in range(11)) / 33
    assert abs(loss.item() - want.item()) < 1e-5
