"""Weight gradients handed to the queue that launches them in whole rounds of workgroups
(tritonformer_amd/_deferred.py): the packing rule on the CPU; on the GPU the gradients that reach
``param.grad`` against those of the in-layer launches (the reference's place for them,
tritonformer/linear.py:21-25), accumulation over passes, weights that are not deferred, and a pass
that raised."""
import pytest
import torch

import tritonformer_amd._deferred as D
import tritonformer_amd.transformer as TM
from tests.golden.make_config1_fixture import build_config1
from tests.util import rel_l2
from tritonformer_amd.transformer import Transformer, TransformerConfig


class _Fake:
    def __init__(self, tiles, key=0):
        self.tiles, self.key = tiles, key


def _simulate(d, f, layers, cus=256):
    """Tile sums of the launches that a backward pass over `layers` blocks of width d / f ends in."""
    t = lambda a, b: -(-a // 256) * -(-b // 256)
    pending, launches = [], []

    def drain(final):
        while pending:
            sub = D._next_launch(pending, cus, final)
            if sub is None:
                return
            assert 1 <= len(sub) <= D._MAX_GROUP and len(set(sub)) == len(sub)
            launches.append(sum(pending[i].tiles for i in sub))
            for i in sorted(sub, reverse=True):
                del pending[i]

    for _ in range(layers):
        pending.extend([_Fake(t(d, f)), _Fake(t(f, d))])
        drain(False)
        pending.extend([_Fake(t(d, 3 * d)), _Fake(t(d, d))])
        drain(False)
    drain(True)
    return launches


def test_packing_fills_whole_rounds():
    # 410M: 64 + 64 + 48 + 16 tiles per layer -> 18 launches of exactly one round of 256 workgroups
    assert _simulate(1024, 4096, 24) == [256] * 18
    # 1.4B: every block's pair is a whole number of rounds by itself and goes at once
    assert _simulate(2048, 8192, 24) == [512, 256] * 24
    # 840M: 252 of 256 or 504 of 512 but for the very last product; nothing lost, nothing launched twice
    l840 = _simulate(1536, 6144, 24)
    assert sum(l840) == 24 * 432 and all(D._fill(s, 256) > 0.98 for s in l840[:-1])
    # 160M: no combination of eight products makes a whole round; what goes goes at 91 % and more, and the
    # leftovers of the pass in launches of at most half a round, which the grouped GEMM splits to fill the chip
    l160 = _simulate(768, 3072, 12)
    assert sum(l160) == 12 * 108 and all(s >= 234 or s <= 128 for s in l160)
    # products of another kind (dtype / device) never share a launch with the oldest one
    sub, _ = D._pick([_Fake(128), _Fake(128, key=1), _Fake(128)], 256)
    assert sub == (0, 2)


def test_submit_needs_a_backward_pass_and_leaf_weights():
    with pytest.raises(RuntimeError):
        D.submit([])
    w = torch.nn.Parameter(torch.zeros(4, 4))
    assert D.deferrable((w,))
    assert not D.deferrable((w * 2,)) and not D.deferrable((torch.zeros(4, 4),))
    h = w.register_hook(lambda g: g)
    assert not D.deferrable((w,))
    h.remove()
    assert not D.active()
    with D.scope(True):
        assert D.active()
        with D.scope(False):
            assert not D.active()
    assert not D.active()


def _model(dev):
    cfg, ref, ids = build_config1()
    cfg = TransformerConfig(*[getattr(cfg, k) for k in TransformerConfig.__dataclass_fields__])
    model = Transformer(cfg, device=dev, param_dtype=torch.float32)
    model.load_state_dict(ref.state_dict())
    return model, ids.to(dev)


def _step(model, ids, zero=True):
    if zero:
        model.zero_grad(set_to_none=True)
    with torch.autocast("cuda", dtype=torch.float16):
        _, loss = model(ids, ids)
    (loss * 1024.0).backward()
    return loss.item(), {n: p.grad.clone() for n, p in model.named_parameters()}


@pytest.mark.gpu
def test_deferred_gradients_equal_in_layer_ones(dev):
    model, ids = _model(dev)
    TM.DEFER_DW = False
    try:
        loss0, g0 = _step(model, ids)
    finally:
        TM.DEFER_DW = True
    loss1, g1 = _step(model, ids)
    assert loss0 == loss1 and not D._pending
    for n in g0:
        # same products; the fp32 sums of a contraction are cut at other places
        assert g1[n].dtype == g0[n].dtype and rel_l2(g1[n], g0[n]) < 1e-5, n
    # a second pass without zeroing adds to what is there: the same bits again, so exactly twice
    _, g2 = _step(model, ids, zero=False)
    for n in g1:
        assert torch.equal(g2[n], 2 * g1[n]), n
    # and the pass is repeatable bit for bit
    _, g3 = _step(model, ids)
    assert all(torch.equal(g3[n], g1[n]) for n in g1)


@pytest.mark.gpu
def test_hooked_and_differentiated_weights_are_not_deferred(dev):
    model, ids = _model(dev)
    _, want = _step(model, ids)
    seen = []
    w = model.layer_list[0].attention.q_proj.weight
    handle = w.register_hook(lambda g: seen.append(g.clone()))
    try:
        _, got = _step(model, ids)
    finally:
        handle.remove()
    assert len(seen) == 1 and rel_l2(seen[0], want["layer_list.0.attention.q_proj.weight"]) < 1e-5
    for n in want:
        assert rel_l2(got[n], want[n]) < 1e-5, n
    # torch.autograd.grad with respect to block weights: with the queue off, the Functions return them
    TM.DEFER_DW = False
    try:
        model.zero_grad(set_to_none=True)
        with torch.autocast("cuda", dtype=torch.float16):
            _, loss = model(ids, ids)
        w2 = model.layer_list[1].mlp.dense_4h_to_h.weight
        (gw, gw2) = torch.autograd.grad(loss * 1024.0, [w, w2])
    finally:
        TM.DEFER_DW = True
    assert rel_l2(gw, want["layer_list.0.attention.q_proj.weight"]) < 1e-5
    assert rel_l2(gw2, want["layer_list.1.mlp.dense_4h_to_h.weight"]) < 1e-5
    assert w.grad is None and w2.grad is None


@pytest.mark.gpu
def test_a_pass_that_raised_leaves_nothing_behind(dev):
    model, ids = _model(dev)
    _, want = _step(model, ids)

    def boom(_):
        raise ValueError("stop here")

    # the embedding's gradient is the last one of the pass: every block has handed its products over by then
    handle = model.embed_tokens.weight.register_hook(boom)
    try:
        with pytest.raises(ValueError):
            _step(model, ids)
    finally:
        handle.remove()
    _, got = _step(model, ids)
    assert not D._pending
    for n in want:
        assert torch.equal(got[n], want[n]), n


@pytest.mark.gpu
def test_forward_on_a_stream_of_its_own(dev):
    """The engine runs each backward node on the stream of its forward; what the queue launches when the
    pass ends goes to that stream too, not to the caller's current one."""
    model, ids = _model(dev)
    _, want = _step(model, ids)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    model.zero_grad(set_to_none=True)
    with torch.cuda.stream(side):
        with torch.autocast("cuda", dtype=torch.float16):
            _, loss = model(ids, ids)
        scaled = loss * 1024.0
    scaled.backward()            # called with the default stream current
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    for n, p in model.named_parameters():
        assert torch.equal(p.grad, want[n]), n


@pytest.mark.gpu
@pytest.mark.parametrize("fuse_qkv", [False, True])
def test_reference_named_linears_defer_too(fuse_qkv, dev):
    """With the model-level fusions off the model is the reference's graph node for node
    (LinearNoBias x 4 + LinearNoBiasReLU / LinearNoBias per block, transformer.py:153-217, the LM head a
    Linear as well): their weight gradients take the queue too, and equal the in-layer ones; with
    FUSE_QKV alone the packed projection hands over one product for three weights."""
    model, ids = _model(dev)
    flags = ("FUSE_QKV", "FUSE_MLP", "FUSE_ATTN_BLOCK", "FUSE_ADD_LN", "FUSE_EMBED", "FUSE_HEAD")
    saved = {n: getattr(TM, n) for n in flags}
    try:
        for n in flags:
            setattr(TM, n, False)
        TM.FUSE_QKV = fuse_qkv
        TM.DEFER_DW = False
        loss0, g0 = _step(model, ids)
        TM.DEFER_DW = True
        loss1, g1 = _step(model, ids)
        _, g2 = _step(model, ids)
    finally:
        TM.DEFER_DW = True
        for n, v in saved.items():
            setattr(TM, n, v)
    assert loss0 == loss1 and not D._pending and not D._pending_ln
    for n in g0:
        assert g1[n].dtype == g0[n].dtype and rel_l2(g1[n], g0[n]) < 1e-5, n
        assert torch.equal(g1[n], g2[n]), n
