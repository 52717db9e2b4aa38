"""Host-side mirror of the reference interface: names, constructor signatures,
parameter names and layouts, ALiBi mask, and the no-CPU-fallback rule.  CPU only."""
import inspect

import pytest
import torch

import tritonformer_amd.transformer as TM

import tritonformer_amd as T
from oracle import ref_torch as R
from tritonformer_amd import nn as tnn
from tritonformer_amd.transformer import Transformer, TransformerConfig, generate_alibi_mask, get_slopes


def test_package_aliases_match_reference_init():
    # reference tritonformer/__init__.py:1-8
    for name in ["fast_causal_attention_with_bias", "fast_causal_attention", "cross_entropy_loss", "layer_norm",
                 "linear_bias", "linear_fused_bias_relu", "linear_no_bias", "linear_fused_relu"]:
        assert issubclass(getattr(T, name), torch.autograd.Function)
    assert T.linear_no_bias.__name__ == "LinearNoBias" and T.linear_fused_relu.__name__ == "LinearNoBiasReLU"
    assert T.linear_bias.__name__ == "LinearBias" and T.linear_fused_bias_relu.__name__ == "LinearBiasReLU"


def test_module_constructor_signatures():
    # reference nn.py:17-19, 45-53
    lin = inspect.signature(tnn.Linear.__init__).parameters
    assert list(lin)[1:] == ["in_features", "out_features", "bias", "fuse_activation", "device", "dtype"]
    assert lin["bias"].default is True and lin["fuse_activation"].default is False
    ln = inspect.signature(tnn.LayerNorm.__init__).parameters
    assert list(ln)[1:] == ["normalized_shape", "eps", "device", "dtype"] and ln["eps"].default == 1e-5
    m = tnn.Linear(8, 16, bias=True)
    assert m.weight.shape == (8, 16) and m.bias.shape == (16,)      # weight is (in, out)
    assert tnn.Linear(8, 16, bias=False).bias is None


def test_config_fields():
    assert list(TransformerConfig.__dataclass_fields__) == [
        "vocab_size", "hidden_size", "max_position_embeddings", "num_attention_heads", "head_dim", "ffn_dim",
        "num_hidden_layers", "use_linear_bias", "attn_bias"]


@pytest.mark.parametrize("bias,alibi", [(True, False), (False, True)])
def test_parameter_names_and_shapes_match_oracle_model(bias, alibi):
    cfg = TransformerConfig(512, 64, 64, 2, 32, 128, 2, bias, alibi)
    ours = Transformer(cfg, device="cpu", param_dtype=torch.float32)
    ref = R.RefTransformer(R.RefConfig(512, 64, 64, 2, 32, 128, 2, bias, alibi))
    a = {n: tuple(p.shape) for n, p in ours.named_parameters()}
    b = {n: tuple(p.shape) for n, p in ref.named_parameters()}
    assert a == b
    assert ("embed_positions.weight" in a) == (not alibi)
    assert a["layer_list.0.mlp.dense_h_to_4h.weight"] == (64, 128)
    ours.load_state_dict(ref.state_dict())  # interchangeable, buffers included
    ref.load_state_dict(ours.state_dict())
    if alibi:
        # no dense matrix is kept (the kernels work from the slopes); a state dict still carries it
        assert ours.attn_bias is None and ours.alibi_slopes.dtype == torch.float16
        assert torch.equal(ours.state_dict()["attn_bias"], ref.attn_bias)
        TM.FUSE_ALIBI = False
        try:
            dense = Transformer(cfg, device="cpu", param_dtype=torch.float32)
        finally:
            TM.FUSE_ALIBI = True
        dense.load_state_dict(ours.state_dict())
        assert dense.alibi_slopes is None and torch.equal(dense.attn_bias, ref.attn_bias)


def test_initialisation_follows_reference():
    cfg = TransformerConfig(512, 64, 64, 2, 32, 128, 8, True, False)
    torch.manual_seed(0)
    m = Transformer(cfg, device="cpu", param_dtype=torch.float32)
    assert m.logits_out.weight.abs().max() == 0                      # LM head zeros (transformer.py:104-105)
    assert (m.final_layernorm.weight == 1).all() and (m.final_layernorm.bias == 0).all()
    assert (m.layer_list[0].mlp.dense_h_to_4h.bias == 0).all()
    q_std = m.layer_list[0].attention.q_proj.weight.std().item()
    o_std = m.layer_list[0].attention.out_proj.weight.std().item()
    assert abs(q_std - 0.02) < 0.002 and abs(o_std - 0.02 / 4.0) < 0.001   # 0.02 / sqrt(2 * 8)


def test_alibi_matches_oracle():
    for n in (4, 8, 12, 16, 24):
        assert get_slopes(n) == R.get_slopes(n)
    for s, nh in [(16, 4), (70, 12)]:
        ours = generate_alibi_mask(s, nh)[0]
        assert torch.equal(ours, R.alibi_mask(s, nh))


def test_no_cpu_fallback():
    x = torch.randn(1, 4, 8, dtype=torch.float16)
    w = torch.randn(8, 8, dtype=torch.float16)
    with pytest.raises(ValueError):
        T.linear_no_bias.apply(x, w)
    with pytest.raises(ValueError):
        T.layer_norm.apply(x, torch.ones(8, dtype=torch.float16), torch.zeros(8, dtype=torch.float16), 1e-5)
    with pytest.raises(ValueError):
        T.Softmax.apply(x)


def test_wrapper_preconditions():
    from tritonformer_amd import kernels as K

    h = torch.float16
    with pytest.raises(ValueError):   # 3-D x 2-D only (reference kernels/gemm.py:373)
        K.gemm(torch.zeros(4, 8, dtype=h), torch.zeros(8, 8, dtype=h))
    with pytest.raises(ValueError):   # inner dimensions
        K.gemm(torch.zeros(1, 4, 8, dtype=h), torch.zeros(16, 8, dtype=h))
    q = torch.zeros(1, 2, 100, 64, dtype=h)
    with pytest.raises(ValueError):   # S % 64 (reference kernels/attention.py:181-183)
        K.flash_wrapper_fwd(q, q, q)
    q = torch.zeros(1, 2, 128, 48, dtype=h)
    with pytest.raises(ValueError):   # head_dim (reference kernels/attention.py:567)
        K.flash_wrapper_fwd(q, q, q)
    q = torch.zeros(1, 2, 128, 64, dtype=h)
    with pytest.raises(ValueError):   # bias heads (reference kernels/biased_attention.py:199-207)
        K.flash_wrapper_fwd(q, q, q, torch.zeros(3, 128, 128, dtype=h))
    with pytest.raises(ValueError):
        K.flash_wrapper_fwd(q, q, q, torch.zeros(2, 64, 64, dtype=h))
    with pytest.raises(TypeError):    # fp16/bf16 only (reference kernels/layernorm.py:71)
        K.layernorm_fwd(torch.zeros(1, 4, 8), torch.ones(8), torch.zeros(8), 1e-5)
    with pytest.raises(ValueError):
        K.layernorm_fwd(torch.zeros(4, 8, dtype=h), torch.ones(8, dtype=h), torch.zeros(8, dtype=h), 1e-5)


def test_weight_cast_cache_invalidation():
    """The cache of 16-bit weight copies returns the stored tensor only while the very same parameter
    objects hold the same storage at the same version; in-place updates, a new storage, another
    parameter object or another dtype convert again.  (Host logic: runs on CPU tensors.)"""
    import torch
    from tritonformer_amd import _amp

    calls = []

    def convert(ws, dt):
        calls.append(1)
        return torch.cat([w.to(dt) for w in ws], dim=1)

    a, b = torch.nn.Parameter(torch.randn(4, 3)), torch.nn.Parameter(torch.randn(4, 5))
    assert not _amp.weight_cast_cache_enabled()
    _amp.cached_conversion([a, b], torch.float16, convert)
    _amp.cached_conversion([a, b], torch.float16, convert)
    assert len(calls) == 2                               # off by default: every call converts
    _amp.set_weight_cast_cache(True)
    try:
        first = _amp.cached_conversion([a, b], torch.float16, convert)
        assert _amp.cached_conversion([a, b], torch.float16, convert) is first and len(calls) == 3
        with torch.no_grad():
            a.add_(1.0)                                  # in-place update: version counter moves
        second = _amp.cached_conversion([a, b], torch.float16, convert)
        assert second is not first and len(calls) == 4
        assert torch.equal(second, torch.cat([a.half(), b.half()], dim=1))
        torch.autograd.graph.increment_version(b)        # what the fused AdamW does after its kernel
        assert _amp.cached_conversion([a, b], torch.float16, convert) is not second and len(calls) == 5
        a.data = torch.randn(4, 3)                       # new storage
        _amp.cached_conversion([a, b], torch.float16, convert)
        assert len(calls) == 6
        _amp.cached_conversion([a, b], torch.bfloat16, convert)     # another dtype: its own entry
        assert len(calls) == 7
        _amp.cached_conversion([a.detach(), b.detach()], torch.float16, convert)   # not parameters: never cached
        _amp.cached_conversion([a.detach(), b.detach()], torch.float16, convert)
        assert len(calls) == 9
        _amp.clear_weight_cast_cache()
        _amp.cached_conversion([a, b], torch.float16, convert)
        assert len(calls) == 10
    finally:
        _amp.set_weight_cast_cache(False)
