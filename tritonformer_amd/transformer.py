"""GPT-2 style decoder built on the tritonformer_amd operators.

Host-side counterpart of the reference's top-level ``transformer.py``: the same
``TransformerConfig`` fields, module tree and parameter names
(``embed_tokens``, ``embed_positions``, ``layer_list.{i}.input_layernorm``,
``...attention.{q,k,v,out}_proj``, ``...mlp.dense_h_to_4h`` / ``dense_4h_to_h``,
``final_layernorm``, ``logits_out``, buffer ``attn_bias``), the same
initialisation and the same loss (mean over the B*(S-1) shifted positions), so
a state dict moves between the two unchanged.  Two additions: the device is a
parameter instead of the hard-coded "cuda:0", and ``param_dtype`` selects fp16
parameters (the reference's choice, transformer.py:124-151) or fp32 master
weights used under autocast.
"""
import math
from dataclasses import dataclass
from typing import List, Optional, Tuple

import torch
import torch.nn as nn

from . import (
    add_layer_norm,
    attention_block,
    embedding_sum,
    fast_causal_attention,
    fast_causal_attention_qkvpacked,
    fast_causal_attention_with_bias,
    linear_no_bias_packed,
    lm_head_loss,
    mlp_fused_relu,
    shifted_cross_entropy_loss,
)
from . import _deferred
from . import nn as tnn


@dataclass(frozen=True)
class TransformerConfig:
    vocab_size: int
    hidden_size: int
    max_position_embeddings: int
    num_attention_heads: int
    head_dim: int
    ffn_dim: int
    num_hidden_layers: int
    use_linear_bias: bool
    attn_bias: bool


def get_slopes(n: int) -> List[float]:
    """ALiBi slopes (reference transformer.py:37-52): for n = 2^k the geometric
    sequence 2^(-8/n), 2^(-16/n), ...; otherwise the slopes of the largest
    power of two below n followed by every other slope of the next power."""
    def power_of_two(m):
        base = 2.0 ** (-(2.0 ** -(math.log2(m) - 3)))
        return [base * base ** i for i in range(m)]  # same operation order as the reference: bit-identical slopes

    if n & (n - 1) == 0:
        return power_of_two(n)
    lower = 1 << (n.bit_length() - 1)
    return power_of_two(lower) + get_slopes(2 * lower)[0::2][: n - lower]


def generate_alibi_mask(seq_len: int, num_heads: int, device=None, dtype=torch.float16) -> torch.Tensor:
    """(1, nh, S, S) additive bias: -slope_h * (i - j) for j <= i, -inf above
    the diagonal, with distances, slopes and their product all rounded to
    ``dtype`` as in reference transformer.py:55-75."""
    pos = torch.arange(seq_len, device=device)
    dist = (pos[None, :] - pos[:, None]).clamp(max=0).to(dtype)            # -(i - j) on and below the diagonal
    slopes = torch.tensor(get_slopes(num_heads), device=device, dtype=dtype)
    bias = dist[None] * slopes[:, None, None]
    above = pos[None, :] > pos[:, None]
    return bias.masked_fill(above[None], float("-inf"))[None]


# True: q/k/v projections run as one packed GEMM + packed attention (same parameters and
# arithmetic per output element); False: three projections exactly as the reference
# module does (transformer.py:158-182).
FUSE_QKV = True
# True: the MLP block is one autograd node (ReLU gradient mask fused into a GEMM write-out);
# False: two Linear modules as in the reference (transformer.py:214-217).
FUSE_MLP = True
# True (with FUSE_QKV): projections, attention and output projection are one autograd node, whose
# two weight-gradient products run as one grouped launch.
FUSE_ATTN_BLOCK = True
# True: every residual addition runs inside the LayerNorm kernel that consumes its result
# (forward), and the residual-stream gradient is added inside that LayerNorm's backward
# kernel: no separate elementwise addition kernels.  False: `residual + hidden_states`
# as the reference writes it (transformer.py:245-250).
FUSE_ADD_LN = True
# True: token gather, position gather, their addition and the rounding to the compute type are
# one kernel, and the table gradients a chain-ordered scatter-add; False: two nn.Embedding
# calls and an addition as in the reference (transformer.py:311-323).
FUSE_EMBED = True
# True: LM head, shifted cross-entropy and the mean are one autograd node -- the cross-entropy forward
# writes the logits gradient in the pass that reads the logits, and the 1/N of the mean rides on the
# write-out of the two LM-head gradient GEMMs; False: logits_out module, shifted_cross_entropy_loss
# and .mean() one after the other (the reference's sequence, transformer.py:330-343).
FUSE_HEAD = True
# True (read when a model with attn_bias=True is built): no dense (nh, S, S) ALiBi matrix --
# 805 MB at 24 heads x 4096 -- is made; the attention kernels compute -slope_h * (i - j) from
# the nh slopes with the roundings of that matrix, bit-identical results.  False: the dense
# buffer "attn_bias" as in the reference (transformer.py:296-302).
FUSE_ALIBI = True
# True: the weight gradients of the fused attention and MLP blocks are not launched inside each layer's
# backward but handed to a queue that launches the products of several layers together, in whole
# rounds of one workgroup per CU with unsplit contractions (410M: 1.1 ms per step less).  They are in
# ``param.grad`` when ``backward()`` returns, as before; ``torch.autograd.grad`` with respect to
# those weights needs False.
DEFER_DW = True


def _weights_init(model: nn.Module, num_layers: int) -> None:
    """Reference transformer.py:83-105: N(0, 0.02) for every Linear/Embedding
    weight, N(0, 0.02/sqrt(2L)) for the two residual-output projections, zeros
    for the LM head and all biases, LayerNorm gamma=1 beta=0."""
    for name, m in model.named_modules():
        if isinstance(m, tnn.Linear):
            std = 0.02
            leaf = name.rsplit(".", 1)[-1]
            if leaf in ("out_proj", "dense_4h_to_h"):
                std = 0.02 / math.sqrt(2 * num_layers)
            if leaf == "logits_out":
                m.weight.data.zero_()
            else:
                m.weight.data.normal_(mean=0.0, std=std)
            if m.bias is not None:
                nn.init.zeros_(m.bias)
        elif isinstance(m, nn.Embedding):
            m.weight.data.normal_(mean=0.0, std=0.02)
        elif isinstance(m, tnn.LayerNorm):
            nn.init.ones_(m.weight)
            nn.init.zeros_(m.bias)


class CausalAttention(nn.Module):
    """Self-attention block (reference transformer.py:113-190)."""

    def __init__(self, config: TransformerConfig, device=None, dtype=torch.float16):
        super().__init__()
        self.hidden_size = config.hidden_size
        self.num_attention_heads = config.num_attention_heads
        self.hidden_size_per_attention_head = config.hidden_size // config.num_attention_heads
        kw = dict(device=device, dtype=dtype, bias=False)
        self.q_proj = tnn.Linear(config.hidden_size, config.hidden_size, **kw)
        self.k_proj = tnn.Linear(config.hidden_size, config.hidden_size, **kw)
        self.v_proj = tnn.Linear(config.hidden_size, config.hidden_size, **kw)
        self.out_proj = tnn.Linear(config.hidden_size, config.hidden_size, **kw)

    def _heads(self, x: torch.Tensor) -> torch.Tensor:
        b, s, _ = x.shape  # "b s (nh hd) -> b nh s hd" as a view, strides (S*d, hd, d, 1)
        return x.view(b, s, self.num_attention_heads, self.hidden_size_per_attention_head).permute(0, 2, 1, 3)

    def forward(self, hidden_states: torch.Tensor, attn_bias: Optional[torch.Tensor] = None) -> torch.Tensor:
        batch_size, q_seq_len, hidden_dim = hidden_states.shape
        if FUSE_QKV and FUSE_ATTN_BLOCK:
            return attention_block.apply(hidden_states, self.q_proj.weight, self.k_proj.weight, self.v_proj.weight,
                                         self.out_proj.weight, self.num_attention_heads, attn_bias)
        if FUSE_QKV:
            # one (d, 3d) GEMM instead of three (d, d): same parameters, laid side by side in
            # 16 bits by one conversion kernel; the weight gradient comes back as three tensors
            qkv = linear_no_bias_packed.apply(hidden_states, self.q_proj.weight, self.k_proj.weight,
                                              self.v_proj.weight)
            qkv = qkv.view(batch_size, q_seq_len, 3, self.num_attention_heads, self.hidden_size_per_attention_head)
            return self.out_proj(fast_causal_attention_qkvpacked.apply(qkv, attn_bias))
        query_layer = self._heads(self.q_proj(hidden_states))
        key_layer = self._heads(self.k_proj(hidden_states))
        value_layer = self._heads(self.v_proj(hidden_states))
        if attn_bias is None:
            attn = fast_causal_attention.apply(query_layer, key_layer, value_layer)
        else:
            attn = fast_causal_attention_with_bias.apply(query_layer, key_layer, value_layer, attn_bias)
        # attn keeps q's strides, so this is a view, not a copy
        context_layer = attn.transpose(1, 2).contiguous().view(batch_size, q_seq_len, hidden_dim)
        return self.out_proj(context_layer)


class MLPBlock(nn.Module):
    """Linear(+bias)+ReLU fused, then Linear(+bias) (reference transformer.py:193-217)."""

    def __init__(self, config: TransformerConfig, device=None, dtype=torch.float16):
        super().__init__()
        self.dense_h_to_4h = tnn.Linear(config.hidden_size, config.ffn_dim, device=device, dtype=dtype,
                                        fuse_activation=True, bias=config.use_linear_bias)
        self.dense_4h_to_h = tnn.Linear(config.ffn_dim, config.hidden_size, device=device, dtype=dtype,
                                        bias=config.use_linear_bias)

    def forward(self, hidden_states: torch.Tensor) -> torch.Tensor:
        if FUSE_MLP:
            return mlp_fused_relu.apply(hidden_states, self.dense_h_to_4h.weight, self.dense_h_to_4h.bias,
                                        self.dense_4h_to_h.weight, self.dense_4h_to_h.bias)
        return self.dense_4h_to_h(self.dense_h_to_4h(hidden_states))


class TransformerLayer(nn.Module):
    """Pre-LN block (reference transformer.py:220-251)."""

    def __init__(self, config: TransformerConfig, device=None, dtype=torch.float16):
        super().__init__()
        self.input_layernorm = tnn.LayerNorm(config.hidden_size, device=device, dtype=dtype)
        self.post_attention_layernorm = tnn.LayerNorm(config.hidden_size, device=device, dtype=dtype)
        self.attention = CausalAttention(config, device=device, dtype=dtype)
        self.mlp = MLPBlock(config, device=device, dtype=dtype)

    def forward(self, hidden_states: torch.Tensor, attn_bias: Optional[torch.Tensor] = None) -> torch.Tensor:
        hidden_states = hidden_states + self.attention(self.input_layernorm(hidden_states), attn_bias)
        return hidden_states + self.mlp(self.post_attention_layernorm(hidden_states))

    def forward_deferred(self, hidden_states: torch.Tensor, pending: Optional[torch.Tensor],
                         attn_bias: Optional[torch.Tensor] = None):
        """Same block with the additions folded into the LayerNorms: takes the residual stream
        and a branch output not yet added to it (None for the first block), returns the stream
        after the attention residual and this block's MLP output, still to be added."""
        ln1, ln2 = self.input_layernorm, self.post_attention_layernorm
        if pending is None:
            normed = ln1(hidden_states)
        else:
            hidden_states, normed = add_layer_norm.apply(hidden_states, pending, ln1.weight, ln1.bias, ln1.eps)
        attn_out = self.attention(normed, attn_bias)
        hidden_states, normed = add_layer_norm.apply(hidden_states, attn_out, ln2.weight, ln2.bias, ln2.eps)
        return hidden_states, self.mlp(normed)


class Transformer(nn.Module):
    """Decoder stack + LM head + shifted cross-entropy (reference transformer.py:254-346)."""

    def __init__(self, config: TransformerConfig, device=None, param_dtype=torch.float16):
        super().__init__()
        self.config = config
        self.embed_tokens = nn.Embedding(config.vocab_size, config.hidden_size, device=device, dtype=param_dtype)
        self.embed_positions = None
        if not config.attn_bias:
            self.embed_positions = nn.Embedding(config.max_position_embeddings, config.hidden_size, device=device,
                                                dtype=param_dtype)
        self.layer_list = nn.ModuleList(
            [TransformerLayer(config, device=device, dtype=param_dtype) for _ in range(config.num_hidden_layers)]
        )
        self.final_layernorm = tnn.LayerNorm(config.hidden_size, device=device, dtype=param_dtype)
        self.logits_out = tnn.Linear(config.hidden_size, config.vocab_size, bias=False, device=device,
                                     dtype=param_dtype, fuse_activation=False)
        _weights_init(self, config.num_hidden_layers)
        if config.attn_bias and FUSE_ALIBI:
            # the kernels rebuild the bias from the slopes; a checkpoint's dense "attn_bias" entry
            # is dropped on load and regenerated on save, so state dicts stay interchangeable
            self.attn_bias = None
            self.register_buffer("alibi_slopes", torch.tensor(get_slopes(config.num_attention_heads), device=device,
                                                              dtype=torch.float16), persistent=False)
            self._register_load_state_dict_pre_hook(lambda state, prefix, *_: state.pop(prefix + "attn_bias", None))

            def add_dense_bias(module, state, prefix, _metadata):
                # a saved state dict still holds the reference's buffer, built when it is asked for
                state[prefix + "attn_bias"] = generate_alibi_mask(
                    config.max_position_embeddings, config.num_attention_heads, device=module.alibi_slopes.device)[0]

            self._register_state_dict_hook(add_dense_bias)
        elif config.attn_bias:
            self.alibi_slopes = None
            # the bias is an activation-side tensor: always 16-bit, like the reference's
            self.register_buffer(
                "attn_bias",
                generate_alibi_mask(config.max_position_embeddings, config.num_attention_heads, device=device)[0],
            )
        else:
            self.attn_bias = self.alibi_slopes = None

    def forward(self, input_ids: torch.Tensor, labels: Optional[torch.Tensor]):
        batch_size, seq_len = input_ids.shape
        attn_bias = self.attn_bias
        # under autocast the residual stream is kept in the 16-bit compute type, as it is in
        # the reference (whose embeddings are fp16 parameters, transformer.py:259-272)
        amp_dtype = torch.get_autocast_dtype("cuda") if torch.is_autocast_enabled("cuda") else None
        if FUSE_EMBED and input_ids.is_cuda:
            # gathers, addition and the rounding to the compute type in one kernel
            pos_w = None if self.embed_positions is None else self.embed_positions.weight
            hidden_states = embedding_sum.apply(input_ids, self.embed_tokens.weight, pos_w, amp_dtype)
        else:
            hidden_states = self.embed_tokens(input_ids)
            if self.embed_positions is not None:
                positions = torch.arange(seq_len, device=hidden_states.device)[None].expand(batch_size, -1)
                hidden_states = hidden_states + self.embed_positions(positions)
            if amp_dtype is not None:
                hidden_states = hidden_states.to(amp_dtype)
        if amp_dtype is not None and attn_bias is not None:
            attn_bias = attn_bias.to(amp_dtype)
        if self.alibi_slopes is not None:
            attn_bias = self.alibi_slopes
        with _deferred.scope(DEFER_DW):
            if FUSE_ADD_LN and len(self.layer_list) > 0:
                pending = None
                for layer in self.layer_list:
                    hidden_states, pending = layer.forward_deferred(hidden_states, pending, attn_bias)
                ln = self.final_layernorm
                _, hidden_states = add_layer_norm.apply(hidden_states, pending, ln.weight, ln.bias, ln.eps)
            else:
                for layer in self.layer_list:
                    hidden_states = layer(hidden_states, attn_bias)
                hidden_states = self.final_layernorm(hidden_states)
        head = self.logits_out
        if (FUSE_HEAD and labels is not None and isinstance(head, tnn.Linear) and head.bias is None
                and not head.fuse_activation and hidden_states.is_cuda):
            return lm_head_loss.apply(hidden_states, head.weight, labels)   # (logits, mean shifted loss)
        logits_lm = head(hidden_states)
        if labels is None:
            return logits_lm
        # same rows and labels as the reference's shift-copy-then-cross-entropy
        # (transformer.py:333-341), read from logits_lm in place
        loss = shifted_cross_entropy_loss.apply(logits_lm, labels)
        return logits_lm, loss.mean()
