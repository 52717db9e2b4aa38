"""Causal flash-attention autograd Functions; same classes and ``apply``
signatures as the reference's tritonformer/attention.py."""
from typing import Any, Tuple

import torch
from torch.autograd import Function

from . import _deferred
from ._amp import amp_bwd, amp_fwd, cached_conversion
from .kernels import (
    cast_pack,
    flash_wrapper_bwd,
    flash_wrapper_bwd_attn_bias,
    flash_wrapper_fwd,
    flash_wrapper_fwd_attn_bias,
    mm,
    mm_dw_group,
)


def _bias_for(attn_bias, dtype):
    """A dense bias in the compute dtype (what autocast's cast of the argument would give);
    ALiBi slopes -- a (nh,) vector -- stay float16, the precision the reference builds its
    bias matrix from."""
    if attn_bias is None or attn_bias.ndim == 1 or attn_bias.dtype == dtype:
        return attn_bias
    return attn_bias.to(dtype)


class CausalAttention(Function):
    """softmax(causal(Q K^T / sqrt(hd))) V (reference attention.py:13-34)."""

    @staticmethod
    @amp_fwd
    def forward(ctx: Any, query: torch.Tensor, key: torch.Tensor, value: torch.Tensor) -> torch.Tensor:
        out, lse = flash_wrapper_fwd(query, key, value)
        ctx.save_for_backward(lse, query, key, value, out)
        return out

    @staticmethod
    @amp_bwd
    def backward(ctx: Any, grad_output: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
        lse, query, key, value, out = ctx.saved_tensors
        return flash_wrapper_bwd(grad_output, out, query, key, value, lse)


class BiasedCausalAttention(Function):
    """As CausalAttention with ``+ attn_bias[h, i, j]`` added to the scaled
    scores; no gradient for the bias (reference attention.py:37-60, which has no
    autocast hook on this class).  Extension: ``attn_bias`` may be the (nh,) float16
    vector of ALiBi slopes instead of the dense (nh, S, S) matrix built from them
    (reference transformer.py:55-75); the results are the same bit for bit."""

    @staticmethod
    def forward(ctx: Any, query: torch.Tensor, key: torch.Tensor, value: torch.Tensor,
                attn_bias: torch.Tensor) -> torch.Tensor:
        out, lse = flash_wrapper_fwd_attn_bias(query, key, value, attn_bias)
        ctx.save_for_backward(lse, query, key, value, out, attn_bias)
        return out

    @staticmethod
    def backward(ctx: Any, grad_output: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor, None]:
        lse, query, key, value, out, attn_bias = ctx.saved_tensors
        dq, dk, dv = flash_wrapper_bwd_attn_bias(grad_output, out, query, key, value, lse, attn_bias)
        return dq, dk, dv, None


class PackedCausalAttention(Function):
    """Causal attention on a packed projection: ``apply(qkv, attn_bias_or_None)``
    with qkv (B, S, 3, nh, hd) -- the output of ONE (d, 3d) GEMM -- returns
    (B, S, nh*hd); the backward writes dq, dk, dv straight into one packed
    (B, S, 3, nh, hd) gradient, so the projection's dX and dW are single GEMMs
    too.  Same kernels as CausalAttention / BiasedCausalAttention, which take the
    three strided slices as they are.  No counterpart in the reference (three
    separate projections, transformer.py:158-175)."""

    @staticmethod
    @amp_fwd(keep=(1,))
    def forward(ctx: Any, qkv: torch.Tensor, attn_bias) -> torch.Tensor:
        if qkv.ndim != 5 or qkv.shape[2] != 3:
            raise ValueError("packed attention takes qkv of shape (B, S, 3, nh, hd)")
        attn_bias = _bias_for(attn_bias, qkv.dtype)
        if not qkv.is_contiguous():
            qkv = qkv.contiguous()
        b, s, _, nh, hd = qkv.shape
        q, k, v = (qkv[:, :, i].permute(0, 2, 1, 3) for i in range(3))
        out = torch.empty((b, s, nh, hd), dtype=qkv.dtype, device=qkv.device)
        _, lse = flash_wrapper_fwd(q, k, v, attn_bias, out=out.permute(0, 2, 1, 3))
        ctx.save_for_backward(lse, qkv, out, attn_bias)
        return out.view(b, s, nh * hd)

    @staticmethod
    @amp_bwd
    def backward(ctx: Any, grad_output: torch.Tensor):
        lse, qkv, out, attn_bias = ctx.saved_tensors
        b, s, _, nh, hd = qkv.shape
        q, k, v = (qkv[:, :, i].permute(0, 2, 1, 3) for i in range(3))
        dqkv = torch.empty_like(qkv)
        grads = tuple(dqkv[:, :, i].permute(0, 2, 1, 3) for i in range(3))
        grad_output = grad_output.reshape(b, s, nh, hd).permute(0, 2, 1, 3)
        flash_wrapper_bwd(grad_output, out.permute(0, 2, 1, 3), q, k, v, lse, attn_bias, grads=grads)
        return dqkv, None


class AttentionBlock(Function):
    """The whole self-attention block of the reference model (transformer.py:153-190) as
    ONE autograd node: ``apply(x, Wq, Wk, Wv, Wo, nh, attn_bias_or_None)`` =
    ``attention(x Wq, x Wk, x Wv) Wo`` for bias-free projections (in, out) = (d, d).
    Same GEMM and attention kernels as linear_no_bias_packed, fast_causal_attention_qkvpacked
    and linear_no_bias one after the other; being one node, the weight gradients of the
    packed q/k/v projection and of the output projection -- outputs with few tiles each --
    are computed by one grouped launch."""

    @staticmethod
    @amp_fwd(keep=(1, 2, 3, 4, 6))
    def forward(ctx: Any, x, wq, wk, wv, wo, num_heads, attn_bias):
        if x.ndim != 3 or wq.shape != (x.shape[-1], x.shape[-1]) or wo.shape != wq.shape:
            raise ValueError("attention block takes x (B, S, d) and four (d, d) weights")
        attn_bias = _bias_for(attn_bias, x.dtype)
        b, s, d = x.shape
        hd = d // num_heads
        weights = (wq, wk, wv, wo)
        same = all(w.dtype == wq.dtype for w in weights)
        # the weights as the caller holds them: where their gradients go when they are deferred
        ctx.defer_to = weights if _deferred.active() and same and _deferred.deferrable(weights) else None
        # the four (d, d) weights side by side in one 16-bit (d, 4d) matrix, one conversion kernel;
        # the GEMMs take its first three column blocks and its last one as strided operands
        packed = cached_conversion([wq, wk, wv, wo], x.dtype, cast_pack)
        w_qkv, w_o = packed[:, : 3 * d], packed[:, 3 * d:]
        qkv = mm(x, w_qkv).view(b, s, 3, num_heads, hd)
        q, k, v = (qkv[:, :, i].permute(0, 2, 1, 3) for i in range(3))
        attn = torch.empty((b, s, num_heads, hd), dtype=x.dtype, device=x.device)
        _, lse = flash_wrapper_fwd(q, k, v, attn_bias, out=attn.permute(0, 2, 1, 3))
        attn = attn.view(b, s, d)
        ctx.save_for_backward(x, packed, qkv, attn, lse, attn_bias)
        ctx.weight_dtype = wq.dtype
        return mm(attn, w_o)

    @staticmethod
    @amp_bwd
    def backward(ctx: Any, grad_output: torch.Tensor):
        x, packed, qkv, attn, lse, attn_bias = ctx.saved_tensors
        b, s, _, nh, hd = qkv.shape
        w_qkv, w_o = packed[:, : 3 * nh * hd], packed[:, 3 * nh * hd:]
        d_attn = mm(grad_output, w_o.T).view(b, s, nh, hd).permute(0, 2, 1, 3)
        q, k, v = (qkv[:, :, i].permute(0, 2, 1, 3) for i in range(3))
        dqkv = torch.empty_like(qkv)
        grads = tuple(dqkv[:, :, i].permute(0, 2, 1, 3) for i in range(3))
        flash_wrapper_bwd(d_attn, attn.view(b, s, nh, hd).permute(0, 2, 1, 3), q, k, v, lse, attn_bias, grads=grads)
        dqkv = dqkv.view(b, s, 3 * nh * hd)
        if ctx.defer_to is not None:
            # launched later, together with those of other layers, in whole rounds of workgroups
            _deferred.submit([(x, dqkv, 3, ctx.defer_to[:3], ctx.weight_dtype),
                              (attn, grad_output, 1, ctx.defer_to[3:], ctx.weight_dtype)])
            grad_x = mm(dqkv, w_qkv.T) if ctx.needs_input_grad[0] else None
            return grad_x, None, None, None, None, None, None
        # weight gradients first, the input gradient (what the next kernel reads) last
        d_wqkv, d_wo = mm_dw_group([(x, dqkv), (attn, grad_output)], out_dtype=ctx.weight_dtype, chunks=[3, 1])
        grad_x = mm(dqkv, w_qkv.T) if ctx.needs_input_grad[0] else None
        return grad_x, d_wqkv[0], d_wqkv[1], d_wqkv[2], d_wo, None, None
