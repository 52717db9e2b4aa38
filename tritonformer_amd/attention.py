"""Causal flash-attention autograd Functions; same classes and ``apply``
signatures as the reference's tritonformer/attention.py."""
from typing import Any, Tuple

import torch
from torch.autograd import Function

from ._amp import amp_bwd, amp_fwd
from .kernels import (
    flash_wrapper_bwd,
    flash_wrapper_bwd_attn_bias,
    flash_wrapper_fwd,
    flash_wrapper_fwd_attn_bias,
)


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
    autocast hook on this class)."""

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
