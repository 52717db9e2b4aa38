"""Cross-entropy autograd Function; same ``apply(logits2d, labels1d) -> (N,)``
as the reference's tritonformer/crossentropy.py."""
from typing import Any, Tuple

import torch
from torch.autograd import Function

from ._amp import amp_bwd, amp_fwd
from .kernels import (
    cross_entropy_bwd,
    cross_entropy_fwd,
    shifted_cross_entropy_bwd,
    shifted_cross_entropy_fwd,
)


class CrossEntropyLoss(Function):
    """Softmax Cross Entropy, one loss value per row."""

    @staticmethod
    @amp_fwd
    def forward(ctx: Any, input: torch.Tensor, labels: torch.Tensor) -> torch.Tensor:
        output, lse, logits, labels = cross_entropy_fwd(input, labels)
        ctx.save_for_backward(labels, logits, lse)
        return output

    @staticmethod
    @amp_bwd
    def backward(ctx: Any, grad_output: torch.Tensor) -> Tuple[torch.Tensor, None]:
        saved_labels, saved_logits, lse = ctx.saved_tensors
        return cross_entropy_bwd(grad_output, saved_logits, saved_labels, lse), None


class ShiftedCrossEntropyLoss(Function):
    """Next-token cross entropy straight from (B, S, V) logits and (B, S) labels:
    ``apply(logits, labels) -> (B*(S-1),)`` equals
    ``CrossEntropyLoss.apply(logits[:, :-1].reshape(-1, V), labels[:, 1:].reshape(-1))``
    without materialising the shifted copy of the logits or of their gradient
    (no counterpart in the reference, which copies: transformer.py:333-341)."""

    @staticmethod
    @amp_fwd
    def forward(ctx: Any, input: torch.Tensor, labels: torch.Tensor) -> torch.Tensor:
        output, lse, logits, shift_labels = shifted_cross_entropy_fwd(input, labels)
        ctx.save_for_backward(shift_labels, logits, lse)
        return output

    @staticmethod
    @amp_bwd
    def backward(ctx: Any, grad_output: torch.Tensor) -> Tuple[torch.Tensor, None]:
        shift_labels, logits, lse = ctx.saved_tensors
        return shifted_cross_entropy_bwd(grad_output, logits, shift_labels, lse), None
