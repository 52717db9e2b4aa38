"""Cross-entropy autograd Function; same ``apply(logits2d, labels1d) -> (N,)``
as the reference's tritonformer/crossentropy.py."""
from typing import Any, Tuple

import torch
from torch.autograd import Function

from ._amp import amp_bwd, amp_fwd
from .kernels import cross_entropy_bwd, cross_entropy_fwd


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
