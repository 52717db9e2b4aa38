"""Cross-entropy autograd Function; same ``apply(logits2d, labels1d) -> (N,)``
as the reference's tritonformer/crossentropy.py."""
from typing import Any, Tuple

import torch
from torch.autograd import Function

from ._amp import amp_bwd, amp_fwd, cached_conversion
from ._lib import KMAJOR, KMINOR
from .kernels import (
    cross_entropy_bwd,
    cross_entropy_fwd,
    gemm_scaled,
    mm,
    mm_dw,
    shifted_cross_entropy_bwd,
    shifted_cross_entropy_fwd,
    shifted_cross_entropy_fwd_grad,
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


class LMHeadLoss(Function):
    """The tail of the reference model (transformer.py:330-343) as ONE autograd node:
    ``apply(hidden (B, S, d), W (d, V), labels (B, S)) -> (logits (B, S, V), loss)`` with
    ``logits = hidden @ W`` and ``loss`` the mean next-token cross entropy over the B*(S-1) shifted
    rows -- what ``linear_no_bias`` + ``shifted_cross_entropy_loss`` + ``.mean()`` return, bit for
    bit.  Being one node it can do what three cannot:
      * the cross-entropy forward writes ``softmax - onehot`` while it still holds each row in
        registers, so the logits are read once instead of twice and the (B, S, V) gradient is
        written once, unscaled (times 1024 in fp16, which keeps probabilities of 1e-5 clear of
        the subnormal range, where ``(softmax - onehot) / N`` in fp16 loses most of its bits);
      * the factor ``grad_loss / N`` (and 1/1024) goes into the write-out of the two LM-head
        gradient products as a device scalar: no pass over the (N, V) matrix for it
        (reference crossentropy.py:24), no host round trip.
    No counterpart in the reference."""

    @staticmethod
    @amp_fwd(keep=(1,))
    def forward(ctx: Any, hidden: torch.Tensor, weight: torch.Tensor, labels: torch.Tensor):
        if weight.dtype != hidden.dtype and ctx.amp_active:
            weight = cached_conversion([weight], hidden.dtype, lambda ws, dt: ws[0].to(dt))
        logits = mm(hidden, weight)
        ctx.set_materialize_grads(False)
        if ctx.needs_input_grad[0] or ctx.needs_input_grad[1]:
            ctx.store_scale = 1024.0 if logits.dtype == torch.float16 else 1.0
            rows, _, dlogits = shifted_cross_entropy_fwd_grad(logits, labels, ctx.store_scale)
            ctx.save_for_backward(hidden, weight, dlogits)
        else:
            rows = shifted_cross_entropy_fwd(logits, labels)[0]
        ctx.rows = rows.numel()
        return logits, rows.mean()

    @staticmethod
    @amp_bwd
    def backward(ctx: Any, grad_logits, grad_loss):
        hidden, weight, dlogits = ctx.saved_tensors
        if grad_logits is None and grad_loss is None:
            return None, None, None
        b, s, v = dlogits.shape
        d = hidden.shape[-1]
        master = torch.float32 if ctx.arg_dtypes[1] == torch.float32 else None
        if grad_logits is not None:
            # the logits were used outside the loss as well: form the whole gradient, then plain products
            total = grad_logits.float()
            if grad_loss is not None:
                total = total + dlogits.float() * (grad_loss.float() / (ctx.rows * ctx.store_scale))
            total = total.to(dlogits.dtype)
            grad_w = mm_dw(hidden, total, out_dtype=master) if ctx.needs_input_grad[1] else None
            grad_h = mm(total, weight.T) if ctx.needs_input_grad[0] else None
            return grad_h, grad_w, None
        alpha = (grad_loss.float() / (ctx.rows * ctx.store_scale)).reshape(1)
        h2, dl2 = hidden.reshape(b * s, d), dlogits.view(b * s, v)
        if not h2.is_contiguous():
            h2 = h2.contiguous()
        grad_w = grad_h = None
        if ctx.needs_input_grad[1]:   # dW = alpha * hidden^T . dlogits, contraction over all tokens
            grad_w = torch.empty((d, v), dtype=master or dlogits.dtype, device=dlogits.device)
            gemm_scaled(h2, KMINOR, d, b * s, d, dl2, KMINOR, v, v, alpha, grad_w)
        if ctx.needs_input_grad[0]:   # dX = alpha * dlogits . W^T, W (d, V) read with the contraction along its rows
            w = weight if weight.stride(-1) == 1 else weight.contiguous()
            grad_h = torch.empty((b, s, d), dtype=dlogits.dtype, device=dlogits.device)
            gemm_scaled(dl2, KMAJOR, b * s, v, v, w, KMAJOR, d, w.stride(0), alpha, grad_h.view(b * s, d))
        return grad_h, grad_w, None
