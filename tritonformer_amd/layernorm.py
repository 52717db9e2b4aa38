"""LayerNorm autograd Function; same ``apply(input, alpha, beta, eps)`` as the
reference's tritonformer/layernorm.py."""
from torch.autograd import Function

from . import _deferred
from ._amp import amp_bwd, amp_fwd
from .kernels import add_layernorm_bwd, add_layernorm_fwd, layernorm_bwd, layernorm_fwd


def _deferral_targets(alpha, beta):
    """(gamma, beta) as the caller holds them when their gradients are to be summed at the end of the
    backward pass, all LayerNorms in one launch; None when the Function returns them itself."""
    if _deferred.active() and alpha.dtype == beta.dtype and _deferred.deferrable((alpha, beta)):
        return (alpha, beta)
    return None


class LayerNorm(Function):
    @staticmethod
    @amp_fwd(keep=(1, 2))  # fp32 master gamma / beta are read by the kernel as they are
    def forward(ctx, input, alpha, beta, eps):
        x_ln, mean, rstd = layernorm_fwd(input, alpha, beta, eps)
        ctx.save_for_backward(input, alpha, mean, rstd)
        ctx.eps = eps
        ctx.defer_to = _deferral_targets(alpha, beta)
        return x_ln

    @staticmethod
    @amp_bwd
    def backward(ctx, grad_output):
        input, alpha, mean, rstd = ctx.saved_tensors
        if ctx.defer_to is not None:
            grad_input, partial = layernorm_bwd(grad_output, input, alpha, mean, rstd, leave_partials=True)
            _deferred.submit_layernorm(partial, alpha.shape[0], ctx.defer_to)
            return grad_input, None, None, None
        grad_input, grad_alpha, grad_beta = layernorm_bwd(grad_output, input, alpha, mean, rstd)
        return grad_input, grad_alpha, grad_beta, None


class AddLayerNorm(Function):
    """``apply(x, branch, alpha, beta, eps) -> (x + branch, layernorm(x + branch))``: the
    residual addition of the reference's TransformerLayer (transformer.py:245-246, :250)
    and the LayerNorm that follows it as one graph node with one kernel per direction.
    Both outputs are differentiable; the backward returns one tensor as the gradient of
    both summands."""

    @staticmethod
    @amp_fwd(keep=(2, 3))
    def forward(ctx, x, branch, alpha, beta, eps):
        total, x_ln, mean, rstd = add_layernorm_fwd(x, branch, alpha, beta, eps)
        ctx.save_for_backward(total, alpha, mean, rstd)
        ctx.set_materialize_grads(False)  # an unused output arrives as None, not as zeros
        ctx.defer_to = _deferral_targets(alpha, beta)
        return total, x_ln

    @staticmethod
    @amp_bwd
    def backward(ctx, grad_total, grad_ln):
        total, alpha, mean, rstd = ctx.saved_tensors
        if grad_ln is None:  # only the sum was used downstream
            return grad_total, grad_total, None, None, None
        leave = ctx.defer_to is not None
        if grad_total is None:
            dx, *rest = layernorm_bwd(grad_ln, total, alpha, mean, rstd, leave_partials=leave)
        else:
            dx, *rest = add_layernorm_bwd(grad_ln, grad_total, total, alpha, mean, rstd, leave_partials=leave)
        if leave:
            _deferred.submit_layernorm(rest[0], alpha.shape[0], ctx.defer_to)
            return dx, dx, None, None, None
        return dx, dx, rest[0], rest[1], None
