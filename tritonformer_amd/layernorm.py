"""LayerNorm autograd Function; same ``apply(input, alpha, beta, eps)`` as the
reference's tritonformer/layernorm.py."""
from torch.autograd import Function

from ._amp import amp_bwd, amp_fwd
from .kernels import layernorm_bwd, layernorm_fwd


class LayerNorm(Function):
    @staticmethod
    @amp_fwd(keep=(1, 2))  # fp32 master gamma / beta are read by the kernel as they are
    def forward(ctx, input, alpha, beta, eps):
        x_ln, mean, rstd = layernorm_fwd(input, alpha, beta, eps)
        ctx.save_for_backward(input, alpha, mean, rstd)
        ctx.eps = eps
        return x_ln

    @staticmethod
    @amp_bwd
    def backward(ctx, grad_output):
        input, alpha, mean, rstd = ctx.saved_tensors
        grad_input, grad_alpha, grad_beta = layernorm_bwd(grad_output, input, alpha, mean, rstd)
        return grad_input, grad_alpha, grad_beta, None
