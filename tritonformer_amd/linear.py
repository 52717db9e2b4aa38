"""Linear-layer autograd Functions; same classes and ``apply`` signatures as
the reference's tritonformer/linear.py.  Weight layout is (in, out): y = x @ W."""
import torch
from torch.autograd import Function

from . import _deferred
from ._amp import amp_bwd, amp_fwd, cached_conversion
from .kernels import (cast_pack, gemm, gemm_relu_bits, mask_grad, mm, mm_dw, mm_dw_group, mm_masked_bits,
                      unbroadcast_leading)


# True: weight gradients that are available together are computed by one grouped launch
GROUP_DW = True
# True: the fused MLP keeps the ReLU gradient mask as one bit per element, written by the first GEMM
RELU_BITS = True
# True: fp32 master weights of one block are converted to 16 bits by one kernel launch, not one each
PACK_CASTS = True


def _bias_grad(ctx, grad, index):
    """Column sums of ``grad`` as the gradient of the bias passed at argument ``index``: fp32 sums
    stored unrounded for an fp32 master bias (as the weight gradients are), else in 16 bits."""
    return unbroadcast_leading(grad, torch.float32 if ctx.arg_dtypes[index] == torch.float32 else None)


def _deferral_target(ctx, index=1):
    """The weight parameter passed at ``index`` when its gradient is to go through the model's queue
    (several layers' weight gradients in one launch), else None: call in forward, keep on ctx."""
    w = ctx.arg_params[index]
    return w if w is not None and _deferred.active() and GROUP_DW and _deferred.deferrable((w,)) else None


def _grads(ctx, grad_output, inputs, weights):
    """dX = dY W^T (W read as stored, contraction along its rows) and
    dW = X^T dY with the batch folded into the contraction
    (reference linear.py:21-25 goes through bmm + torch.sum)."""
    grad_weights = None
    if ctx.needs_input_grad[1]:
        # an fp32 master weight (cast to 16 bit by autocast on the way in) gets its
        # gradient straight from the fp32 accumulators instead of a rounded copy
        master = torch.float32 if ctx.arg_dtypes[1] == torch.float32 else None
        if getattr(ctx, "defer_to", None) is not None:
            # launched later, together with those of other layers, in whole rounds of workgroups
            _deferred.submit([(inputs, grad_output, 1, (ctx.defer_to,), master)])
        else:
            grad_weights = mm_dw(inputs, grad_output, out_dtype=master)
    # the input gradient last: it is what the next kernel of the backward pass reads
    grad_input = mm(grad_output, weights.T) if ctx.needs_input_grad[0] else None
    return grad_input, grad_weights


class LinearNoBias(Function):
    """MM(X,A) kernel call (reference linear.py:10-25)."""

    @staticmethod
    @amp_fwd
    def forward(ctx, input, weight):
        ctx.save_for_backward(input, weight)
        ctx.defer_to = _deferral_target(ctx)
        return mm(input, weight)

    @staticmethod
    @amp_bwd
    def backward(ctx, grad_output):
        inputs, weights = ctx.saved_tensors
        return _grads(ctx, grad_output, inputs, weights)


class LinearBias(Function):
    """Fused GEMM(X,A,B) in a single kernel call (reference linear.py:28-44)."""

    @staticmethod
    @amp_fwd
    def forward(ctx, input, weight, bias):
        ctx.save_for_backward(input, weight)
        ctx.defer_to = _deferral_target(ctx)
        return gemm(input, weight, bias, False)

    @staticmethod
    @amp_bwd
    def backward(ctx, grad_output):
        inputs, weights = ctx.saved_tensors
        grad_input, grad_weights = _grads(ctx, grad_output, inputs, weights)
        grad_bias = _bias_grad(ctx, grad_output, 2) if ctx.needs_input_grad[2] else None
        return grad_input, grad_weights, grad_bias


class LinearNoBiasReLU(Function):
    """Fused ReLU(MM(X,A)) in a single kernel call (reference linear.py:47-69)."""

    @staticmethod
    @amp_fwd
    def forward(ctx, input, weight):
        out_w_act = mm(input, weight, True)
        ctx.save_for_backward(input, weight, out_w_act)
        ctx.defer_to = _deferral_target(ctx)
        return out_w_act

    @staticmethod
    @amp_bwd
    def backward(ctx, grad_output):
        inputs, weights, out_w_act = ctx.saved_tensors
        grad_output = mask_grad(grad_output, out_w_act)  # new tensor: autograd's buffer stays intact
        return _grads(ctx, grad_output, inputs, weights)


class LinearBiasReLU(Function):
    """Fused ReLU(GEMM(X,A,bias)) in a single kernel call (reference linear.py:72-102)."""

    @staticmethod
    @amp_fwd
    def forward(ctx, input, weight, bias):
        out_w_act = gemm(input, weight, bias, True)
        ctx.save_for_backward(input, weight, out_w_act)
        ctx.defer_to = _deferral_target(ctx)
        return out_w_act

    @staticmethod
    @amp_bwd
    def backward(ctx, grad_output):
        inputs, weights, out_w_act = ctx.saved_tensors
        grad_output = mask_grad(grad_output, out_w_act)
        grad_input, grad_weights = _grads(ctx, grad_output, inputs, weights)
        grad_bias = _bias_grad(ctx, grad_output, 2) if ctx.needs_input_grad[2] else None
        return grad_input, grad_weights, grad_bias


class MLPReLU(Function):
    """Two linears with a ReLU between them as ONE autograd node:
    ``apply(x, W1, b1_or_None, W2, b2_or_None) = relu(x W1 + b1) W2 + b2``.
    Forward and weight/input gradients are the same GEMM calls as
    LinearNoBiasReLU / LinearBiasReLU followed by LinearNoBias / LinearBias; being
    one node lets the ReLU gradient mask ride on the write-out of dH = dY W2^T
    instead of a pass of its own over (B, S, ffn).  No counterpart in the reference
    (two Functions and an in-place mask kernel, linear.py:47-102)."""

    @staticmethod
    @amp_fwd(keep=(1, 3))
    def forward(ctx, input, w1, b1, w2, b2):
        # the weights as the caller holds them: where their gradients go when they are deferred
        ctx.defer_to = (w1, w2) if _deferred.active() and GROUP_DW and _deferred.deferrable((w1, w2)) else None
        if ctx.amp_active and (w1.dtype != input.dtype or w2.dtype != input.dtype):
            # what autocast's cast of the two weights does -- as ONE conversion kernel over both when
            # they are stored alike (two matrices of d*f elements each seen as two rows)
            if (PACK_CASTS and w1.dtype == w2.dtype == torch.float32 and w1.numel() == w2.numel()
                    and w1.is_contiguous() and w2.is_contiguous() and w1.numel() % 8 == 0):
                both = cached_conversion([w1, w2], input.dtype,
                                         lambda ws, dt: cast_pack([ws[0].view(1, -1), ws[1].view(1, -1)], dt))
                w1, w2 = both[0, : w1.numel()].view(w1.shape), both[0, w1.numel():].view(w2.shape)
            else:
                w1, w2 = w1.to(input.dtype), w2.to(input.dtype)
        if RELU_BITS:
            hidden, bits = gemm_relu_bits(input, w1, b1)
        else:
            hidden, bits = gemm(input, w1, b1, True), None
        out = gemm(hidden, w2, b2, False)
        ctx.save_for_backward(input, w1, w2, hidden)
        ctx.relu_bits = bits
        ctx.has_bias = (b1 is not None, b2 is not None)
        return out

    @staticmethod
    @amp_bwd
    def backward(ctx, grad_output):
        input, w1, w2, hidden = ctx.saved_tensors
        f32 = torch.float32
        if ctx.relu_bits is not None:
            # (dY W2^T) * (hidden > 0); `hidden` itself is the mask where this product (contraction
            # over d_out) misses the preconditions that the forward one (over d_in) met
            grad_hidden = mm_masked_bits(grad_output, w2.T, ctx.relu_bits, act=hidden)
        else:
            grad_hidden = mm(grad_output, w2.T, mask_act=hidden)
        grad_b2 = _bias_grad(ctx, grad_output, 4) if ctx.has_bias[1] else None
        # the weight gradients first, the input gradient last: what the next kernel of the backward
        # pass reads is then what was written last (0.1 ms per step of the 410M model)
        if ctx.defer_to is not None and ctx.arg_dtypes[1] == ctx.arg_dtypes[3]:
            # launched later, together with those of other layers, in whole rounds of workgroups
            master = f32 if ctx.arg_dtypes[1] == f32 else None
            _deferred.submit([(input, grad_hidden, 1, ctx.defer_to[:1], master),
                              (hidden, grad_output, 1, ctx.defer_to[1:], master)])
            grad_w1 = grad_w2 = None
        elif GROUP_DW and ctx.arg_dtypes[1] == ctx.arg_dtypes[3]:
            # both weight gradients side by side in one launch
            grad_w1, grad_w2 = mm_dw_group([(input, grad_hidden), (hidden, grad_output)],
                                           out_dtype=f32 if ctx.arg_dtypes[1] == f32 else None)
        else:
            grad_w2 = mm_dw(hidden, grad_output, out_dtype=f32 if ctx.arg_dtypes[3] == f32 else None)
            grad_w1 = mm_dw(input, grad_hidden, out_dtype=f32 if ctx.arg_dtypes[1] == f32 else None)
        grad_b1 = _bias_grad(ctx, grad_hidden, 2) if ctx.has_bias[0] else None
        grad_input = mm(grad_hidden, w1.T) if ctx.needs_input_grad[0] else None
        return grad_input, grad_w1, grad_b1, grad_w2, grad_b2


class PackedLinearNoBias(Function):
    """``apply(x, W_0, ..., W_{c-1})`` (c <= 4 weights of one shape (in, out)) returns
    x @ [W_0 | ... | W_{c-1}], shape (B, S, c*out): c bias-free projections of the same
    input (the q, k, v projections of reference transformer.py:158-160) as ONE product.
    The 16-bit side-by-side operand is built from the weights as they are stored (fp32
    master weights under autocast, or 16-bit) by one conversion kernel; the backward is
    one dX product and one dW product whose column blocks land in c separate contiguous
    gradients.  Same arithmetic per output element as c LinearNoBias calls."""

    @staticmethod
    @amp_fwd(keep=(1, 2, 3, 4))
    def forward(ctx, input, *weights):
        packed = cached_conversion(list(weights), input.dtype, cast_pack)
        ctx.save_for_backward(input, packed)
        ctx.count = len(weights)
        ctx.weight_dtype = weights[0].dtype
        ctx.defer_to = weights if _deferred.active() and GROUP_DW and _deferred.deferrable(weights) else None
        return mm(input, packed)

    @staticmethod
    @amp_bwd
    def backward(ctx, grad_output):
        input, packed = ctx.saved_tensors
        if ctx.defer_to is not None:
            _deferred.submit([(input, grad_output, ctx.count, ctx.defer_to, ctx.weight_dtype)])
            grad_input = mm(grad_output, packed.T) if ctx.needs_input_grad[0] else None
            return (grad_input,) + (None,) * ctx.count
        grad_w = mm_dw(input, grad_output, out_dtype=ctx.weight_dtype, chunks=ctx.count)
        grad_input = mm(grad_output, packed.T) if ctx.needs_input_grad[0] else None
        return (grad_input,) + tuple(grad_w[j] for j in range(ctx.count))
