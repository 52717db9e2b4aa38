"""Autocast hooks for the autograd Functions.

Same behaviour as ``torch.cuda.amp.custom_fwd(cast_inputs=torch.float16)`` /
``custom_bwd`` used by the reference wrappers (e.g. tritonformer/linear.py:14,20):
inside an autocast region every floating-point CUDA tensor argument is cast to
the 16-bit type and the body runs with autocast disabled; outside autocast
nothing is cast.  One extension: when the autocast dtype is bfloat16 the cast
goes to bfloat16 instead of float16 (the reference hard-codes float16).
"""
import functools

import torch


def _cast(value, dtype):
    if isinstance(value, torch.Tensor):
        if value.is_floating_point() and value.is_cuda and value.dtype != torch.float64:
            return value.to(dtype)
        return value
    if isinstance(value, (list, tuple)):
        return type(value)(_cast(v, dtype) for v in value)
    return value


def amp_fwd(fwd=None, *, keep=()):
    """``keep``: positions of arguments that are passed through uncast (small fp32
    parameter vectors the kernel reads directly)."""
    if fwd is None:
        return functools.partial(amp_fwd, keep=keep)

    @functools.wraps(fwd)
    def wrapper(ctx, *args):
        ctx._dtype = torch.get_autocast_dtype("cuda")
        ctx._fwd_used_autocast = False
        # dtypes the caller passed in, before any autocast cast (fp32 master weights)
        ctx.arg_dtypes = tuple(a.dtype if isinstance(a, torch.Tensor) else None for a in args)
        ctx.amp_active = torch.is_autocast_enabled("cuda")  # for bodies that cast their `keep` arguments themselves
        if ctx.amp_active:
            dtype = torch.bfloat16 if ctx._dtype == torch.bfloat16 else torch.float16
            with torch.autocast(device_type="cuda", enabled=False):
                cast = tuple(a if i in keep else _cast(a, dtype) for i, a in enumerate(args))
                return fwd(ctx, *cast)
        return fwd(ctx, *args)

    return wrapper


amp_bwd = torch.amp.custom_bwd(device_type="cuda")
