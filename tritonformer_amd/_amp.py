"""Autocast hooks for the autograd Functions.

Same behaviour as ``torch.cuda.amp.custom_fwd(cast_inputs=torch.float16)`` /
``custom_bwd`` used by the reference wrappers (e.g. tritonformer/linear.py:14,20):
inside an autocast region every floating-point CUDA tensor argument is cast to
the 16-bit type and the body runs with autocast disabled; outside autocast
nothing is cast.  One extension: when the autocast dtype is bfloat16 the cast
goes to bfloat16 instead of float16 (the reference hard-codes float16).
"""
import functools
import weakref

import torch

# ---------------------------------------------------------------------------------------------
# 16-bit copies of fp32 master weights, kept between forward passes.
#
# Under autocast every forward pass converts each fp32 weight to 16 bits (the reference keeps
# fp16 parameters and converts nothing).  While a weight does not change -- evaluation, the
# micro-batches of one gradient-accumulation step, a benchmark loop without optimizer -- the
# conversion produces the same bits every time.  With the cache switched on, a conversion is
# redone only when the parameter object, its storage address or its version counter changed.
# The version counter sees every in-place operation on the parameter itself
# (``load_state_dict``, ``torch.optim`` steps, ``tritonformer_amd.optim.AdamW``) but NOT writes
# through ``param.data`` or raw pointers: after such a write call clear_weight_cast_cache().
# Off by default.
# ---------------------------------------------------------------------------------------------
_cache_on = False
_cache = {}


def set_weight_cast_cache(enabled: bool) -> None:
    global _cache_on
    _cache_on = bool(enabled)
    if not _cache_on:
        _cache.clear()


def weight_cast_cache_enabled() -> bool:
    return _cache_on


def clear_weight_cast_cache() -> None:
    _cache.clear()


def cached_conversion(weights, dtype, convert):
    """``convert(weights, dtype)``, or the tensor it returned last time for these very parameters
    if none of them changed since.  Only leaf fp32 parameters are cached."""
    if not _cache_on or not all(isinstance(w, torch.nn.Parameter) and w.dtype == torch.float32 for w in weights):
        return convert(weights, dtype)
    key = tuple(id(w) for w in weights) + (dtype,)
    state = tuple((w.data_ptr(), w._version, tuple(w.shape), tuple(w.stride())) for w in weights)
    hit = _cache.get(key)
    if hit is not None and hit[1] == state and all(r() is w for r, w in zip(hit[0], weights)):
        return hit[2]
    out = convert(weights, dtype)
    # the entry (and the 16-bit copy it holds) goes when any of its parameters does
    refs = tuple(weakref.ref(w, lambda _, key=key: _cache.pop(key, None)) for w in weights)
    _cache[key] = (refs, state, out)
    return out


def _cast(value, dtype):
    if isinstance(value, torch.Tensor):
        if value.is_floating_point() and value.is_cuda and value.dtype != torch.float64:
            if _cache_on and value.dtype == torch.float32 and value.ndim == 2 and isinstance(value, torch.nn.Parameter):
                return cached_conversion([value], dtype, lambda ws, dt: ws[0].to(dt))
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
        # the parameters as the caller holds them (autocast hands the body 16-bit copies): where a deferred
        # gradient is delivered
        ctx.arg_params = tuple(a if isinstance(a, torch.nn.Parameter) else None for a in args)
        if ctx.amp_active:
            dtype = torch.bfloat16 if ctx._dtype == torch.bfloat16 else torch.float16
            with torch.autocast(device_type="cuda", enabled=False):
                cast = tuple(a if i in keep else _cast(a, dtype) for i, a in enumerate(args))
                return fwd(ctx, *cast)
        return fwd(ctx, *args)

    return wrapper


amp_bwd = torch.amp.custom_bwd(device_type="cuda")
