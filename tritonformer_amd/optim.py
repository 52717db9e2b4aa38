"""AdamW on the GPU as one fused multi-tensor kernel (csrc/optim.hip).  The reference ships no
optimizer; this is the step that turns its timed forward + backward (README.md:62-77) into a
training step: fp32 master parameters, fp32 moments, the arithmetic of ``torch.optim.AdamW``."""
import ctypes
from typing import Optional

import torch

from ._lib import AdamTensor, check, dtype_code, load
from .kernels import require_cuda, stream_ptr


class AdamW(torch.optim.Optimizer):
    """Same constructor arguments and state names (``step``, ``exp_avg``, ``exp_avg_sq``) as
    ``torch.optim.AdamW`` (no amsgrad, no maximize).  Parameters and gradients must be
    contiguous float32 CUDA tensors.  ``shadow_dtype``: also keep a float16 / bfloat16 copy of
    every parameter, rewritten by the same kernel pass (``optimizer.shadow(p)``)."""

    def __init__(self, params, lr: float = 1e-3, betas=(0.9, 0.999), eps: float = 1e-8, weight_decay: float = 1e-2,
                 shadow_dtype: Optional[torch.dtype] = None):
        if lr < 0 or eps < 0 or weight_decay < 0 or not 0 <= betas[0] < 1 or not 0 <= betas[1] < 1:
            raise ValueError("invalid AdamW hyper-parameters")
        if shadow_dtype not in (None, torch.float16, torch.bfloat16):
            raise TypeError("shadow copies are float16 or bfloat16")
        super().__init__(params, dict(lr=lr, betas=betas, eps=eps, weight_decay=weight_decay))
        self.shadow_dtype = shadow_dtype

    def shadow(self, param: torch.Tensor) -> Optional[torch.Tensor]:
        """The 16-bit copy of ``param`` as of the last step (None before the first one)."""
        return self.state[param].get("shadow") if param in self.state else None

    @torch.no_grad()
    def step(self, closure=None):
        loss = None
        if closure is not None:
            with torch.enable_grad():
                loss = closure()
        lib = load()
        for group in self.param_groups:
            by_step = {}
            for p in group["params"]:
                if p.grad is None:
                    continue
                if p.dtype != torch.float32 or p.grad.dtype != torch.float32 or p.grad.is_sparse:
                    raise TypeError("AdamW takes dense float32 parameters and gradients")
                if not p.is_contiguous():
                    raise ValueError("AdamW takes contiguous parameters")
                require_cuda(p, p.grad)
                st = self.state[p]
                if not st:
                    st["step"] = 0
                    st["exp_avg"] = torch.zeros_like(p, memory_format=torch.contiguous_format)
                    st["exp_avg_sq"] = torch.zeros_like(p, memory_format=torch.contiguous_format)
                    if self.shadow_dtype is not None:
                        st["shadow"] = torch.empty_like(p, dtype=self.shadow_dtype, memory_format=torch.contiguous_format)
                st["step"] += 1
                by_step.setdefault(st["step"], []).append((p, p.grad.contiguous(), st))
            for step, items in by_step.items():
                arr = (AdamTensor * len(items))()
                for a, (p, g, st) in zip(arr, items):
                    a.param, a.grad = p.data_ptr(), g.data_ptr()
                    a.exp_avg, a.exp_avg_sq = st["exp_avg"].data_ptr(), st["exp_avg_sq"].data_ptr()
                    a.shadow = st["shadow"].data_ptr() if "shadow" in st else None
                    a.count = p.numel()
                check(lib.tf_adamw_step(stream_ptr(), dtype_code(self.shadow_dtype or torch.float16), len(items),
                                        ctypes.cast(arr, ctypes.c_void_p), group["lr"], group["betas"][0],
                                        group["betas"][1], group["eps"], group["weight_decay"], step))
                # the kernel wrote through raw pointers: tell autograd (and anything keyed on the
                # version counter, like the cache of 16-bit weight copies) that the values changed
                for p, _, _ in items:
                    torch.autograd.graph.increment_version(p)
        return loss
