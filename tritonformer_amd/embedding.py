"""Token + position embedding as one autograd Function.  The reference leaves this part
of the model to two nn.Embedding modules and an addition (transformer.py:259-272,
311-323); the parameters keep those modules' names and shapes, this Function only
replaces the three PyTorch kernels of the forward (two gathers, one add, plus the cast
of the residual stream under autocast) and the sort-based scatter of the backward."""
from typing import Any, Optional

import torch
from torch.autograd import Function

from .kernels import embedding_bwd, embedding_fwd


class EmbeddingSum(Function):
    """``apply(ids, token_table, position_table_or_None, out_dtype_or_None)`` ->
    ``token_table[ids] + position_table[arange(S)]`` of shape (B, S, d) in ``out_dtype``
    (default: the tables' dtype).  Table gradients come back in the tables' dtype."""

    @staticmethod
    def forward(ctx: Any, ids: torch.Tensor, tok_w: torch.Tensor, pos_w: Optional[torch.Tensor],
                out_dtype: Optional[torch.dtype]) -> torch.Tensor:
        out = embedding_fwd(ids, tok_w, pos_w, tok_w.dtype if out_dtype is None else out_dtype)
        ctx.save_for_backward(ids)
        ctx.tok_shape = tuple(tok_w.shape)
        ctx.pos_shape = None if pos_w is None else tuple(pos_w.shape)
        ctx.param_dtype = tok_w.dtype
        return out

    @staticmethod
    def backward(ctx: Any, grad_output: torch.Tensor):
        (ids,) = ctx.saved_tensors
        want_pos = ctx.pos_shape is not None and ctx.needs_input_grad[2]
        d_tok, d_pos = embedding_bwd(grad_output, ids, ctx.tok_shape, ctx.pos_shape if want_pos else None,
                                     ctx.param_dtype)
        return None, d_tok, d_pos, None
