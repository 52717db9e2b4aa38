"""Parameter gradients of the transformer blocks, launched when it suits the GPU rather than the graph.

A weight gradient dW = X^T dY is needed by nobody until the backward pass ends, and the output of one
such product has few 256x256 tiles (16 to 64 per weight of the 410M model on 256 CUs): launched where
the reference launches it (linear.py:21-25, inside the layer's backward) it fills the chip only by
splitting its contraction, which costs fp32 partial sums and a second pass.  Here the linear and block
Functions that run inside the model's forward hand their (X, dY) pairs over instead; products of several layers are launched together as soon as their
tiles make (nearly) whole rounds of one workgroup per CU, unsplit, and what is left goes when the
engine finishes the pass.  The gradients are complete, on the stream the pass ran on, when
``loss.backward()`` returns -- the same contract as before -- but they reach ``param.grad`` directly
instead of through the Function's return value: a weight that is not a leaf, or carries hooks, is not
deferred, and ``torch.autograd.grad`` with respect to such a weight must run with deferral off
(it reports the weight as unused otherwise).

The LayerNorms of the model use the same queue for the second stage of their gamma / beta gradients: the
row pass leaves the column sums of its row blocks in place, and one launch at the end of the pass sums
those of every LayerNorm (the reference launches that stage once per LayerNorm, kernels/layernorm.py:226-259).
"""
import contextlib

import torch

from .kernels import layernorm_param_grads, mm_dw_group

# products per launch (the grouped GEMM entry point takes up to sixteen)
_MAX_GROUP = 16
# a launch goes as soon as its tiles fill this share of a whole number of rounds
_FILL = 0.97
# pending products beyond which the oldest are launched whatever they fill (bounds the memory held)
_MAX_PENDING = 24

_enabled = False
_pending = []
_pending_ln = []
_task = None
_stream = None
_cus = {}


@contextlib.contextmanager
def scope(enabled):
    """Block Functions whose forward runs inside ``scope(True)`` defer their weight gradients."""
    global _enabled
    previous = _enabled
    _enabled = bool(enabled)
    try:
        yield
    finally:
        _enabled = previous


def active():
    return _enabled


def deferrable(params):
    """True when every weight is a leaf that takes its gradient in ``.grad`` and nobody watches it arrive."""
    for p in params:
        if not (isinstance(p, torch.Tensor) and p.is_leaf and p.requires_grad):
            return False
        if p._backward_hooks or getattr(p, "_post_accumulate_grad_hooks", None):
            return False
    return True


class _Product:
    __slots__ = ("x", "grad", "chunks", "params", "out_dtype", "tiles", "key")

    def __init__(self, x, grad, chunks, params, out_dtype):
        self.x, self.grad, self.chunks, self.params, self.out_dtype = x, grad, chunks, params, out_dtype
        kin, nout = x.shape[-1], grad.shape[-1]
        self.tiles = -(-kin // 256) * -(-nout // 256)
        self.key = (x.dtype, out_dtype or x.dtype, x.device)


def _round(device):
    n = _cus.get(device)
    if n is None:
        n = _cus[device] = torch.cuda.get_device_properties(device).multi_processor_count
    return n


def _fill(tiles, cus):
    return tiles / (-(-tiles // cus) * cus)


def _fill_split(tiles, cus):
    """The share of the chip a launch keeps busy when the grouped GEMM may split contractions: at most half
    a round of tiles runs as cus // tiles slices per tile (fp32 partial sums and a second pass: rated 0.9)."""
    if 2 * tiles <= cus:
        return 0.9 * tiles * (cus // tiles) / cus
    return _fill(tiles, cus)


def _pick(items, cus, rate=_fill):
    """Indices of up to _MAX_GROUP products (of the first one's kind) whose tiles best fill whole rounds;
    among equals the oldest, then the most tiles.  Returns (indices, fill)."""
    reach = {0: ()}
    for idx, it in enumerate(items):
        if it.key != items[0].key:
            continue
        for s, sub in list(reach.items()):
            if len(sub) < _MAX_GROUP and s + it.tiles not in reach:
                reach[s + it.tiles] = sub + (idx,)
    best, best_rank = None, None
    for s, sub in reach.items():
        if not sub:
            continue
        f = rate(s, cus)
        rank = (min(f, _FILL), 0 in sub, s)
        if best_rank is None or rank > best_rank:
            best, best_rank = sub, rank
    return best, best_rank[0]


def _launch(items):
    pairs = [(it.x, it.grad) for it in items]
    outs = mm_dw_group(pairs, out_dtype=items[0].out_dtype, chunks=[it.chunks for it in items])
    with torch.no_grad():
        for it, out in zip(items, outs):
            grads = [out] if it.chunks == 1 else [out[j] for j in range(it.chunks)]
            for p, g in zip(it.params, grads):
                if p.grad is None:
                    p.grad = g
                else:
                    p.grad.add_(g)


def _next_launch(items, cus, final):
    """Indices of the products to launch now, or None to wait for more."""
    sub, fill = _pick(items, cus)
    if fill < _FILL:
        if not final and len(items) < _MAX_PENDING:
            return None
        # nothing more is coming (or too much is held): what fills the chip best, split contractions included
        sub, fill = _pick(items, cus, _fill_split)
    return sub


def _drain(final):
    while _pending:
        sub = _next_launch(_pending, _round(_pending[0].x.device), final)
        if sub is None:
            return
        items = [_pending[i] for i in sub]
        for i in reversed(sub):
            del _pending[i]
        _launch(items)


def _finish_ln():
    # one launch per kind (width, parameter dtype, device) -- one kind in a model
    kinds = {}
    for partial, d, params in _pending_ln:
        kinds.setdefault((d, params[0].dtype, partial[0].device), []).append((partial, params))
    with torch.no_grad():
        for (d, dtype, _), members in kinds.items():
            out = layernorm_param_grads([m[0] for m in members], d, dtype)
            for i, (_, params) in enumerate(members):
                for j, p in enumerate(params):
                    if p.grad is None:
                        p.grad = out[i, j]
                    else:
                        p.grad.add_(out[i, j])


def _finish():
    global _task, _stream
    _task = None
    try:
        # on the stream the pass ran on (the engine runs this on the thread that called backward(), whose
        # current stream is another one when the forward pass ran under a stream of its own)
        with torch.cuda.stream(_stream):
            _drain(final=True)
            if _pending_ln:
                _finish_ln()
    finally:
        _stream = None
        _pending.clear()
        _pending_ln.clear()


def _join_pass():
    global _task, _stream
    task = torch._C._current_graph_task_id()
    if task < 0:
        raise RuntimeError("deferred parameter gradients are submitted from inside a backward pass")
    if task != _task:
        # first submission of this pass (what an earlier pass that raised left behind is dropped)
        _pending.clear()
        _pending_ln.clear()
        _task = task
        _stream = torch.cuda.current_stream()
        torch.autograd.Variable._execution_engine.queue_callback(_finish)


def submit_layernorm(partial, d, params):
    """``partial``: what layernorm_bwd(..., leave_partials=True) returned beside dx; ``params`` = (gamma, beta)
    of width ``d``, whose ``.grad`` receive the sums when the pass ends."""
    _join_pass()
    _pending_ln.append((partial, d, tuple(params)))


def submit(products):
    """``products``: (x, grad, chunks, params, out_dtype) -- dW = x^T grad in ``out_dtype`` (None: the
    operands'), cut into ``chunks`` equal column blocks, block j added to ``params[j].grad``.  Call from
    inside a backward pass only."""
    _join_pass()
    for x, grad, chunks, params, out_dtype in products:
        _pending.append(_Product(x, grad, chunks, tuple(params), out_dtype))
    _drain(final=False)
