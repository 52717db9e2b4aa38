"""Launcher functions: torch tensors in, one C-ABI call each, torch tensors out.

They take the place of the launchers under the reference's
``tritonformer/kernels/`` (``mm``/``gemm``/``bmm``, ``flash_wrapper_*``,
``layernorm_fwd``/``dx_layernorm``/``layernorm_da_db``, ``softmax_*``,
``cross_entropy_*``, ``unbroadcast_leading``, ``mask_grad``).  Outputs and
scratch buffers are ``torch.empty`` tensors owned by the caller's allocator;
the native side keeps nothing.
"""
import ctypes
import math
from functools import lru_cache

import torch

from . import _lib
from ._lib import KMAJOR, KMINOR, check, dtype_code, load, require_cuda, stream_ptr


def _rows2d(x):
    """View x as (rows, last) with a single row stride; copy only if needed."""
    if x.stride(-1) != 1 or not x.is_contiguous():
        x = x.contiguous()
    return x, x.numel() // x.shape[-1], x.shape[-1]


@lru_cache(maxsize=None)
def _gemm_ws(la, lb, m, n, k):
    return load().tf_gemm_workspace_bytes(la, lb, m, n, k)


def _gemm(dtype, la, lb, m, n, k, a, lda, b, ldb, c, ldc, bias, relu, mask=None, chunk_n=0, chunk_stride=0):
    lib = load()
    ws_bytes = 0 if mask is not None else _gemm_ws(la, lb, m, n, k)
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=c.device) if ws_bytes else None
    check(lib.tf_gemm_out_chunked(stream_ptr(), dtype_code(dtype), dtype_code(c.dtype), la, lb, m, n, k, a.data_ptr(),
                                  lda, b.data_ptr(), ldb, c.data_ptr(), ldc, chunk_n, chunk_stride,
                                  bias.data_ptr() if bias is not None else None, int(relu),
                                  mask.data_ptr() if mask is not None else None, n if mask is not None else 0,
                                  ws.data_ptr() if ws is not None else None, ws_bytes))


def _gemm_group(dtype, out_dtype, la, lb, problems, device):
    """One tf_gemm_group call for a ctypes array of GemmProblem."""
    lib = load()
    n = len(problems)
    ws_bytes = lib.tf_gemm_group_workspace_bytes(la, lb, n, problems)
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=device) if ws_bytes else None
    check(lib.tf_gemm_group(stream_ptr(), dtype_code(dtype), dtype_code(out_dtype), la, lb, n, problems,
                            ws.data_ptr() if ws is not None else None, ws_bytes))


def _check_linear(a, b, bias=None):
    # same preconditions as kernels/gemm.py:370-377, 584-591 of the reference
    if a.ndim != 3 or b.ndim != 2:
        raise ValueError("Incorrect number of dimensions for LHS or RHS")
    if a.shape[2] != b.shape[0]:
        raise ValueError("Inner dimensions of the two operands do not match")
    if a.dtype not in (torch.float16, torch.bfloat16):
        raise TypeError("linear kernels take float16 or bfloat16 operands (use autocast for fp32 parameters)")
    if a.dtype != b.dtype or (bias is not None and bias.dtype != a.dtype):
        raise TypeError("operands must share one 16-bit dtype")
    if bias is not None and (bias.ndim != 1 or bias.shape[0] != b.shape[1]):
        raise ValueError("bias must have one entry per output column")
    require_cuda(a, b, bias)


def _operand_b(b, n, k):
    if b.stride(-1) == 1 and b.stride(0) >= n:
        return b, KMINOR, b.stride(0)          # (in, out) row-major: contraction strided
    if b.stride(0) == 1 and b.stride(1) >= k:
        return b, KMAJOR, b.stride(1)          # a transposed view, as linear.py:23 passes
    return b.contiguous(), KMINOR, n


def gemm(a, b, bias=None, fuse_relu=False, mask_act=None):
    """``relu?(a @ b + bias)`` for a (B, S, in), b (in, out) — reference ``mm``
    (kernels/gemm.py:361-401) and ``gemm`` (kernels/gemm.py:572-616).
    ``mask_act`` (same shape as the result): zero the result where it is <= 0,
    i.e. reference ``mask_grad`` (kernels/activation.py:27-44) fused into the GEMM
    that produces the gradient being masked."""
    _check_linear(a, b, bias)
    if mask_act is not None:
        if bias is not None or fuse_relu:
            raise ValueError("mask_act excludes bias and ReLU")
        if mask_act.shape != a.shape[:-1] + (b.shape[1],) or mask_act.dtype != a.dtype:
            raise ValueError("mask_act must have the shape and dtype of the result")
        if not mask_act.is_contiguous():
            mask_act = mask_act.contiguous()
    a2, m, k = _rows2d(a)
    n = b.shape[1]
    b, lb, ldb = _operand_b(b, n, k)
    if bias is not None and not bias.is_contiguous():
        bias = bias.contiguous()
    out = torch.empty(a.shape[:-1] + (n,), dtype=a.dtype, device=a.device)
    _gemm(a.dtype, KMAJOR, lb, m, n, k, a2, k, b, ldb, out, n, bias, fuse_relu, mask_act)
    return out


_BITS_NOT_SERVED = -4  # TF_ESHAPE from tf_gemm_relu_bits: the product misses the bit kernel's preconditions


def _gemm_bits(dtype, lb, m, n, k, a, b, ldb, c, bias, bits_out, bits_in):
    """One tf_gemm_relu_bits call (A contraction-contiguous); returns the status code."""
    return load().tf_gemm_relu_bits(stream_ptr(), dtype_code(dtype), dtype_code(dtype), KMAJOR, lb, m, n, k,
                                    a.data_ptr(), k, b.data_ptr(), ldb, c.data_ptr(), n,
                                    bias.data_ptr() if bias is not None else None,
                                    bits_out.data_ptr() if bits_out is not None else None,
                                    bits_in.data_ptr() if bits_in is not None else None, n // 8)


def gemm_relu_bits(a, b, bias=None):
    """``relu(a @ b + bias)`` and its sign bits: a uint8 tensor (rows, out / 8), bit n % 8 of byte
    n / 8 of a row set where the result is positive -- the ReLU gradient mask at a sixteenth of
    the activation's size (reference mask_grad reads the activation, kernels/activation.py:27-44).
    The bits are None when the kernel that produces them cannot take the problem."""
    _check_linear(a, b, bias)
    a2, m, k = _rows2d(a)
    n = b.shape[1]
    b, lb, ldb = _operand_b(b, n, k)
    if bias is not None and not bias.is_contiguous():
        bias = bias.contiguous()
    out = torch.empty(a.shape[:-1] + (n,), dtype=a.dtype, device=a.device)
    if n % 8 == 0:
        bits = torch.empty((m, n // 8), dtype=torch.uint8, device=a.device)
        rc = _gemm_bits(a.dtype, lb, m, n, k, a2, b, ldb, out, bias, bits, None)
        if rc == 0:
            return out, bits
        if rc != _BITS_NOT_SERVED:
            check(rc)
    _gemm(a.dtype, KMAJOR, lb, m, n, k, a2, k, b, ldb, out, n, bias, True, None)
    return out, None


def mm_masked_bits(a, b, bits, act=None):
    """``(a @ b) * mask`` with the mask given as the sign bits of gemm_relu_bits.  The kernel that
    reads the bits has preconditions of its own (whole 64-wide contraction steps, aligned
    operands) which this product may miss although the one that wrote the bits met them; ``act``,
    the activation the bits were taken from, then serves as the mask (``mm(..., mask_act=act)``)."""
    _check_linear(a, b, None)
    a2, m, k = _rows2d(a)
    n = b.shape[1]
    if bits.dtype != torch.uint8 or bits.shape != (m, n // 8) or n % 8 or not bits.is_contiguous():
        raise ValueError("bits must be the contiguous (rows, out / 8) uint8 tensor of gemm_relu_bits")
    require_cuda(bits)
    b, lb, ldb = _operand_b(b, n, k)
    out = torch.empty(a.shape[:-1] + (n,), dtype=a.dtype, device=a.device)
    rc = _gemm_bits(a.dtype, lb, m, n, k, a2, b, ldb, out, None, None, bits)
    if rc == _BITS_NOT_SERVED and act is not None:
        return gemm(a, b, None, False, act)  # any other status is an error and is raised below
    check(rc)
    return out


def _gemm_scaled(dtype, la, lb, m, n, k, a, lda, b, ldb, c, ldc, alpha):
    lib = load()
    ws_bytes = _gemm_ws(la, lb, m, n, k)
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=c.device) if ws_bytes else None
    check(lib.tf_gemm_scaled(stream_ptr(), dtype_code(dtype), dtype_code(c.dtype), la, lb, m, n, k, a.data_ptr(), lda,
                             b.data_ptr(), ldb, c.data_ptr(), ldc, alpha.data_ptr(),
                             ws.data_ptr() if ws is not None else None, ws_bytes))


def gemm_scaled(a, la, m, k, lda, b, lb, n, ldb, alpha, out):
    """``out (m, n) = alpha * A . B`` through tf_gemm_scaled; ``alpha``: a one-element float32 tensor on
    the GPU; operands given with their layouts as in the C header.  ``out``: float32 or the operand dtype."""
    if alpha.dtype != torch.float32 or alpha.numel() != 1:
        raise TypeError("alpha must be a one-element float32 tensor")
    require_cuda(a, b, alpha, out)
    _gemm_scaled(a.dtype, la, lb, m, n, k, a, lda, b, ldb, out, out.stride(0), alpha)
    return out


def mm(a, b, fuse_relu=False, mask_act=None):
    return gemm(a, b, None, fuse_relu, mask_act)


def mm_dw(x, grad, out_dtype=None, chunks=1):
    """``sum_b x[b]^T @ grad[b]`` -> (in, out): reference ``bmm`` of the
    transposed view (kernels/gemm.py:161-200) followed by ``torch.sum`` over the
    batch (linear.py:24-25), as ONE contraction over all B*S tokens.
    ``out_dtype=torch.float32`` stores the fp32 accumulators unrounded (gradient
    of an fp32 master weight).  ``chunks=c > 1`` returns (c, in, out/c): the
    column blocks of the product as c separate contiguous matrices (the gradients
    of c weights whose outputs were computed side by side in one product)."""
    if x.shape[:-1] != grad.shape[:-1]:
        raise ValueError("Leading dimensions of the two operands do not match")
    if x.dtype != grad.dtype:
        raise TypeError("operands must share one 16-bit dtype")
    require_cuda(x, grad)
    x2, t, kin = _rows2d(x)
    g2, _, nout = _rows2d(grad)
    if chunks > 1:
        if nout % chunks or (nout // chunks) % 8:
            raise ValueError("column blocks must be equal and multiples of 8 wide")
        each = nout // chunks
        out = torch.empty((chunks, kin, each), dtype=out_dtype or x.dtype, device=x.device)
        _gemm(x.dtype, KMINOR, KMINOR, kin, nout, t, x2, kin, g2, nout, out, each, None, False,
              chunk_n=each, chunk_stride=kin * each)
        return out
    out = torch.empty((kin, nout), dtype=out_dtype or x.dtype, device=x.device)
    _gemm(x.dtype, KMINOR, KMINOR, kin, nout, t, x2, kin, g2, nout, out, nout, None, False)
    return out


def mm_dw_group(pairs, out_dtype=None, chunks=None):
    """``[mm_dw(x, g) for x, g in pairs]`` (up to sixteen weight gradients that are available
    at the same time) through ONE launch where the kernel's preconditions allow: products
    whose outputs have few tiles then share the GPU instead of each splitting its contraction
    into many slices.  ``chunks[i] > 1`` as in mm_dw."""
    chunks = list(chunks) if chunks is not None else [1] * len(pairs)
    if not 1 <= len(pairs) <= 16 or len(chunks) != len(pairs):
        raise ValueError("mm_dw_group takes 1..16 (x, grad) pairs")
    probs = (_lib.GemmProblem * len(pairs))()
    outs, keep = [], []
    dt = pairs[0][0].dtype
    for i, ((x, grad), ch) in enumerate(zip(pairs, chunks)):
        if x.shape[:-1] != grad.shape[:-1]:
            raise ValueError("Leading dimensions of the two operands do not match")
        if x.dtype != grad.dtype or x.dtype != dt:
            raise TypeError("operands must share one 16-bit dtype")
        require_cuda(x, grad)
        x2, t, kin = _rows2d(x)
        g2, _, nout = _rows2d(grad)
        keep += [x2, g2]
        if ch > 1:
            if nout % ch or (nout // ch) % 8:
                raise ValueError("column blocks must be equal and multiples of 8 wide")
            each = nout // ch
            out = torch.empty((ch, kin, each), dtype=out_dtype or dt, device=x.device)
            ldc, cn, cs = each, each, kin * each
        else:
            out = torch.empty((kin, nout), dtype=out_dtype or dt, device=x.device)
            ldc, cn, cs = nout, 0, 0
        outs.append(out)
        probs[i] = _lib.GemmProblem(kin, nout, t, x2.data_ptr(), kin, g2.data_ptr(), nout, out.data_ptr(), ldc, cn, cs)
    _gemm_group(dt, outs[0].dtype, KMINOR, KMINOR, probs, outs[0].device)
    return outs


def cast_pack(weights, dtype):
    """The (in, out_j) matrices ``weights`` (all one shape and dtype: float32 or ``dtype``)
    converted to the 16-bit ``dtype`` side by side in one (in, sum out_j) matrix, one launch."""
    w0 = weights[0]
    if not 1 <= len(weights) <= 4 or any(w.shape != w0.shape or w.dtype != w0.dtype or w.ndim != 2 for w in weights):
        raise ValueError("cast_pack takes 1..4 matrices of one shape and dtype")
    if dtype not in (torch.float16, torch.bfloat16) or w0.dtype not in (torch.float32, dtype):
        raise TypeError("cast_pack converts float32 (or already 16-bit) matrices to float16 / bfloat16")
    require_cuda(*weights)
    weights = [w if w.is_contiguous() else w.contiguous() for w in weights]
    rows, cols = w0.shape
    out = torch.empty((rows, len(weights) * cols), dtype=dtype, device=w0.device)
    ptrs = (ctypes.c_void_p * len(weights))(*[w.data_ptr() for w in weights])
    check(load().tf_cast_pack(stream_ptr(), dtype_code(w0.dtype), dtype_code(dtype), len(weights), rows, cols, ptrs,
                              cols, out.data_ptr(), len(weights) * cols))
    return out


def embedding_fwd(ids, tok_w, pos_w, out_dtype):
    """(B, S) int64 ids -> (B, S, d): ``tok_w[ids] + pos_w[arange(S)]`` (``pos_w`` may be None),
    added in fp32 and rounded once to ``out_dtype`` (reference transformer.py:311-323)."""
    require_cuda(ids, tok_w)
    if ids.ndim != 2 or ids.dtype != torch.int64 or tok_w.ndim != 2:
        raise ValueError("embedding takes (B, S) int64 ids and a (V, d) table")
    if pos_w is not None and (pos_w.ndim != 2 or pos_w.shape[1] != tok_w.shape[1] or pos_w.dtype != tok_w.dtype):
        raise ValueError("position table must be (P, d) of the token table's dtype")
    ids = ids.contiguous()
    tok_w = tok_w if tok_w.stride(-1) == 1 else tok_w.contiguous()
    if pos_w is not None and pos_w.stride(-1) != 1:
        pos_w = pos_w.contiguous()
    b, s = ids.shape
    v, d = tok_w.shape
    out = torch.empty((b, s, d), dtype=out_dtype, device=tok_w.device)
    check(load().tf_embedding_fwd(stream_ptr(), dtype_code(tok_w.dtype), dtype_code(out_dtype), b * s, s, d, v,
                                  0 if pos_w is None else pos_w.shape[0], ids.data_ptr(), tok_w.data_ptr(),
                                  tok_w.stride(0), None if pos_w is None else pos_w.data_ptr(),
                                  0 if pos_w is None else pos_w.stride(0), out.data_ptr(), d))
    return out


def embedding_bwd(grad_out, ids, tok_shape, pos_shape, param_dtype):
    """Gradients of embedding_fwd's tables: (V, d) scatter-add by token id and, when
    ``pos_shape`` is given, (P, d) sum over sequences; fp32 accumulation in position order."""
    require_cuda(grad_out, ids)
    ids = ids.contiguous()
    b, s = ids.shape
    v, d = tok_shape
    g = grad_out.reshape(b * s, d)
    if g.stride(-1) != 1:
        g = g.contiguous()
    lib = load()
    d_tok = torch.empty((v, d), dtype=param_dtype, device=g.device)
    d_pos = None if pos_shape is None else torch.empty(tuple(pos_shape), dtype=param_dtype, device=g.device)
    nbytes = lib.tf_embedding_bwd_workspace_bytes(b * s)
    ws = torch.empty(nbytes, dtype=torch.uint8, device=g.device)
    check(lib.tf_embedding_bwd(stream_ptr(), dtype_code(g.dtype), dtype_code(param_dtype), b * s, s, d, v,
                               0 if d_pos is None else d_pos.shape[0], ids.data_ptr(), g.data_ptr(), g.stride(0),
                               d_tok.data_ptr(), d, None if d_pos is None else d_pos.data_ptr(), d, ws.data_ptr(), nbytes))
    return d_tok, d_pos


def unbroadcast_leading(x, out_dtype=None):
    """Sum over every dimension but the last, fp32 accumulation -> (cols,)
    (reference kernels/reductions.py:97-122).  ``out_dtype=torch.float32`` stores the fp32 sums
    unrounded (gradient of an fp32 master bias)."""
    require_cuda(x)
    lib = load()
    x2, rows, cols = _rows2d(x)
    out = torch.empty((cols,), dtype=out_dtype or x.dtype, device=x.device)
    pb = lib.tf_colsum_partial_bytes(rows, cols)
    part = torch.empty(pb, dtype=torch.uint8, device=x.device)
    check(lib.tf_colsum(stream_ptr(), dtype_code(x.dtype), dtype_code(out.dtype), rows, cols, x2.data_ptr(), cols,
                        out.data_ptr(), part.data_ptr(), pb))
    return out


def mask_grad(grad, out_act):
    """``where(out_act > 0, grad, 0)`` into a NEW tensor (the reference,
    kernels/activation.py:27-44, overwrites ``grad``)."""
    require_cuda(grad, out_act)
    if grad.shape != out_act.shape or grad.dtype != out_act.dtype:
        raise ValueError("grad and activation must agree in shape and dtype")
    g2, rows, cols = _rows2d(grad)
    a2, _, _ = _rows2d(out_act)
    out = torch.empty(grad.shape, dtype=grad.dtype, device=grad.device)
    check(load().tf_relu_mask(stream_ptr(), dtype_code(grad.dtype), rows, cols, g2.data_ptr(), cols, a2.data_ptr(),
                              cols, out.data_ptr(), cols))
    return out


# --------------------------------------------------------------------------- attention
def _attn_layout(q, *others):
    """All tensors must share q's strides, unit stride along hd and 16-byte
    aligned rows; otherwise everything is copied to contiguous (B, nh, S, hd)."""
    ok = q.stride(-1) == 1 and all(s % 8 == 0 for s in q.stride()[:-1]) and q.data_ptr() % 16 == 0
    ok = ok and all(t.stride() == q.stride() and t.data_ptr() % 16 == 0 for t in others)
    if ok:
        return (q,) + tuple(others)
    return tuple(t.contiguous() for t in (q,) + tuple(others))


def _check_attn(q, k, v, bias):
    if q.ndim != 4 or q.shape != k.shape or q.shape != v.shape:
        raise ValueError("q, k, v must be (B, nh, S, hd) tensors of one shape")
    b, nh, s, hd = q.shape
    if hd not in (32, 64, 128):
        raise ValueError("Only head_dims of [32,64,128] are supported.")
    # kernels/attention.py:177-183 of the reference: 64-row blocks, 32-row blocks at head_dim 128
    if s % (32 if hd == 128 else 64) != 0:
        raise ValueError("Sequence length must be a multiple of the block size (64; 32 at head_dim 128)")
    if not (q.dtype == k.dtype == v.dtype) or q.dtype not in (torch.float16, torch.bfloat16):
        raise TypeError("q, k, v must share one 16-bit dtype")
    require_cuda(q, k, v, bias)
    if bias is not None and bias.ndim == 1:
        # ALiBi in closed form: the nh slopes as the reference rounds them (fp16, transformer.py:68)
        if bias.shape[0] != nh or bias.dtype != torch.float16:
            raise ValueError("ALiBi slopes must be a (nh,) float16 vector")
    elif bias is not None:
        # kernels/biased_attention.py:199-207 of the reference
        if bias.ndim != 3 or bias.shape[0] != nh:
            raise ValueError("attention bias must be (nh, S', S')")
        if bias.shape[1] != bias.shape[2] or bias.shape[1] < s:
            raise ValueError("attention bias must be square and cover the sequence")
        if bias.dtype != q.dtype:
            raise TypeError("attention bias must have the dtype of q")


def _bias_args(bias):
    if bias is None:
        return None, None, 0, 0
    if bias.stride(-1) != 1 or bias.stride(0) % 8 or bias.stride(1) % 8 or bias.data_ptr() % 16:
        # rows of whole 16-byte chunks: copy into storage whose row pitch is padded to 8 elements
        nh, rows, cols = bias.shape
        padded = torch.empty((nh, rows, (cols + 7) // 8 * 8), dtype=bias.dtype, device=bias.device)
        padded[..., :cols].copy_(bias)
        bias = padded[..., :cols]
    return bias, bias.data_ptr(), bias.stride(0), bias.stride(1)


def _strided_ok(t):
    return t.stride(-1) == 1 and all(st % 8 == 0 for st in t.stride()[:-1]) and t.data_ptr() % 16 == 0


def flash_wrapper_fwd(q, k, v, bias=None, out=None):
    """Causal attention forward -> (out, lse).  ``bias``: None, a dense (nh, S', S') matrix, or
    the (nh,) float16 ALiBi slopes (the bias -slope_h * (i - j) is then computed in the kernel
    with the roundings of the reference's dense matrix).  ``out`` has q's strides unless a
    (B, nh, S, hd) view is passed in; ``lse`` is (B, nh, S) fp32 in the log2
    domain (the reference keeps fp16 m and l, kernels/attention.py:171-217 and
    kernels/biased_attention.py:188-245).  S % 32 == 0 for every head_dim (the reference: S % 64 == 0,
    S % 32 == 0 at head_dim 128, kernels/attention.py:177-183)."""
    _check_attn(q, k, v, bias)
    b, nh, s, hd = q.shape
    if out is not None and (out.shape != q.shape or out.dtype != q.dtype or not _strided_ok(out)):
        raise ValueError("attention output buffer must match q in shape and dtype, with aligned strides")
    q, k, v = _attn_layout(q, k, v)
    if out is None:
        out = torch.empty_strided(q.shape, q.stride(), dtype=q.dtype, device=q.device)
    lse = torch.empty((b, nh, s), dtype=torch.float32, device=q.device)
    if bias is not None and bias.ndim == 1:
        slopes = bias.contiguous()
        check(load().tf_attn_alibi_fwd(stream_ptr(), dtype_code(q.dtype), b, nh, s, hd, q.data_ptr(), k.data_ptr(),
                                       v.data_ptr(), out.data_ptr(), q.stride(0), q.stride(1), q.stride(2),
                                       out.stride(0), out.stride(1), out.stride(2), lse.data_ptr(), slopes.data_ptr(),
                                       1.0 / math.sqrt(hd)))
        return out, lse
    bias, bptr, bsh, bsr = _bias_args(bias)
    check(load().tf_attn_fwd(stream_ptr(), dtype_code(q.dtype), b, nh, s, hd, q.data_ptr(), k.data_ptr(),
                             v.data_ptr(), out.data_ptr(), q.stride(0), q.stride(1), q.stride(2), out.stride(0),
                             out.stride(1), out.stride(2), lse.data_ptr(), bptr, bsh, bsr, 1.0 / math.sqrt(hd)))
    return out, lse


def flash_wrapper_bwd(grad_out, out, q, k, v, lse, bias=None, grads=None):
    """Causal attention backward -> (dq, dk, dv), each with q's strides (or written
    into the three (B, nh, S, hd) views given as ``grads``); reference
    kernels/attention.py:550-607, kernels/biased_attention.py:598-660."""
    _check_attn(q, k, v, bias)
    q, k, v = _attn_layout(q, k, v)
    if not _strided_ok(out):
        out = out.contiguous()
    if grad_out.stride() != out.stride() or grad_out.data_ptr() % 16:
        g = torch.empty_strided(out.shape, out.stride(), dtype=out.dtype, device=out.device)
        g.copy_(grad_out)
        grad_out = g
    b, nh, s, hd = q.shape
    if grads is None:
        grads = tuple(torch.empty_strided(q.shape, q.stride(), dtype=q.dtype, device=q.device) for _ in range(3))
    dq, dk, dv = grads
    if any(t.stride() != q.stride() or t.data_ptr() % 16 for t in grads):
        raise ValueError("attention gradient buffers must share q's strides")
    delta = torch.empty((b, nh, s), dtype=torch.float32, device=q.device)
    if bias is not None and bias.ndim == 1:
        slopes = bias.contiguous()
        check(load().tf_attn_alibi_bwd(stream_ptr(), dtype_code(q.dtype), b, nh, s, hd, q.data_ptr(), k.data_ptr(),
                                       v.data_ptr(), out.data_ptr(), grad_out.data_ptr(), dq.data_ptr(), dk.data_ptr(),
                                       dv.data_ptr(), q.stride(0), q.stride(1), q.stride(2), out.stride(0),
                                       out.stride(1), out.stride(2), lse.data_ptr(), delta.data_ptr(),
                                       slopes.data_ptr(), 1.0 / math.sqrt(hd)))
        return dq, dk, dv
    bias, bptr, bsh, bsr = _bias_args(bias)
    check(load().tf_attn_bwd(stream_ptr(), dtype_code(q.dtype), b, nh, s, hd, q.data_ptr(), k.data_ptr(),
                             v.data_ptr(), out.data_ptr(), grad_out.data_ptr(), dq.data_ptr(), dk.data_ptr(),
                             dv.data_ptr(), q.stride(0), q.stride(1), q.stride(2), out.stride(0), out.stride(1),
                             out.stride(2), lse.data_ptr(), delta.data_ptr(), bptr, bsh, bsr,
                             1.0 / math.sqrt(hd)))
    return dq, dk, dv


def flash_wrapper_fwd_attn_bias(q, k, v, attn_bias):
    return flash_wrapper_fwd(q, k, v, attn_bias)


def flash_wrapper_bwd_attn_bias(grad_out, out, q, k, v, lse, attn_bias):
    return flash_wrapper_bwd(grad_out, out, q, k, v, lse, attn_bias)


# --------------------------------------------------------------------------- layernorm
def _check_ln(x, d):
    # kernels/layernorm.py:68-71 of the reference: 3-D, 16-bit, on the GPU
    if x.ndim != 3:
        raise ValueError("LayerNorm input must be 3-dimensional (B, S, d)")
    if x.dtype not in (torch.float16, torch.bfloat16):
        raise TypeError("LayerNorm input must be float16 or bfloat16")
    if x.shape[-1] != d:
        raise ValueError("LayerNorm parameters do not match the last dimension")
    require_cuda(x)


def layernorm_fwd(x, alpha, beta, eps):
    """-> (y, mean, rstd); reference kernels/layernorm.py:64-87."""
    _check_ln(x, alpha.shape[0])
    if alpha.dtype != beta.dtype or alpha.dtype not in (x.dtype, torch.float32):
        raise TypeError("LayerNorm parameters must have the input's dtype or be float32")
    require_cuda(alpha, beta)
    x2, rows, d = _rows2d(x)
    y = torch.empty(x.shape, dtype=x.dtype, device=x.device)
    mean = torch.empty((rows,), dtype=torch.float32, device=x.device)
    rstd = torch.empty((rows,), dtype=torch.float32, device=x.device)
    check(load().tf_layernorm_fwd(stream_ptr(), dtype_code(x.dtype), dtype_code(alpha.dtype), rows, d, x2.data_ptr(), d,
                                  alpha.contiguous().data_ptr(), beta.contiguous().data_ptr(), float(eps),
                                  y.data_ptr(), d, mean.data_ptr(), rstd.data_ptr()))
    return y, mean, rstd


def layernorm_bwd(grad_out, x, alpha, mean, rstd, leave_partials=False):
    """-> (dx, dalpha, dbeta); reference dx_layernorm (kernels/layernorm.py:140-162)
    and layernorm_da_db (kernels/layernorm.py:226-259) in one pass.  With ``leave_partials``
    -> (dx, partial): the column sums of the row blocks as they are, for layernorm_param_grads."""
    lib = load()
    x2, rows, d = _rows2d(x)
    g2, _, _ = _rows2d(grad_out)
    dx = torch.empty(x.shape, dtype=x.dtype, device=x.device)
    da = db = None
    if not leave_partials:
        da = torch.empty((d,), dtype=alpha.dtype, device=x.device)
        db = torch.empty((d,), dtype=alpha.dtype, device=x.device)
    pb = lib.tf_layernorm_bwd_partial_bytes(rows, d)
    part = torch.empty(pb, dtype=torch.uint8, device=x.device)
    check(lib.tf_layernorm_bwd(stream_ptr(), dtype_code(x.dtype), dtype_code(alpha.dtype), rows, d, g2.data_ptr(), d,
                               x2.data_ptr(), d,
                               alpha.contiguous().data_ptr(), mean.data_ptr(), rstd.data_ptr(), dx.data_ptr(), d,
                               None if da is None else da.data_ptr(), None if db is None else db.data_ptr(),
                               part.data_ptr(), pb))
    if leave_partials:
        return dx, (part, lib.tf_layernorm_bwd_parts(rows))
    return dx, da, db


def layernorm_param_grads(partials, d, dtype):
    """``partials``: (buffer, parts) pairs that layernorm_bwd / add_layernorm_bwd left behind.  -> a
    (len(partials), 2, d) tensor of ``dtype``: [i, 0] = dgamma and [i, 1] = dbeta of the i-th LayerNorm,
    all of them summed by one launch (per 64)."""
    lib = load()
    n = len(partials)
    device = partials[0][0].device
    out = torch.empty((n, 2, d), dtype=dtype, device=device)
    items = (_lib.LnParamGrads * n)()
    step = 2 * d * out.element_size()
    for i, (buf, parts) in enumerate(partials):
        require_cuda(buf)
        items[i] = _lib.LnParamGrads(buf.data_ptr(), parts, out.data_ptr() + i * step, out.data_ptr() + i * step + step // 2)
    check(lib.tf_layernorm_param_grads(stream_ptr(), dtype_code(dtype), d, n, items))
    return out


def add_layernorm_fwd(x, res, alpha, beta, eps):
    """-> (sum, y, mean, rstd) with sum = x + res and y = layernorm(sum), one kernel for the
    residual addition (reference transformer.py:245-246, :250) and the LayerNorm after it."""
    _check_ln(x, alpha.shape[0])
    if res.shape != x.shape or res.dtype != x.dtype:
        raise ValueError("the two summands must have the same shape and dtype")
    if alpha.dtype != beta.dtype or alpha.dtype not in (x.dtype, torch.float32):
        raise TypeError("LayerNorm parameters must have the input's dtype or be float32")
    require_cuda(res, alpha, beta)
    x2, rows, d = _rows2d(x)
    r2, _, _ = _rows2d(res)
    total = torch.empty(x.shape, dtype=x.dtype, device=x.device)
    y = torch.empty(x.shape, dtype=x.dtype, device=x.device)
    mean = torch.empty((rows,), dtype=torch.float32, device=x.device)
    rstd = torch.empty((rows,), dtype=torch.float32, device=x.device)
    check(load().tf_add_layernorm_fwd(stream_ptr(), dtype_code(x.dtype), dtype_code(alpha.dtype), rows, d,
                                      x2.data_ptr(), d, r2.data_ptr(), d, total.data_ptr(), d,
                                      alpha.contiguous().data_ptr(), beta.contiguous().data_ptr(), float(eps),
                                      y.data_ptr(), d, mean.data_ptr(), rstd.data_ptr()))
    return total, y, mean, rstd


def add_layernorm_bwd(grad_out, grad_sum, total, alpha, mean, rstd, leave_partials=False):
    """-> (dx, dalpha, dbeta): dx = layernorm backward of grad_out at the saved sum, plus
    grad_sum (the gradient of the sum arriving along the residual stream).  ``leave_partials`` as in
    layernorm_bwd."""
    lib = load()
    x2, rows, d = _rows2d(total)
    g2, _, _ = _rows2d(grad_out)
    s2, _, _ = _rows2d(grad_sum)
    dx = torch.empty(total.shape, dtype=total.dtype, device=total.device)
    da = db = None
    if not leave_partials:
        da = torch.empty((d,), dtype=alpha.dtype, device=total.device)
        db = torch.empty((d,), dtype=alpha.dtype, device=total.device)
    pb = lib.tf_layernorm_bwd_partial_bytes(rows, d)
    part = torch.empty(pb, dtype=torch.uint8, device=total.device)
    check(lib.tf_add_layernorm_bwd(stream_ptr(), dtype_code(total.dtype), dtype_code(alpha.dtype), rows, d,
                                   g2.data_ptr(), d, s2.data_ptr(), d, x2.data_ptr(), d,
                                   alpha.contiguous().data_ptr(), mean.data_ptr(), rstd.data_ptr(), dx.data_ptr(), d,
                                   None if da is None else da.data_ptr(), None if db is None else db.data_ptr(),
                                   part.data_ptr(), pb))
    if leave_partials:
        return dx, (part, lib.tf_layernorm_bwd_parts(rows))
    return dx, da, db


# --------------------------------------------------------------------------- softmax
def softmax_fwd(x):
    """Row softmax over the last dim (reference kernels/softmax.py:37-54)."""
    require_cuda(x)
    if x.ndim != 3:
        raise ValueError("Softmax input must be 3-dimensional")
    x2, rows, cols = _rows2d(x)
    y = torch.empty(x.shape, dtype=x.dtype, device=x.device)
    check(load().tf_softmax_fwd(stream_ptr(), dtype_code(x.dtype), rows, cols, x2.data_ptr(), cols, y.data_ptr(),
                                cols))
    return y


def softmax_bwd(grad_out, saved_out):
    """``y * (dy - sum(y*dy))`` into a new tensor (reference kernels/softmax.py:95-111
    writes over grad_out)."""
    require_cuda(grad_out, saved_out)
    g2, rows, cols = _rows2d(grad_out)
    y2, _, _ = _rows2d(saved_out)
    dx = torch.empty(saved_out.shape, dtype=saved_out.dtype, device=saved_out.device)
    check(load().tf_softmax_bwd(stream_ptr(), dtype_code(saved_out.dtype), rows, cols, g2.data_ptr(), cols,
                                y2.data_ptr(), cols, dx.data_ptr(), cols))
    return dx


# --------------------------------------------------------------------------- cross entropy
def _check_ce(logits, labels):
    if labels.dtype != torch.int64:
        raise TypeError("labels must be int64")
    if logits.dtype not in (torch.float16, torch.bfloat16):
        raise TypeError("logits must be float16 or bfloat16")
    require_cuda(logits, labels)


def cross_entropy_fwd(logits, labels):
    """-> (per-row loss in logits' dtype, lse fp32, logits, labels); reference
    kernels/crossentropy.py:47-75 (which keeps the full (N, V) matrix instead)."""
    if logits.ndim != 2 or labels.ndim != 1 or labels.shape[0] != logits.shape[0]:
        raise ValueError("cross entropy takes (N, V) logits and (N,) labels")
    _check_ce(logits, labels)
    if logits.stride(-1) != 1:
        logits = logits.contiguous()
    labels = labels.contiguous()
    n, v = logits.shape
    loss = torch.empty((n,), dtype=logits.dtype, device=logits.device)
    lse = torch.empty((n,), dtype=torch.float32, device=logits.device)
    check(load().tf_cross_entropy_fwd(stream_ptr(), dtype_code(logits.dtype), n, v, logits.data_ptr(),
                                      logits.stride(0), 0, 0, labels.data_ptr(), loss.data_ptr(), lse.data_ptr()))
    return loss, lse, logits, labels


def cross_entropy_bwd(grad_out, logits, labels, lse):
    """``(softmax(logits) - onehot) * grad_out[:, None]`` (reference
    kernels/crossentropy.py:110-127 and the multiply at crossentropy.py:24)."""
    n, v = logits.shape
    if grad_out.dtype != logits.dtype:
        grad_out = grad_out.to(logits.dtype)
    gstride = grad_out.stride(0) if grad_out.ndim == 1 else 0
    dlogits = torch.empty((n, v), dtype=logits.dtype, device=logits.device)
    check(load().tf_cross_entropy_bwd(stream_ptr(), dtype_code(logits.dtype), n, v, logits.data_ptr(),
                                      logits.stride(0), 0, 0, labels.data_ptr(), lse.data_ptr(),
                                      grad_out.data_ptr(), gstride, dlogits.data_ptr(), v, 0))
    return dlogits


def shifted_cross_entropy_fwd(logits, labels):
    """Next-token loss of a (B, S, V) logits tensor against (B, S) labels:
    row (b, s), s < S-1, is scored against labels[b, s+1], reading the logits in
    place (the reference copies logits[..., :-1, :] first, transformer.py:333-334).
    -> (loss (B*(S-1),), lse, logits, shifted labels)"""
    if logits.ndim != 3 or labels.shape != logits.shape[:2]:
        raise ValueError("shifted cross entropy takes (B, S, V) logits and (B, S) labels")
    _check_ce(logits, labels)
    if not logits.is_contiguous():
        logits = logits.contiguous()
    b, s, v = logits.shape
    shift_labels = labels[:, 1:].contiguous().view(-1)
    n = b * (s - 1)
    loss = torch.empty((n,), dtype=logits.dtype, device=logits.device)
    lse = torch.empty((n,), dtype=torch.float32, device=logits.device)
    check(load().tf_cross_entropy_fwd(stream_ptr(), dtype_code(logits.dtype), n, v, logits.data_ptr(), v, s - 1,
                                      s * v, shift_labels.data_ptr(), loss.data_ptr(), lse.data_ptr()))
    return loss, lse, logits, shift_labels


def shifted_cross_entropy_fwd_grad(logits, labels, grad_scale):
    """shifted_cross_entropy_fwd that also returns ``(softmax - onehot) * grad_scale`` for every row,
    as a (B, S, V) tensor whose last position per sequence is zero, written by the same kernel pass
    (reference kernels/crossentropy.py:47-75 and :110-127 in one).  ``grad_scale`` must be exactly
    representable in the logits' dtype (a power of two).
    -> (loss (B*(S-1),), lse, dlogits)"""
    if logits.ndim != 3 or labels.shape != logits.shape[:2]:
        raise ValueError("shifted cross entropy takes (B, S, V) logits and (B, S) labels")
    _check_ce(logits, labels)
    if not logits.is_contiguous():
        logits = logits.contiguous()
    b, s, v = logits.shape
    shift_labels = labels[:, 1:].contiguous().view(-1)
    n = b * (s - 1)
    loss = torch.empty((n,), dtype=logits.dtype, device=logits.device)
    lse = torch.empty((n,), dtype=torch.float32, device=logits.device)
    dlogits = torch.empty((b, s, v), dtype=logits.dtype, device=logits.device)
    dlogits[:, -1].zero_()
    scale_dev = torch.full((1,), grad_scale, dtype=logits.dtype, device=logits.device)
    check(load().tf_cross_entropy_fwd_grad(stream_ptr(), dtype_code(logits.dtype), n, v, logits.data_ptr(), v, s - 1,
                                           s * v, shift_labels.data_ptr(), loss.data_ptr(), lse.data_ptr(),
                                           dlogits.data_ptr(), v, s * v, float(grad_scale), scale_dev.data_ptr()))
    return loss, lse, dlogits


def shifted_cross_entropy_bwd(grad_out, logits, shift_labels, lse):
    """Gradient with respect to the full (B, S, V) logits: rows s < S-1 as
    cross_entropy_bwd, the last position of every sequence zero."""
    b, s, v = logits.shape
    n = b * (s - 1)
    if grad_out.dtype != logits.dtype:
        grad_out = grad_out.to(logits.dtype)
    gstride = grad_out.stride(0) if grad_out.ndim == 1 else 0
    dlogits = torch.empty((b, s, v), dtype=logits.dtype, device=logits.device)
    dlogits[:, -1].zero_()
    check(load().tf_cross_entropy_bwd(stream_ptr(), dtype_code(logits.dtype), n, v, logits.data_ptr(), v, s - 1,
                                      s * v, shift_labels.data_ptr(), lse.data_ptr(), grad_out.data_ptr(), gstride,
                                      dlogits.data_ptr(), v, s * v))
    return dlogits
