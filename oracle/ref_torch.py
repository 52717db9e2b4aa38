"""fp32 PyTorch restatement of fattorib/tritonformer's math -- TEST
INFRASTRUCTURE ONLY (see oracle/__init__.py).

Per-operator functions follow the oracle one-liners of the reference's own
tests, evaluated in fp32 instead of fp16; ``RefTransformer`` restates the
reference's ``transformer.py`` with the same parameter names, so a state dict
can be moved between it and ``tritonformer_amd.transformer.Transformer``.
Gradients come from autograd of these forward expressions; closed-form
backward formulas are also given (``*_bwd``) and are cross-checked against
autograd and against the brute-force C restatement (oracle/ref_ops.c) in
tests/test_oracle.py.

Pinning status (which independent check fixes each function):
  linear / linear_bwd       brute-force loops in ref_ops.c; identity / permutation weights
  layer_norm / _bwd         ref_ops.c loops; F.layer_norm; constant row -> beta; sum(dx)=0
  softmax / _bwd            ref_ops.c loops; rows sum to 1; shift invariance
  cross_entropy / _bwd      ref_ops.c loops; uniform logits -> ln V; F.cross_entropy
  causal_attention          ref_ops.c loops (fwd + explicit bwd); SDPA(is_causal); row 0 = v[0];
                            zero bias == no bias
  get_slopes / alibi mask   closed forms for n = 8, 16, 24
  embedding / _bwd          element loops on a tiny case (tests/test_oracle.py); F.embedding and
                            its autograd; one-hot matrix product
  adamw_step                torch.optim.AdamW on the CPU over several steps; closed form of the
                            first step (p - lr*wd*p - lr*sign(g) up to eps)
  RefTransformer            zero-initialised LM head -> loss = ln(vocab) exactly and zero grads
                            upstream; parameter-name list; committed config-1 fixture
No function of this oracle is "parity unpinned".
"""
import math
from dataclasses import dataclass
from typing import List, Optional

import torch
import torch.nn as nn
import torch.nn.functional as F


# --------------------------------------------------------------------------- operators
def linear(x, w, b=None, relu=False):
    """reference tritonformer/test_linear.py:19-25 (``torch.matmul(x, W) + bias``);
    ReLU epilogue as kernels/gemm.py:355-356, 566-567.  W is (in, out)."""
    y = torch.matmul(x.float(), w.float())
    if b is not None:
        y = y + b.float()
    return torch.relu(y) if relu else y


def linear_bwd(x, w, dy, act=None, with_bias=False):
    """dX = dY W^T, dW = sum_b X_b^T dY_b, db = sum_{b,s} dY
    (reference linear.py:21-25, 39-44); when ``act`` is given dY is first masked
    by act > 0 (kernels/activation.py:22, linear.py:62, 87)."""
    x, w, dy = x.float(), w.float(), dy.float()
    if act is not None:
        dy = torch.where(act.float() > 0, dy, torch.zeros_like(dy))
    dx = dy @ w.t()
    dw = x.reshape(-1, x.shape[-1]).t() @ dy.reshape(-1, dy.shape[-1])
    db = dy.reshape(-1, dy.shape[-1]).sum(0) if with_bias else None
    return dx, dw, db


def layer_norm(x, gamma, beta, eps=1e-5):
    """reference tritonformer/test_layernorm.py:19-23 (``F.layer_norm``); biased
    variance and rstd = 1/sqrt(var + eps) as kernels/layernorm.py:46-54."""
    x = x.float()
    mean = x.mean(-1, keepdim=True)
    var = ((x - mean) ** 2).mean(-1, keepdim=True)
    return (x - mean) / torch.sqrt(var + eps) * gamma.float() + beta.float()


def layer_norm_bwd(x, gamma, dy, eps=1e-5):
    """Closed forms of kernels/layernorm.py:124-133 (dx) and :200-218 (dgamma, dbeta)."""
    x, gamma, dy = x.float(), gamma.float(), dy.float()
    mean = x.mean(-1, keepdim=True)
    rstd = 1.0 / torch.sqrt(((x - mean) ** 2).mean(-1, keepdim=True) + eps)
    xh = (x - mean) * rstd
    g = dy * gamma
    dx = (g - xh * (g * xh).mean(-1, keepdim=True) - g.mean(-1, keepdim=True)) * rstd
    d = x.shape[-1]
    return dx, (dy * xh).reshape(-1, d).sum(0), dy.reshape(-1, d).sum(0)


def softmax(x):
    """reference tritonformer/test_softmax.py:18-20."""
    return F.softmax(x.float(), dim=-1)


def softmax_bwd(y, dy):
    """kernels/softmax.py:80-92: dx = y * (dy - sum(y * dy))."""
    y, dy = y.float(), dy.float()
    return y * (dy - (y * dy).sum(-1, keepdim=True))


def cross_entropy(logits, labels):
    """Per-row loss, the contract transformer.py:336-343 relies on (the wrapper
    returns (N,), the caller takes .mean()); kernels/crossentropy.py:30-44."""
    return F.cross_entropy(logits.float(), labels, reduction="none")


def cross_entropy_bwd(logits, labels, gout):
    """kernels/crossentropy.py:93-107 (softmax - onehot) times crossentropy.py:24."""
    p = F.softmax(logits.float(), dim=-1)
    p[torch.arange(p.shape[0]), labels] -= 1.0
    return p * gout.float()[:, None]


def causal_attention(q, k, v, bias=None):
    """reference tritonformer/test_attention.py:43-62 and
    test_biased_attention.py:79-102, in fp32 throughout: softmax over
    q k^T / sqrt(hd) (+ bias[h, :S, :S]) with keys above the diagonal masked."""
    q, k, v = q.float(), k.float(), v.float()
    s = q.shape[-2]
    scores = torch.matmul(q, k.transpose(-1, -2)) / math.sqrt(q.shape[-1])
    if bias is not None:
        scores = scores + bias[..., :s, :s].float()
    keep = torch.tril(torch.ones(s, s, dtype=torch.bool, device=q.device))
    scores = scores.masked_fill(~keep, float("-inf"))
    return torch.matmul(F.softmax(scores, dim=-1), v)


# --------------------------------------------------------------------------- ALiBi
def embedding(ids, tok_w, pos_w=None):
    """tok_w[ids] + pos_w[arange(S)] for (B, S) ids: reference transformer.py:311-323."""
    out = tok_w.float()[ids]
    if pos_w is not None:
        out = out + pos_w.float()[torch.arange(ids.shape[1])][None]
    return out


def embedding_bwd(ids, g, vocab: int, positions: Optional[int] = None):
    """Gradients of ``embedding``: rows of g (B, S, d) added up by token id -> (vocab, d), and
    by position -> (positions, d) (rows >= S stay zero)."""
    b, s = ids.shape
    g = g.float()
    d_tok = torch.zeros((vocab, g.shape[-1]), dtype=torch.float32)
    d_tok.index_add_(0, ids.reshape(-1), g.reshape(b * s, -1))
    if positions is None:
        return d_tok, None
    d_pos = torch.zeros((positions, g.shape[-1]), dtype=torch.float32)
    d_pos[:s] = g.sum(0)
    return d_tok, d_pos


def adamw_step(p, g, m, v, step: int, lr=1e-3, betas=(0.9, 0.999), eps=1e-8, weight_decay=1e-2):
    """One AdamW step (decoupled weight decay, no amsgrad) on fp32 tensors, out of place:
    returns (p, m, v) after the step; ``step`` counts from 1."""
    b1, b2 = betas
    p = p * (1.0 - lr * weight_decay)
    m = m + (g - m) * (1.0 - b1)
    v = v * b2 + (1.0 - b2) * g * g
    bc1, bc2 = 1.0 - b1 ** step, 1.0 - b2 ** step
    denom = v.sqrt() / math.sqrt(bc2) + eps
    return p - (lr / bc1) * (m / denom), m, v


def get_slopes(n: int) -> List[float]:
    """reference transformer.py:37-52."""
    def pow2(m):
        start = 2 ** (-(2 ** -(math.log2(m) - 3)))
        return [start * start ** i for i in range(m)]

    if math.log2(n).is_integer():
        return pow2(n)
    lower = 2 ** math.floor(math.log2(n))
    return pow2(lower) + get_slopes(2 * lower)[0::2][: n - lower]


def alibi_mask(seq_len: int, num_heads: int, dtype=torch.float16) -> torch.Tensor:
    """reference transformer.py:55-75 -> (nh, S, S): -(i-j) rounded to ``dtype``,
    times the slope rounded to ``dtype``, product rounded to ``dtype``; -inf above
    the diagonal."""
    i = torch.arange(seq_len).view(seq_len, 1)
    j = torch.arange(seq_len).view(1, seq_len)
    a = (-torch.tril(i - j)).to(dtype)
    slopes = torch.tensor(get_slopes(num_heads), dtype=dtype)
    out = a[None] * slopes[:, None, None]
    return out.masked_fill((j > i)[None], float("-inf"))


# --------------------------------------------------------------------------- model
@dataclass(frozen=True)
class RefConfig:
    vocab_size: int
    hidden_size: int
    max_position_embeddings: int
    num_attention_heads: int
    head_dim: int
    ffn_dim: int
    num_hidden_layers: int
    use_linear_bias: bool
    attn_bias: bool


class _Linear(nn.Module):  # weight (in, out), y = x @ W (+ b): reference nn.py:42-91
    def __init__(self, fin, fout, bias, relu=False):
        super().__init__()
        self.weight = nn.Parameter(torch.empty(fin, fout))
        self.bias = nn.Parameter(torch.empty(fout)) if bias else None
        self.relu = relu

    def forward(self, x):
        return linear(x, self.weight, self.bias, self.relu)


class _LayerNorm(nn.Module):  # reference nn.py:14-39
    def __init__(self, d, eps=1e-5):
        super().__init__()
        self.weight = nn.Parameter(torch.empty(d))
        self.bias = nn.Parameter(torch.empty(d))
        self.eps = eps

    def forward(self, x):
        return F.layer_norm(x, (x.shape[-1],), self.weight, self.bias, self.eps)


class _Attention(nn.Module):  # reference transformer.py:113-190
    def __init__(self, cfg, sdpa):
        super().__init__()
        d = cfg.hidden_size
        self.nh, self.hd, self.sdpa = cfg.num_attention_heads, d // cfg.num_attention_heads, sdpa
        self.q_proj, self.k_proj = _Linear(d, d, False), _Linear(d, d, False)
        self.v_proj, self.out_proj = _Linear(d, d, False), _Linear(d, d, False)

    def forward(self, x, bias):
        b, s, d = x.shape
        q, k, v = (p(x).view(b, s, self.nh, self.hd).transpose(1, 2) for p in (self.q_proj, self.k_proj, self.v_proj))
        if self.sdpa and bias is None:  # same math, no S x S matrix kept for backward
            o = F.scaled_dot_product_attention(q, k, v, is_causal=True)
        else:
            o = causal_attention(q, k, v, bias)
        return self.out_proj(o.transpose(1, 2).reshape(b, s, d))


class _MLP(nn.Module):  # reference transformer.py:193-217
    def __init__(self, cfg):
        super().__init__()
        self.dense_h_to_4h = _Linear(cfg.hidden_size, cfg.ffn_dim, cfg.use_linear_bias, relu=True)
        self.dense_4h_to_h = _Linear(cfg.ffn_dim, cfg.hidden_size, cfg.use_linear_bias)

    def forward(self, x):
        return self.dense_4h_to_h(self.dense_h_to_4h(x))


class _Layer(nn.Module):  # reference transformer.py:220-251
    def __init__(self, cfg, sdpa):
        super().__init__()
        self.input_layernorm = _LayerNorm(cfg.hidden_size)
        self.post_attention_layernorm = _LayerNorm(cfg.hidden_size)
        self.attention = _Attention(cfg, sdpa)
        self.mlp = _MLP(cfg)

    def forward(self, x, bias):
        x = x + self.attention(self.input_layernorm(x), bias)
        return x + self.mlp(self.post_attention_layernorm(x))


class RefTransformer(nn.Module):
    """fp32 restatement of reference transformer.py:254-346 (CPU or GPU)."""

    def __init__(self, cfg, sdpa: bool = False):
        super().__init__()
        self.config = cfg
        self.embed_tokens = nn.Embedding(cfg.vocab_size, cfg.hidden_size)
        self.embed_positions = None if cfg.attn_bias else nn.Embedding(cfg.max_position_embeddings, cfg.hidden_size)
        self.layer_list = nn.ModuleList([_Layer(cfg, sdpa) for _ in range(cfg.num_hidden_layers)])
        self.final_layernorm = _LayerNorm(cfg.hidden_size)
        self.logits_out = _Linear(cfg.hidden_size, cfg.vocab_size, False)
        self.reset_parameters()
        if cfg.attn_bias:
            self.register_buffer("attn_bias", alibi_mask(cfg.max_position_embeddings, cfg.num_attention_heads))
        else:
            self.attn_bias = None

    def reset_parameters(self):
        """reference transformer.py:83-105."""
        n_layers = self.config.num_hidden_layers
        for name, p in self.named_parameters():
            if "layernorm" in name:
                (nn.init.ones_ if name.endswith("weight") else nn.init.zeros_)(p)
            elif name.endswith("bias"):
                nn.init.zeros_(p)
            elif "logits_out" in name:
                nn.init.zeros_(p)
            elif "out_proj" in name or "dense_4h_to_h" in name:
                nn.init.normal_(p, 0.0, 0.02 / math.sqrt(2 * n_layers))
            else:
                nn.init.normal_(p, 0.0, 0.02)

    def forward(self, input_ids, labels: Optional[torch.Tensor]):
        b, s = input_ids.shape
        x = self.embed_tokens(input_ids)
        if self.embed_positions is not None:
            x = x + self.embed_positions(torch.arange(s, device=x.device))[None]
        for layer in self.layer_list:
            x = layer(x, self.attn_bias)
        logits = self.logits_out(self.final_layernorm(x))
        if labels is None:
            return logits
        loss = cross_entropy(logits[:, :-1].reshape(-1, logits.shape[-1]), labels[:, 1:].reshape(-1))
        return logits, loss.mean()


def step_flops(cfg, batch: int, seq: int) -> float:
    """Algorithmic FLOPs of one fwd+bwd step: 6*T*P_mat + 7*L*B*S^2*d (causal
    attention at its real half cost, FA-2 backward = 2.5x forward)."""
    d, f, L, V = cfg.hidden_size, cfg.ffn_dim, cfg.num_hidden_layers, cfg.vocab_size
    p_mat = L * (4 * d * d + 2 * d * f) + d * V
    return 6.0 * batch * seq * p_mat + 7.0 * L * batch * seq * seq * d
