"""GPU parity of the four Linear Functions against the fp32 oracle; mirrors the
reference's tritonformer/test_linear.py (random shapes that are not tile
multiples, x ~ N(0,1), W ~ N(0,1)/sqrt(in), dy ~ N(0,1)) and adds the ReLU
variants, bf16 and the baseline configurations' exact shapes, which the
reference does not test.

Tolerance (fp16): |err| <= 1e-2 + 1e-3*|ref| per element (the reference uses
atol 1e-2 against an fp16 result; the relative term is one fp16 rounding of the
fp32 reference); bias gradient: relative L2 < 1e-3, as test_linear.py:28-30,169.
"""
import numpy as np
import pytest
import torch

import tritonformer_amd as T
import tritonformer_amd.kernels as K_mod
from oracle import ref_torch as R
from tests.util import NUM_TEST, assert_close, rel_l2

pytestmark = pytest.mark.gpu
rng = np.random.RandomState(0)

RANDOM_DIMS = [(int(b), int(m), int(n), int(k))
               for b in rng.randint(1, 8, size=NUM_TEST)
               for m in rng.randint(64, 1024, size=1)
               for n in rng.randint(64, 1536, size=NUM_TEST)
               for k in rng.randint(64, 1536, size=1)]
EDGE_DIMS = [(1, 1, 8, 8), (1, 64, 64, 64), (2, 77, 333, 129), (3, 130, 264, 520), (1, 257, 1024, 72),
             (2, 512, 768, 3072), (1, 300, 4096, 1024)]
# the upper end of the reference's draws (test_linear.py:36-41: B < 32, M, N, K < 4096), ragged
UPPER_DIMS = [(31, 4001, 4093, 3999)]
VARIANTS = {
    "nobias": (T.linear_no_bias, False, False),
    "bias": (T.linear_bias, True, False),
    "relu": (T.linear_fused_relu, False, True),
    "biasrelu": (T.linear_fused_bias_relu, True, True),
}


def make(dims, dtype, dev, seed):
    b, m, n, k = dims
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(b, m, n, generator=g).to(dtype)
    w = (torch.randn(n, k, generator=g) / n ** 0.5).to(dtype)
    bias = torch.randn(k, generator=g).to(dtype)
    dy = torch.randn(b, m, k, generator=g).to(dtype)
    return x, w, bias, dy


def run_case(dims, variant, dtype, dev, seed=0, oracle_on_gpu=False):
    """``oracle_on_gpu``: the fp32 oracle expressions evaluated on the GPU (rocBLAS fp32) instead
    of the CPU, for cases whose CPU time would run to minutes."""
    fn, use_bias, relu = VARIANTS[variant]
    x, w, bias, dy = make(dims, dtype, dev, seed)
    xd, wd, bd = (t.to(dev).requires_grad_(True) for t in (x, w, bias))
    y = fn.apply(xd, wd, bd) if use_bias else fn.apply(xd, wd)
    y.backward(dy.to(dev))
    if oracle_on_gpu:
        x, w, bias, dy = (t.to(dev) for t in (x, w, bias, dy))
    y_ref = R.linear(x, w, bias if use_bias else None, relu)
    assert_close(y, y_ref, dtype, f"{variant} y {dims}")
    # the ReLU gradient mask is the sign of the kernel's own rounded output (as in the
    # reference, linear.py:62): on a pre-activation within rounding of zero fp32 and
    # 16-bit math may disagree, which is not an error of the backward kernels
    act = (y.detach() if oracle_on_gpu else y.detach().cpu()) if relu else None
    dx_ref, dw_ref, db_ref = R.linear_bwd(x, w, dy, act=act, with_bias=use_bias)
    big = dims[0] * dims[1]  # contraction length of dW: rounding noise grows like sqrt
    assert_close(xd.grad, dx_ref, dtype, f"{variant} dx {dims}")
    assert_close(wd.grad, dw_ref, dtype, f"{variant} dw {dims}", atol=1e-2 * max(1.0, (big / 512) ** 0.5) * (6 if dtype == torch.bfloat16 else 1))
    assert wd.grad.shape == w.shape
    if use_bias:
        assert bd.grad.shape == bias.shape
        assert rel_l2(bd.grad, db_ref) < (1e-3 if dtype == torch.float16 else 8e-3), f"{variant} db {dims}"


@pytest.mark.parametrize("dims", RANDOM_DIMS + EDGE_DIMS)
@pytest.mark.parametrize("variant", ["nobias", "bias"])
def test_linear_fwd_bwd(dims, variant, dev):
    run_case(dims, variant, torch.float16, dev)


@pytest.mark.parametrize("dims", UPPER_DIMS)
@pytest.mark.parametrize("variant", ["bias", "relu"])
def test_linear_upper_end_of_reference_range(dims, variant, dev):
    run_case(dims, variant, torch.float16, dev, oracle_on_gpu=True)


def test_linear_large_ragged_against_cpu_oracle(dev):
    """M, N, K near the top of the reference's range, ragged, with the oracle on the CPU."""
    run_case((3, 3999, 4093, 4001), "biasrelu", torch.float16, dev)


@pytest.mark.parametrize("dims", EDGE_DIMS + RANDOM_DIMS[:3])
@pytest.mark.parametrize("variant", ["relu", "biasrelu"])
def test_linear_relu_fwd_bwd(dims, variant, dev):
    run_case(dims, variant, torch.float16, dev)


@pytest.mark.parametrize("dims", [(2, 77, 333, 129), (2, 256, 1024, 512)])
@pytest.mark.parametrize("variant", list(VARIANTS))
def test_linear_bf16(dims, variant, dev):
    run_case(dims, variant, torch.bfloat16, dev)


def test_relu_fused_equals_unfused(dev):
    x, w, bias, _ = make((2, 100, 256, 384), torch.float16, dev, 3)
    xd, wd, bd = x.to(dev), w.to(dev), bias.to(dev)
    assert torch.equal(T.linear_fused_relu.apply(xd, wd), torch.relu(T.linear_no_bias.apply(xd, wd)))
    assert torch.equal(T.linear_fused_bias_relu.apply(xd, wd, bd), torch.relu(T.linear_bias.apply(xd, wd, bd)))


def test_identity_and_permutation_weights(dev):
    x = torch.randn(2, 70, 128).half().to(dev)
    eye = torch.eye(128).half().to(dev)
    assert torch.equal(T.linear_no_bias.apply(x, eye), x)
    perm = torch.randperm(128)
    assert torch.equal(T.linear_no_bias.apply(x, eye[:, perm.to(dev)]), x[..., perm.to(dev)])


def test_grad_buffers_not_mutated_and_deterministic(dev):
    """The reference masks grad_output in place (kernels/activation.py:24); ours must
    leave autograd's buffer alone, and two runs must agree bit for bit."""
    x, w, bias, dy = make((2, 128, 256, 512), torch.float16, dev, 5)
    xd, wd = x.to(dev).requires_grad_(True), w.to(dev).requires_grad_(True)
    dyd = dy.to(dev)
    keep = dyd.clone()
    y = T.linear_fused_relu.apply(xd, wd)
    y.backward(dyd, retain_graph=True)
    g1 = (xd.grad.clone(), wd.grad.clone())
    assert torch.equal(dyd, keep)
    xd.grad = wd.grad = None
    y.backward(dyd)
    assert torch.equal(g1[0], xd.grad) and torch.equal(g1[1], wd.grad)


def test_transposed_weight_view_and_noncontiguous_input(dev):
    x = torch.randn(2, 96, 160).half()
    w = torch.randn(200, 160).half() / 12.0
    y = T.linear_no_bias.apply(x.to(dev), w.to(dev).T)          # stride-(1, K) view, as linear.py:23 passes
    assert_close(y, R.linear(x, w.T), name="transposed weight")
    xt = torch.randn(2, 160, 96).half()
    y2 = T.linear_no_bias.apply(xt.to(dev).transpose(1, 2), w.to(dev).T)
    assert_close(y2, R.linear(xt.transpose(1, 2), w.T), name="non-contiguous input")


def test_autocast_fp32_master_weights(dev):
    """custom_fwd(cast_inputs=float16) semantics (reference linear.py:14): fp32 inputs are
    cast inside autocast; gradients come back in fp32."""
    x = torch.randn(2, 64, 128, device=dev, requires_grad=True)
    w = (torch.randn(128, 256, device=dev) / 11.3).requires_grad_(True)
    b = torch.randn(256, device=dev, requires_grad=True)
    with torch.autocast("cuda", dtype=torch.float16):
        y = T.linear_bias.apply(x, w, b)
    assert y.dtype == torch.float16
    y.float().sum().backward()
    assert x.grad.dtype == w.grad.dtype == b.grad.dtype == torch.float32
    dx, dw, db = R.linear_bwd(x.detach().cpu(), w.detach().cpu(), torch.ones(2, 64, 256), with_bias=True)
    assert rel_l2(w.grad, dw) < 2e-3 and rel_l2(x.grad, dx) < 2e-3 and rel_l2(b.grad, db) < 1e-3
    with torch.autocast("cuda", dtype=torch.bfloat16):
        assert T.linear_no_bias.apply(x, w).dtype == torch.bfloat16
    with pytest.raises(TypeError):   # outside autocast fp32 inputs are not accepted (16-bit kernels only)
        T.linear_no_bias.apply(x, w)


@pytest.mark.parametrize("shape", [(4, 2048, 1024, 4096), (4, 2048, 4096, 1024), (4, 2048, 1024, 1024)])
def test_headline_config_shapes(shape, dev):
    """410M / ctx 2048 / bs 4 layer shapes at full size against the fp32 oracle on the CPU."""
    b, s, n, k = shape
    g = torch.Generator().manual_seed(1)
    x = torch.randn(b, s, n, generator=g).half().to(dev).requires_grad_(True)
    w = (torch.randn(n, k, generator=g) * 0.02).half().to(dev).requires_grad_(True)
    dy = torch.randn(b, s, k, generator=g).half().to(dev)
    y = T.linear_no_bias.apply(x, w)
    y.backward(dy)
    xc, wc, dyc = x.detach().cpu(), w.detach().cpu(), dy.cpu()
    assert_close(y, R.linear(xc, wc), name="y")
    dx, dw, _ = R.linear_bwd(xc, wc, dyc)
    assert_close(x.grad, dx, name="dx")
    assert rel_l2(w.grad, dw) < 1e-3
    # linearity in dy: the weight gradient of 2*dy is exactly twice (power-of-two scaling is exact in fp16)
    x.grad = w.grad = None
    T.linear_no_bias.apply(x, w).backward(2 * dy)
    assert rel_l2(w.grad, 2 * dw) < 1e-3


def test_logits_projection_shape(dev):
    """hidden -> vocab projection of the headline model on a slice of the tokens."""
    g = torch.Generator().manual_seed(2)
    x = torch.randn(1, 512, 1024, generator=g).half().to(dev).requires_grad_(True)
    w = (torch.randn(1024, 50304, generator=g) * 0.02).half().to(dev).requires_grad_(True)
    y = T.linear_no_bias.apply(x, w)
    dy = (torch.randn(1, 512, 50304, generator=g) * 0.1).half().to(dev)
    y.backward(dy)
    assert_close(y, R.linear(x.detach(), w.detach()), name="logits")
    dx, dw, _ = R.linear_bwd(x.detach(), w.detach(), dy)
    assert_close(x.grad, dx, name="dx", atol=2e-2)
    assert rel_l2(w.grad, dw) < 1e-3


@pytest.mark.parametrize("d_in,f,d_out", [(64, 128, 72), (128, 256, 200), (256, 512, 64), (72, 128, 64)])
@pytest.mark.parametrize("use_bias", [False, True])
def test_fused_mlp_with_different_input_and_output_widths(d_in, f, d_out, use_bias, dev):
    """x (.., d_in) W1 (d_in, f) W2 (f, d_out) with d_out != d_in: the forward product (contraction
    over d_in) may keep the ReLU mask as sign bits while the backward product dH = dY W2^T
    (contraction over d_out) misses the preconditions of the kernel that reads them (d_out not a
    multiple of 64); the backward then masks with the saved activation.  Must equal the two
    Functions bit for bit either way."""
    g = torch.Generator().manual_seed(13)
    x = torch.randn(2, 96, d_in, generator=g).half().to(dev)
    w1 = (torch.randn(d_in, f, generator=g) / d_in ** 0.5).half().to(dev)
    w2 = (torch.randn(f, d_out, generator=g) / f ** 0.5).half().to(dev)
    b1 = torch.randn(f, generator=g).half().to(dev) if use_bias else None
    b2 = torch.randn(d_out, generator=g).half().to(dev) if use_bias else None
    dy = torch.randn(2, 96, d_out, generator=g).half().to(dev)
    a = [t.clone().requires_grad_(True) if t is not None else None for t in (x, w1, b1, w2, b2)]
    ya = T.mlp_fused_relu.apply(*a)
    ya.backward(dy)
    c = [t.clone().requires_grad_(True) if t is not None else None for t in (x, w1, b1, w2, b2)]
    if use_bias:
        yb = T.linear_bias.apply(T.linear_fused_bias_relu.apply(c[0], c[1], c[2]), c[3], c[4])
    else:
        yb = T.linear_no_bias.apply(T.linear_fused_relu.apply(c[0], c[1]), c[3])
    yb.backward(dy)
    assert torch.equal(ya, yb)
    for ta, tb in zip(a, c):
        if ta is not None:
            assert torch.equal(ta.grad, tb.grad)
    hidden = R.linear(x.cpu(), w1.cpu(), b1.cpu() if use_bias else None, True).half()
    assert_close(ya, R.linear(hidden, w2.cpu(), b2.cpu() if use_bias else None), name="mlp y", atol=2e-2)


def test_bias_gradient_of_fp32_master_bias_is_unrounded(dev):
    """Under autocast an fp32 bias gets the fp32 column sums themselves, not a 16-bit rounding of
    them cast back: the sums of 16384 rows of values near 1 would lose 3 digits in fp16."""
    g = torch.Generator().manual_seed(17)
    x = torch.randn(8, 2048, 64, generator=g).to(dev).requires_grad_(True)
    w = (torch.randn(64, 128, generator=g) / 8).to(dev).requires_grad_(True)
    b = torch.zeros(128, device=dev, requires_grad=True)
    dy = (1.0 + 0.1 * torch.randn(8, 2048, 128, generator=g)).half()
    with torch.autocast("cuda", dtype=torch.float16):
        y = T.linear_bias.apply(x, w, b)
    y.backward(dy.to(dev))
    want = dy.double().sum((0, 1))
    assert b.grad.dtype == torch.float32
    assert (b.grad.cpu().double() - want).abs().max() <= 2e-6 * want.abs().max()   # fp16 would be off by ~8
    with torch.autocast("cuda", dtype=torch.float16):
        y = T.mlp_fused_relu.apply(x, w, b, w.detach().T.contiguous().requires_grad_(True), None)
    b.grad = None
    y.sum().backward()
    assert b.grad.dtype == torch.float32 and torch.isfinite(b.grad).all()


@pytest.mark.parametrize("layouts", ["fwd", "dx", "dw"])
def test_every_tile_configuration_gives_the_same_product(layouts, dev):
    """The diagnostic entry point imposes each tile configuration in turn on one product that all
    of them can take: an unsplit contraction sums the same 64-wide steps in the same order whatever
    the tile shape, so the results are equal bit for bit; a split one differs in fp32 summation
    order only.  Also with the XCD remap of workgroup ids switched off."""
    from tritonformer_amd import _lib

    d = _lib.load_diag()
    g = torch.Generator().manual_seed(23)
    M, N, K = 640, 768, 512
    la, lb = {"fwd": (0, 1), "dx": (0, 0), "dw": (1, 1)}[layouts]
    a = torch.randn((M, K) if la == 0 else (K, M), generator=g).half().to(dev)
    b = (torch.randn((N, K) if lb == 0 else (K, N), generator=g) / K ** 0.5).half().to(dev)
    a32, b32 = (a.float() if la == 0 else a.float().T), (b.float() if lb == 0 else b.float().T)
    want = a32 @ b32.T
    stream = torch.cuda.current_stream().cuda_stream

    def run(cfg, splits, flags):
        out = torch.empty((M, N), dtype=torch.float16, device=dev)
        nb = d.tf_diag_gemm_workspace_bytes(cfg, splits, M, N, K)
        ws = torch.empty(max(nb, 16), dtype=torch.uint8, device=dev)
        _lib.check(d.tf_diag_gemm(stream, cfg, splits, flags, 0, 0, la, lb, M, N, K, a.data_ptr(), a.stride(0),
                                  b.data_ptr(), b.stride(0), out.data_ptr(), N, None, 0, ws.data_ptr(), nb))
        return out

    base = run(-1, 0, 0)
    assert_close(base, want, name=f"{layouts} auto")
    for cfg in range(6):
        assert torch.equal(run(cfg, 1, 0), base), f"cfg {cfg}"
        assert torch.equal(run(cfg, 1, 1), base), f"cfg {cfg} without the XCD remap"
        assert rel_l2(run(cfg, 4, 0), base) < 1e-3, f"cfg {cfg} split 4"


@pytest.mark.parametrize("layouts", ["fwd", "dx", "dw"])
def test_short_contractions_take_every_peeled_form_of_the_main_loop(layouts, dev):
    """One to nine 64-wide stages: the main loop of the direct-to-LDS kernels peels
    its last two stages (no stage after, one stage after; three with three LDS buffers) from the steady state, and its
    prologue requests the head of the second stage (with three buffers: all of it and the head of the third) before it
    waits for the first.  Every tile configuration,
    against fp32 math, with and without a split that leaves a single stage per slice."""
    from tritonformer_amd import _lib

    d = _lib.load_diag()
    g = torch.Generator().manual_seed(31)
    M, N = 384, 512
    la, lb = {"fwd": (0, 1), "dx": (0, 0), "dw": (1, 1)}[layouts]
    stream = torch.cuda.current_stream().cuda_stream
    for K in (64, 128, 192, 256, 320, 384, 448, 576):   # (the three-buffer configurations peel three stages and rotate)
        a = torch.randn((M, K) if la == 0 else (K, M), generator=g).half().to(dev)
        b = (torch.randn((N, K) if lb == 0 else (K, N), generator=g) / K ** 0.5).half().to(dev)
        want = (a.float() if la == 0 else a.float().T) @ (b.float().T if lb == 0 else b.float())
        for cfg in range(2, 6):
            for splits in (1, K // 64):
                out = torch.empty((M, N), dtype=torch.float16, device=dev)
                nb = d.tf_diag_gemm_workspace_bytes(cfg, splits, M, N, K)
                ws = torch.empty(max(nb, 16), dtype=torch.uint8, device=dev)
                _lib.check(d.tf_diag_gemm(stream, cfg, splits, 0, 0, 0, la, lb, M, N, K, a.data_ptr(), a.stride(0),
                                          b.data_ptr(), b.stride(0), out.data_ptr(), N, None, 0, ws.data_ptr(), nb))
                assert_close(out, want, name=f"{layouts} K={K} cfg {cfg} splits {splits}")


@pytest.mark.parametrize("dims,use_bias", [((2, 128, 256, 1024), False), ((3, 77, 136, 264), True),
                                           ((1, 100, 333, 129), True)])
def test_fused_mlp_equals_two_functions(dims, use_bias, dev):
    """mlp_fused_relu must equal linear_fused_(bias_)relu followed by linear_(no_)bias bit for
    bit (same GEMM calls; the mask is applied in the write-out instead of a separate pass)."""
    b, m, d, f = dims
    g = torch.Generator().manual_seed(9)
    x = torch.randn(b, m, d, generator=g).half().to(dev)
    w1 = (torch.randn(d, f, generator=g) / d ** 0.5).half().to(dev)
    w2 = (torch.randn(f, d, generator=g) / f ** 0.5).half().to(dev)
    b1 = torch.randn(f, generator=g).half().to(dev) if use_bias else None
    b2 = torch.randn(d, generator=g).half().to(dev) if use_bias else None
    dy = torch.randn(b, m, d, generator=g).half().to(dev)

    def leaves():
        return [t.clone().requires_grad_(True) if t is not None else None for t in (x, w1, b1, w2, b2)]

    a = leaves()
    ya = T.mlp_fused_relu.apply(*a)
    ya.backward(dy)
    c = leaves()
    if use_bias:
        yb = T.linear_bias.apply(T.linear_fused_bias_relu.apply(c[0], c[1], c[2]), c[3], c[4])
    else:
        yb = T.linear_no_bias.apply(T.linear_fused_relu.apply(c[0], c[1]), c[3])
    yb.backward(dy)
    assert torch.equal(ya, yb)
    for ta, tb in zip(a, c):
        if ta is not None:
            assert torch.equal(ta.grad, tb.grad)
    y_ref = R.linear(R.linear(x.cpu(), w1.cpu(), b1.cpu() if use_bias else None, True).half(), w2.cpu(),
                     b2.cpu() if use_bias else None)
    assert_close(ya, y_ref, name="mlp y", atol=2e-2)


@pytest.mark.parametrize("dims", [(2, 77, 328, 136), (4, 2048, 1024, 1024), (1, 64, 64, 8)])
@pytest.mark.parametrize("master", [False, True])
def test_packed_projections_equal_separate_functions(dims, master, dev):
    """linear_no_bias_packed(x, Wq, Wk, Wv) against three linear_no_bias calls: the
    forward is the same arithmetic per element (bitwise equal), the weight gradients
    are the same products summed in fp32 (equal up to summation order); dX sums one contraction of length 3*out instead of three rounded partial
    results, so it is compared with the fp32 oracle at the linear tolerance.
    `master`: fp32 weights under autocast (fp32 gradients straight from the accumulators)."""
    b, m, n, k = dims
    g = torch.Generator().manual_seed(11)
    x = torch.randn(b, m, n, generator=g).half()
    ws = [(torch.randn(n, k, generator=g) / n ** 0.5) for _ in range(3)]
    if not master:
        ws = [w.half() for w in ws]
    dy = torch.randn(b, m, 3 * k, generator=g).half()

    def run(packed):
        xd = x.to(dev).requires_grad_(True)
        wd = [w.to(dev).requires_grad_(True) for w in ws]
        with torch.autocast("cuda", dtype=torch.float16, enabled=master):
            if packed:
                y = T.linear_no_bias_packed.apply(xd, *wd)
            else:
                y = torch.cat([T.linear_no_bias.apply(xd, w) for w in wd], dim=-1)
        y.backward(dy.to(dev))
        return y, xd.grad, [w.grad for w in wd]

    y1, dx1, dw1 = run(True)
    y0, dx0, dw0 = run(False)
    assert torch.equal(y1, y0)
    for a, c in zip(dw1, dw0):
        assert a.is_contiguous() and a.dtype == (torch.float32 if master else torch.float16)
        # same products; the contraction over B*S may be split differently for the (in, 3*out)
        # problem than for (in, out), which changes the fp32 summation order only
        assert rel_l2(a, c) < (1e-5 if master else 1e-3)
    w16 = torch.cat([w.half() for w in ws], dim=1)
    dx_ref, _, _ = R.linear_bwd(x, w16, dy, act=None, with_bias=False)
    assert_close(dx1, dx_ref, torch.float16, f"packed dx {dims}", atol=2e-2)


def test_cast_pack_and_chunked_weight_gradient(dev):
    from tritonformer_amd import kernels as K

    g = torch.Generator().manual_seed(2)
    ws = [torch.randn(40, 24, generator=g).to(dev) for _ in range(3)]
    for dt in (torch.float16, torch.bfloat16):
        assert torch.equal(K.cast_pack(ws, dt), torch.cat([w.to(dt) for w in ws], dim=1))
        assert torch.equal(K.cast_pack([w.to(dt) for w in ws[:2]], dt), torch.cat([w.to(dt) for w in ws[:2]], dim=1))
    odd = [torch.randn(5, 7, generator=g).to(dev) for _ in range(4)]     # no 16-byte chunks: element path
    assert torch.equal(K.cast_pack(odd, torch.float16), torch.cat([w.half() for w in odd], dim=1))
    with pytest.raises(ValueError):
        K.cast_pack(ws + ws, torch.float16)
    with pytest.raises(TypeError):
        K.cast_pack([w.half() for w in ws], torch.bfloat16)
    x = torch.randn(2, 300, 72, generator=g).half().to(dev)
    dy = torch.randn(2, 300, 96, generator=g).half().to(dev)
    for od in (None, torch.float32):
        whole = K.mm_dw(x, dy, out_dtype=od)
        parts = K.mm_dw(x, dy, out_dtype=od, chunks=3)
        assert parts.shape == (3, 72, 32)
        assert torch.equal(torch.cat(list(parts), dim=1), whole)
    with pytest.raises(ValueError):
        K.mm_dw(x, dy, chunks=5)


@pytest.mark.parametrize("case", ["mlp-410m", "mlp-840m", "ragged", "chunked", "single", "eight"])
def test_grouped_weight_gradients_equal_separate_products(case, dev):
    """mm_dw_group against one mm_dw per problem: same products, summed in fp32 (the
    contraction may be cut into a different number of slices), fp32 and fp16 outputs;
    'ragged' has extents the one-launch path cannot take and runs problem by problem;
    'mlp-840m' has 288 tiles, a round of workgroups and an eighth: the launch keeps whole tiles
    for the round and splits the contraction of the last tile columns of one product; 'eight' is the
    form in which the weight gradients of several layers are handed over together: 256 tiles, one
    round of workgroups, every contraction unsplit."""
    from tritonformer_amd import kernels as K

    g = torch.Generator().manual_seed(7)
    shapes = {"mlp-410m": [((4, 2048, 1024), 4096), ((4, 2048, 4096), 1024)],
              "mlp-840m": [((1, 4096, 1536), 6144), ((1, 4096, 6144), 1536)],
              "ragged": [((2, 77, 136), 72), ((2, 77, 72), 333)],
              "chunked": [((2, 512, 256), 768), ((2, 512, 256), 256), ((2, 512, 768), 256)],
              "single": [((1, 640, 512), 512)],
              "eight": [((1, 512, 1024), 3072), ((1, 512, 1024), 1024)] * 2
                       + [((1, 512, 1024), 4096), ((1, 512, 4096), 1024)]
                       + [((1, 512, 1024), 3072), ((1, 512, 1024), 1024)]}[case]
    pairs = [((torch.randn(*xs, generator=g)).half().to(dev), torch.randn(*xs[:-1], n, generator=g).half().to(dev))
             for xs, n in shapes]
    chunks = {"chunked": [3, 1, 1], "eight": [3, 1, 3, 1, 1, 1, 3, 1]}.get(case, [1] * len(pairs))
    for od in (torch.float32, None):
        outs = K.mm_dw_group(pairs, out_dtype=od, chunks=chunks)
        for (x, gr), ch, got in zip(pairs, chunks, outs):
            want = K.mm_dw(x, gr, out_dtype=od, chunks=ch)
            assert got.shape == want.shape and got.dtype == want.dtype and got.is_contiguous()
            assert rel_l2(got, want) < (1e-5 if od is torch.float32 else 1e-3)
        if (case.startswith("mlp") or case == "eight") and od is torch.float32:   # and against the fp32 oracle
            for (x, gr), got in zip(pairs, outs):
                ref = x.float().cpu().reshape(-1, x.shape[-1]).T @ gr.float().cpu().reshape(-1, gr.shape[-1])
                assert rel_l2(got.transpose(0, 1).reshape(ref.shape) if got.ndim == 3 else got, ref) < 1e-4
            again = K.mm_dw_group(pairs, out_dtype=od, chunks=chunks)   # fixed summation order: the same bits
            assert all(torch.equal(a, b) for a, b in zip(again, outs))
    with pytest.raises(ValueError):
        K.mm_dw_group(pairs * 17)


@pytest.mark.gpu
@pytest.mark.parametrize("dims", [(2, 128, 256, 1024), (1, 384, 128, 320), (1, 4096, 1536, 6144)])
@pytest.mark.parametrize("use_bias", [False, True])
def test_relu_sign_bits_equal_the_activation_mask(dims, use_bias, dev):
    """gemm_relu_bits returns relu(x W + b) bit-identical to the plain ReLU GEMM, and one bit per
    element that says where it is positive (bit n % 8 of byte n / 8); the masked product taken
    from those bits equals the one that reads the activation (kernels/activation.py:27-44).
    The last case has a round and a half of 256x256 tiles: both products are cut into whole rounds
    and a remainder, each part with its share of the bit rows."""
    import numpy as np
    from tritonformer_amd import kernels as K

    b, m, d, f = dims
    g = torch.Generator().manual_seed(31)
    x = torch.randn(b, m, d, generator=g).half().to(dev)
    w1 = (torch.randn(d, f, generator=g) / d ** 0.5).half().to(dev)
    w2 = (torch.randn(f, d, generator=g) / f ** 0.5).half().to(dev)
    b1 = torch.randn(f, generator=g).half().to(dev) if use_bias else None
    dy = torch.randn(b, m, d, generator=g).half().to(dev)
    hidden, bits = K.gemm_relu_bits(x, w1, b1)
    assert bits is not None and bits.shape == (b * m, f // 8) and bits.dtype == torch.uint8
    assert torch.equal(hidden, K.gemm(x, w1, b1, True))
    expect = np.packbits((hidden.reshape(-1, f) > 0).cpu().numpy(), axis=1, bitorder="little")
    assert np.array_equal(bits.cpu().numpy(), expect)
    assert torch.equal(K.mm_masked_bits(dy, w2.T, bits), K.mm(dy, w2.T, mask_act=hidden))


@pytest.mark.gpu
def test_relu_sign_bits_fall_back_when_the_kernel_cannot_take_the_problem(dev):
    """A contraction length that the direct-to-LDS kernel does not take: no bits, same result;
    the fused MLP then masks with the activation and still matches the two-function form."""
    from tritonformer_amd import kernels as K

    g = torch.Generator().manual_seed(32)
    x = torch.randn(1, 64, 72, generator=g).half().to(dev)
    w1 = (torch.randn(72, 96, generator=g) / 8).half().to(dev)
    w2 = (torch.randn(96, 72, generator=g) / 8).half().to(dev)
    hidden, bits = K.gemm_relu_bits(x, w1, None)
    assert bits is None and torch.equal(hidden, K.gemm(x, w1, None, True))
    a = [t.clone().requires_grad_(True) for t in (x, w1, w2)]
    T.mlp_fused_relu.apply(a[0], a[1], None, a[2], None).sum().backward()
    c = [t.clone().requires_grad_(True) for t in (x, w1, w2)]
    T.linear_no_bias.apply(T.linear_fused_relu.apply(c[0], c[1]), c[2]).sum().backward()
    for ta, tb in zip(a, c):
        assert torch.equal(ta.grad, tb.grad)


@pytest.mark.gpu
def test_product_cut_into_whole_rounds_and_remainder(dev):
    """8192 x 3072 x 1024 (the packed q/k/v projection of the 410M model) runs as one round of
    256 x 256 tiles over the first 2048 columns plus the last 1024 columns as a product of their
    own.  Every output element is the same contraction either way: the result must equal, bit for
    bit, the two column blocks computed by separate calls, bias and ReLU included, and match the
    fp32 oracle."""
    from tritonformer_amd import kernels as K

    g = torch.Generator().manual_seed(41)
    x = torch.randn(4, 2048, 1024, generator=g).half().to(dev)
    w = (torch.randn(1024, 3072, generator=g) * 0.02).half().to(dev)
    bias = torch.randn(3072, generator=g).half().to(dev)
    for b_, relu in ((None, False), (bias, True)):
        y = K.gemm(x, w, b_, relu)
        left = K.gemm(x, w[:, :2048].contiguous(), None if b_ is None else b_[:2048].contiguous(), relu)
        right = K.gemm(x, w[:, 2048:].contiguous(), None if b_ is None else b_[2048:].contiguous(), relu)
        assert torch.equal(y[..., :2048], left) and torch.equal(y[..., 2048:], right)
        assert_close(y, R.linear(x, w, b_, relu), name="y")


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("case", [
    # (la, lb, M, N, K, what the library does with it)
    (0, 1, 100, 333, 129, "ragged, K not a multiple of 64: register-staged kernel"),
    (0, 0, 77, 136, 264, "unaligned leading dimensions cannot occur here, odd extents do: register-staged kernel"),
    (1, 1, 256, 256, 8192, "one tile, long contraction: split over workgroups, scaled in the reduce pass"),
    (0, 1, 8192, 3072, 1024, "1.5 rounds of tiles: cut along N into whole rounds + tail"),
    (0, 0, 512, 1024, 4096, "direct-to-LDS kernel, scaled in its write-out"),
])
def test_gemm_scaled_is_alpha_times_the_product(case, dtype, dev):
    """tf_gemm_scaled multiplies the fp32 sums by a device-resident scalar in whichever write-out the
    product takes (register-staged kernel, direct-to-LDS kernel, reduce pass of a split contraction,
    both halves of a product cut along N): against tf_gemm_out with an fp32 result scaled afterwards,
    for fp32 and for 16-bit output.  The factor is applied before the single rounding, so both
    comparisons are exact."""
    la, lb, M, N, K, _ = case
    g = torch.Generator().manual_seed(41)
    a = torch.randn((M, K) if la == 0 else (K, M), generator=g).to(dtype).to(dev)
    b = (torch.randn((N, K) if lb == 0 else (K, N), generator=g) / K ** 0.5).to(dtype).to(dev)
    alpha = torch.tensor([0.3173], dtype=torch.float32, device=dev)
    plain = torch.empty((M, N), dtype=torch.float32, device=dev)
    K_mod._gemm(dtype, la, lb, M, N, K, a, a.stride(0), b, b.stride(0), plain, N, None, False)
    want = (a.float() if la == 0 else a.float().T) @ (b.float().T if lb == 0 else b.float())
    assert rel_l2(plain, want) < 1e-3
    for out_dtype in (torch.float32, dtype):
        out = torch.full((M, N), float("nan"), dtype=out_dtype, device=dev)
        K_mod.gemm_scaled(a, la, M, K, a.stride(0), b, lb, N, b.stride(0), alpha, out)
        assert torch.equal(out, (plain * alpha).to(out_dtype)), (case, out_dtype)


@pytest.mark.gpu
@pytest.mark.parametrize("pitch,shift", [(40, 0), (48, 8), (37, 0)])
def test_sign_bit_rows_of_any_pitch_and_alignment(pitch, shift, dev):
    """tf_gemm_relu_bits through the C ABI with bit rows that the 16-byte write-out cannot take (a pitch that
    is no multiple of 16 bytes, a buffer that starts 8 bytes into a 16-byte line): the byte-wise write-out
    serves them -- same activation, same bits, and the masked product read back from those rows equals the
    one that reads the activation (kernels/activation.py:27-44)."""
    import numpy as np
    from tritonformer_amd import _lib
    from tritonformer_amd import kernels as K

    lib = _lib.load()
    g = torch.Generator().manual_seed(41)
    m, d, f = 512, 256, 256
    x = torch.randn(m, d, generator=g).half().to(dev)
    w1 = (torch.randn(d, f, generator=g) / d ** 0.5).half().to(dev)
    w2 = (torch.randn(f, d, generator=g) / f ** 0.5).half().to(dev)
    dy = torch.randn(m, d, generator=g).half().to(dev)
    hidden = torch.empty(m, f, dtype=torch.float16, device=dev)
    raw = torch.zeros(m * pitch + 64, dtype=torch.uint8, device=dev)
    bits = raw[shift:shift + m * pitch].view(m, pitch)
    st = _lib.stream_ptr()
    # forward: x (m, d) k-contiguous, W1 (d, f) k-strided
    rc = lib.tf_gemm_relu_bits(st, 0, 0, 0, 1, m, f, d, x.data_ptr(), d, w1.data_ptr(), f, hidden.data_ptr(), f, None,
                               bits.data_ptr(), None, pitch)
    assert rc == 0
    want_h = K.gemm(x.view(1, m, d), w1, None, True).view(m, f)
    assert torch.equal(hidden, want_h)
    expect = np.packbits((want_h > 0).cpu().numpy(), axis=1, bitorder="little")
    assert np.array_equal(bits[:, : f // 8].cpu().numpy(), expect)
    assert not bits[:, f // 8:].any()                      # nothing written between the rows
    # backward: dH = (dY W2^T) masked by the bits; W2 (f, d) read with the contraction contiguous
    dh = torch.empty(m, f, dtype=torch.float16, device=dev)
    rc = lib.tf_gemm_relu_bits(st, 0, 0, 0, 0, m, f, d, dy.data_ptr(), d, w2.data_ptr(), d, dh.data_ptr(), f, None,
                               None, bits.data_ptr(), pitch)
    assert rc == 0
    assert torch.equal(dh, K.mm(dy.view(1, m, d), w2.T, mask_act=want_h.view(1, m, f)).view(m, f))
