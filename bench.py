#!/usr/bin/env python3
"""Headline benchmark: one fwd+bwd training step of the 410M / ctx 2048 / bs 4
GPT-2 style decoder (24 layers, d=1024, 16 heads x 64, MLP 4096 ReLU, no linear
bias, no ALiBi, vocab 50304) on ONE MI355X, fp16 autocast over fp32 master
weights, every Linear / LayerNorm / attention / cross-entropy running on the
tritonformer_amd HIP kernels.  Prints one JSON line.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload NAME] [--no-cpu-baseline]
                    [--no-extras] [--gemm-table FILE]

value        = algorithmic FLOPs of the step (6*T*P_mat + 7*L*B*S^2*d) / step time, in TFLOP/s, for the
               reference's protocol (README.md:62-77: forward under autocast, `loss.backward()` unscaled,
               no optimizer), the 16-bit copies of the unchanged fp32 master weights kept between steps
               (the reference holds fp16 parameters and converts nothing)
extras       = the same step timed in the other regimes, in the same run: `loss_scaled` (backward of
               loss * 1024: without scaling, fp16 flushes most of the 1/N-scaled logit gradients to
               zero and the backward GEMMs multiply near-constant operands, which the matrix cores run
               at a higher clock), `recast_each_step` (weights converted in every forward pass),
               `training_regime` (both of these at once: what a step followed by an optimizer pays),
               `drop_in_graph` (every model-level fusion off: the reference's graph node for node through
               the reference-named Functions) and `workloads` (the other configurations of the baseline)
roofline     = the GEMM kernel (dominant in time): algorithmic FLOPs per launch / mean launch
               duration, the duration measured with HIP events recorded on the launch stream
               around every GEMM launch in instrumented repeats of the same steps; `other_kernels`
               holds the same for the attention kernels (against MFMA peak) and for the LayerNorm and
               cross-entropy kernels (algorithmic bytes against HBM peak)
cpu_baseline = the fp32 PyTorch oracle (oracle/ref_torch.py) on the host cores, on a bounded
               sample: the same step with the stack cut to 2 layers
"""
import argparse
import json
import os
import sys
import time

import torch

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

PEAK_FP16_TFLOPS = 2500.0  # MI355X dense fp16/bf16 MFMA
PEAK_HBM_GBS = 8000.0
# HBM bytes per GEMM launch at the headline workload, from rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE
# scaled against a streaming kernel of known size (profiles/hbm_traffic_410m_step.md)
GEMM_TRAFFIC_BYTES_PER_LAUNCH = {"gpt2-410m-ctx2048-bs4": 170.5e6}

WORKLOADS = {
    # name: (layers, d, heads, head_dim, ffn, seq, batch, linear_bias, alibi)
    "gpt2-410m-ctx2048-bs4": (24, 1024, 16, 64, 4096, 2048, 4, False, False),
    "gpt2-160m-ctx2048-bs8": (12, 768, 12, 64, 3072, 2048, 8, True, False),
    "gpt2-840m-alibi-ctx4096-bs1": (24, 1536, 24, 64, 6144, 4096, 1, False, True),
    "gpt2-1.4b-ctx2048-bs2": (24, 2048, 16, 128, 8192, 2048, 2, False, False),
    "gpt2-tiny-ctx256-bs2": (4, 256, 4, 64, 1024, 256, 2, True, False),
}
VOCAB = 50304


def step_flops(L, d, f, S, B):
    p_mat = L * (4 * d * d + 2 * d * f) + d * VOCAB
    return 6.0 * B * S * p_mat + 7.0 * L * B * S * S * d


def gemm_flops(L, d, f, S, B):
    return 6.0 * B * S * (L * (4 * d * d + 2 * d * f) + d * VOCAB)


def make_model(name, device, dtype):
    from tritonformer_amd.transformer import Transformer, TransformerConfig

    L, d, nh, hd, f, S, B, lin_bias, alibi = WORKLOADS[name]
    cfg = TransformerConfig(VOCAB, d, S, nh, hd, f, L, lin_bias, alibi)
    torch.manual_seed(0)
    model = Transformer(cfg, device=device, param_dtype=torch.float32)
    model.logits_out.weight.data.normal_(0.0, 0.02)  # reference init zeros the LM head; keep the loss path live
    tokens = torch.randint(0, VOCAB, (B, S), device=device)
    return model, tokens


def run_steps(model, tokens, n, dtype, loss_scale=None):
    loss = None
    for _ in range(n):
        model.zero_grad(set_to_none=True)
        with torch.autocast("cuda", dtype=dtype):
            _, loss = model(tokens, tokens)
        (loss if loss_scale is None else loss * loss_scale).backward()
    return loss


def time_steps(model, tokens, steps, warmup, dtype, loss_scale=None):
    """-> (ms per step, last loss): `warmup` untimed steps, then exactly `steps` between two synchronisations."""
    run_steps(model, tokens, warmup, dtype, loss_scale)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    loss = run_steps(model, tokens, steps, dtype, loss_scale)
    torch.cuda.synchronize()
    return (time.perf_counter() - t0) / steps * 1e3, float(loss.detach())


def metric_name(workload):
    L, d, nh, hd, f, S, B, lin_bias, alibi = WORKLOADS[workload]
    size = workload.split("-")[1].upper()
    return f"fwd+bwd model TFLOPs on 1 MI355X, {size} ctx{S} bs{B}; % of fp16 MFMA peak"


def layout_name(la, lb):
    return {(0, 1): "X.W (A k-contiguous, B k-strided)", (0, 0): "dY.W^T (both k-contiguous)",
            (1, 1): "X^T.dY (both k-strided)", (1, 0): "A k-strided, B k-contiguous"}[(la, lb)]


def gemm_table(by_shape, reps, workload, dtype_name):
    """Markdown table of the instrumented GEMM calls: one row per distinct call, HIP-event time per call."""
    rows = []
    for key, (cnt, ms) in by_shape.items():
        if key[0] == "group":
            probs = key[1:]
            flop = sum(2.0 * m * n * k for m, n, k in probs)
            what = "grouped dW: " + " + ".join(f"{m}x{n}x{k}" for m, n, k in probs)
            layout = layout_name(1, 1)
        elif key[0] == "bits":
            _, lb, m, n, k = key
            flop, what, layout = 2.0 * m * n * k, f"{m}x{n}x{k} (ReLU sign bits)", layout_name(0, lb)
        else:
            la, lb, m, n, k = key
            flop, what, layout = 2.0 * m * n * k, f"{m}x{n}x{k}", layout_name(la, lb)
        us = ms / cnt * 1e3
        rows.append((ms / reps, f"| {what} | {layout} | {cnt // reps} | {us:.1f} | {flop / us / 1e6:.0f} | {ms / reps:.3f} |"))
    rows.sort(key=lambda r: -r[0])
    head = [f"# GEMM calls of one step by shape ({workload}, {dtype_name})", "",
            "Command (on the MI355X box, from the repository root):", "",
            f"    python3 bench.py --workload {workload} --dtype {dtype_name} --no-cpu-baseline --no-extras --gemm-table gpurun_out/gemm_table.md",
            "", "M x N x K of `C[M,N] = sum_k A(m,k) B(n,k)`; time = HIP events on the launch stream around the call "
            f"(its GEMM kernel or kernels and, for a split contraction, the reduce pass), mean over {reps} instrumented steps.", "",
            "| product (M x N x K) | operand layout | calls / step | us / call | TFLOP/s | ms / step |", "|---|---|---:|---:|---:|---:|"]
    return "\n".join(head + [r[1] for r in rows]) + "\n"


def _attn_flop(fwd):
    # args: stream, dtype, B, nh, S, hd, ...; causal: 2 (forward) or 5 (backward) products at half cost
    return lambda a: (2.0 if fwd else 5.0) * a[2] * a[3] * a[4] * a[4] * a[5]


# C-ABI entry point -> (kernel family, algorithmic FLOPs or HBM bytes of one call).  Bytes: every operand
# and result of the call once, 2 bytes per element (fp32 statistics and parameter vectors left out):
# LayerNorm forward reads x, writes y; its backward reads dy, x, writes dx; the residual forms read and
# write one more stream each; cross-entropy forward + gradient reads the logits and writes their gradient.
FAMILY_ENTRY_POINTS = {
    "tf_attn_fwd": ("attention", _attn_flop(True)),
    "tf_attn_bwd": ("attention", _attn_flop(False)),
    "tf_attn_alibi_fwd": ("attention", _attn_flop(True)),
    "tf_attn_alibi_bwd": ("attention", _attn_flop(False)),
    "tf_layernorm_fwd": ("layernorm", lambda a: 4.0 * a[3] * a[4]),
    "tf_layernorm_bwd": ("layernorm", lambda a: 6.0 * a[3] * a[4]),
    "tf_add_layernorm_fwd": ("layernorm", lambda a: 8.0 * a[3] * a[4]),
    "tf_add_layernorm_bwd": ("layernorm", lambda a: 8.0 * a[3] * a[4]),
    # second stage of all LayerNorms of a pass at once: 512 partial rows (row passes over >= 2048 rows) of 2d fp32 each
    "tf_layernorm_param_grads": ("layernorm", lambda a: 512.0 * 2 * a[2] * 4 * a[3]),
    "tf_cross_entropy_fwd": ("cross_entropy", lambda a: 2.0 * a[2] * a[3]),
    "tf_cross_entropy_fwd_grad": ("cross_entropy", lambda a: 4.0 * a[2] * a[3]),
    "tf_cross_entropy_bwd": ("cross_entropy", lambda a: 4.0 * a[2] * a[3]),
}
FAMILY_BOUND = {"attention": ("mfma", PEAK_FP16_TFLOPS, "TFLOP/s", 1e12),
                "layernorm": ("hbm", PEAK_HBM_GBS, "GB/s", 1e9),
                "cross_entropy": ("hbm", PEAK_HBM_GBS, "GB/s", 1e9)}


def family_rooflines(by_family, reps):
    """One roofline block per kernel family, from the events of the instrumented steps."""
    out = []
    for family, (cnt, ms, work) in sorted(by_family.items()):
        bound, peak, unit, per = FAMILY_BOUND[family]
        achieved = work / (ms * 1e-3) / per
        out.append({"family": family, "bound": bound, "achieved": round(achieved, 1), "peak": peak, "unit": unit,
                    "frac": round(achieved / peak, 4), "calls_per_step": cnt // reps,
                    "avg_call_us": round(ms / cnt * 1e3, 2), "ms_per_step": round(ms / reps, 3),
                    "work_per_call": round(work / cnt, 1)})
    return out


class GemmTimer:
    """HIP events on the current (launch) stream around every tf_gemm / tf_gemm_scaled / tf_gemm_relu_bits /
    tf_gemm_group call, and around every attention, LayerNorm and cross-entropy call (`by_family`)."""

    def __init__(self, events=8192):
        self.records = []
        # events made (and recorded once, which is when torch creates the HIP event) ahead of the
        # instrumented steps: creating two per call inside them slows the host enough for the GPU
        # to catch up in the forward pass, and a call's events then also cover the idle gap
        self._pool = [torch.cuda.Event(enable_timing=True) for _ in range(events)]
        for e in self._pool:
            e.record()
        torch.cuda.synchronize()

    def _event(self):
        return self._pool.pop() if self._pool else torch.cuda.Event(enable_timing=True)

    def __enter__(self):
        from tritonformer_amd import kernels

        self._kernels = kernels
        self._orig = kernels._gemm

        def timed(dtype, la, lb, m, n, k, *rest, **kw):
            e0, e1 = self._event(), self._event()
            e0.record()
            self._orig(dtype, la, lb, m, n, k, *rest, **kw)
            e1.record()
            self.records.append(((la, lb, m, n, k), e0, e1))

        self._orig_scaled = kernels._gemm_scaled

        def timed_scaled(dtype, la, lb, m, n, k, *rest):
            e0, e1 = self._event(), self._event()
            e0.record()
            self._orig_scaled(dtype, la, lb, m, n, k, *rest)
            e1.record()
            self.records.append(((la, lb, m, n, k), e0, e1))

        self._orig_group = kernels._gemm_group

        def timed_group(dtype, out_dtype, la, lb, problems, device):
            e0, e1 = self._event(), self._event()
            e0.record()
            self._orig_group(dtype, out_dtype, la, lb, problems, device)
            e1.record()
            key = ("group",) + tuple((q.M, q.N, q.K) for q in problems)
            self.records.append((key, e0, e1))

        self._orig_bits = kernels._gemm_bits

        def timed_bits(dtype, lb, m, n, k, *rest):
            e0, e1 = self._event(), self._event()
            e0.record()
            rc = self._orig_bits(dtype, lb, m, n, k, *rest)
            e1.record()
            if rc == 0:  # a refused call launched nothing; the caller falls back to _gemm
                self.records.append((("bits", lb, m, n, k), e0, e1))
            return rc

        kernels._gemm = timed
        kernels._gemm_scaled = timed_scaled
        kernels._gemm_group = timed_group
        kernels._gemm_bits = timed_bits

        # the other kernel families: events around the C-ABI call itself (the launchers look the entry
        # point up on the library object at every call, so replacing the attribute is enough)
        self._lib = kernels.load()
        self._lib_orig = {}
        self.family_records = []
        for name, (family, work) in FAMILY_ENTRY_POINTS.items():
            orig = getattr(self._lib, name)
            self._lib_orig[name] = orig

            def timed_entry(*args, _orig=orig, _family=family, _work=work):
                e0, e1 = self._event(), self._event()
                e0.record()
                rc = _orig(*args)
                e1.record()
                if rc == 0:
                    self.family_records.append((_family, _work(args), e0, e1))
                return rc

            setattr(self._lib, name, timed_entry)
        return self

    def __exit__(self, *exc):
        self._kernels._gemm = self._orig
        self._kernels._gemm_scaled = self._orig_scaled
        self._kernels._gemm_group = self._orig_group
        self._kernels._gemm_bits = self._orig_bits
        for name, orig in self._lib_orig.items():
            setattr(self._lib, name, orig)
        torch.cuda.synchronize()
        self.by_family = {}
        for family, work, e0, e1 in self.family_records:
            cnt, tot, w = self.by_family.get(family, (0, 0.0, 0.0))
            self.by_family[family] = (cnt + 1, tot + e0.elapsed_time(e1), w + work)
        self.by_shape = {}
        for key, e0, e1 in self.records:
            ms = e0.elapsed_time(e1)
            cnt, tot = self.by_shape.get(key, (0, 0.0))
            self.by_shape[key] = (cnt + 1, tot + ms)
        return False


def cpu_baseline(name, seconds_cap=60.0):
    """fp32 oracle on the host: same B, S, d, heads, ffn, vocab; depth cut to 2 layers."""
    from oracle import ref_torch as R

    L, d, nh, hd, f, S, B, lin_bias, alibi = WORKLOADS[name]
    Ls = min(L, 2)
    cores = int(os.environ.get("OMP_NUM_THREADS", 0)) or os.cpu_count()
    cores = min(cores, os.cpu_count())
    torch.set_num_threads(cores)
    cfg = R.RefConfig(VOCAB, d, S, nh, hd, f, Ls, lin_bias, alibi)
    torch.manual_seed(0)
    model = R.RefTransformer(cfg, sdpa=True)
    model.logits_out.weight.data.normal_(0.0, 0.02)
    tokens = torch.randint(0, VOCAB, (B, S))
    flops = step_flops(Ls, d, f, S, B)
    times = []
    t_begin = time.perf_counter()
    for i in range(3):  # first pass is the warm-up
        model.zero_grad(set_to_none=True)
        t0 = time.perf_counter()
        _, loss = model(tokens, tokens)
        loss.backward()
        times.append(time.perf_counter() - t0)
        if time.perf_counter() - t_begin > seconds_cap:
            break
    best = min(times[1:]) if len(times) > 1 else times[0]
    return {
        "value": round(flops / best / 1e12, 4),
        "unit": "TFLOP/s",
        "cores": cores,
        "kind": "port",
        "sample": f"fp32 PyTorch oracle, same step with the stack cut to {Ls} of {L} layers "
                  f"(B={B}, S={S}, d={d}, vocab={VOCAB}; {flops / 1e12:.2f} TFLOP), best of {max(len(times) - 1, 1)} "
                  f"after 1 warm-up, {best:.2f} s/step",
    }


def mfma_probe(dtype, device, iters=20000):
    """TFLOP/s of 256 workgroups x 8 waves issuing nothing but the GEMM step's MFMAs, per kind of operand data."""
    from tritonformer_amd import _lib

    lib = _lib.load_diag()
    wgs = torch.cuda.get_device_properties(device).multi_processor_count
    sink = torch.empty(wgs * 512, dtype=torch.float32, device=device)
    gen = torch.Generator(device="cpu").manual_seed(0)
    kinds = {
        "all ones": torch.ones(24576),
        "uniform in [-1, 1]": torch.rand(24576, generator=gen) * 2 - 1,
        "normal, std 0.02 (weights)": torch.randn(24576, generator=gen) * 0.02,
        "normal, std 1": torch.randn(24576, generator=gen),
    }
    out = {"probe": f"v_mfma_f32_32x32x16 stream of one 256x256x64 GEMM step per trip, {wgs} workgroups x 8 waves, "
                    "no memory traffic", "dtype": str(dtype).replace("torch.", ""), "iters": iters, "tflops": {}}
    flops = lib.tf_diag_mfma_rate_flops(iters, wgs)
    for name, vals in kinds.items():
        ops = vals.to(dtype).to(device)
        stream = torch.cuda.current_stream().cuda_stream
        _lib.check(lib.tf_diag_mfma_rate(stream, _lib.dtype_code(dtype), ops.data_ptr(), 100, wgs, sink.data_ptr()))
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        _lib.check(lib.tf_diag_mfma_rate(stream, _lib.dtype_code(dtype), ops.data_ptr(), iters, wgs, sink.data_ptr()))
        e1.record()
        torch.cuda.synchronize()
        out["tflops"][name] = round(flops / (e0.elapsed_time(e1) * 1e-3) / 1e12, 1)
    return out


def vendor_compare(workload, dtype, device, path, iters=30):
    """The step's dense products, each timed alone (HIP events, `iters` back-to-back calls on random data)
    through this library and through ``torch.matmul`` (the vendor BLAS library torch is built with): a markdown table.
    Operands are given to both exactly as the training step holds them (no transposed copies are made)."""
    from tritonformer_amd import kernels as K

    L, d, nh, hd, f, S, B, lin_bias, alibi = WORKLOADS[workload]
    T = B * S
    gen = torch.Generator(device="cpu").manual_seed(0)

    def rnd(*shape, scale=1.0):
        return (torch.randn(*shape, generator=gen) * scale).to(dtype).to(device)

    def timed(fn):
        for _ in range(3):
            fn()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(iters):
            fn()
        e1.record()
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) / iters * 1e3

    rows = []
    for name, n_in, n_out in (("q/k/v projection (packed)", d, 3 * d), ("attention output projection", d, d),
                              ("MLP up", d, f), ("MLP down", f, d), ("LM head", d, VOCAB)):
        x, w, dy = rnd(1, T, n_in), rnd(n_in, n_out, scale=0.02), rnd(1, T, n_out)
        x2, dy2 = x[0], dy[0]
        flop = 2.0 * T * n_in * n_out
        out = torch.empty(T, n_out, dtype=dtype, device=device)
        out_in = torch.empty(T, n_in, dtype=dtype, device=device)
        out_w = torch.empty(n_in, n_out, dtype=dtype, device=device)
        cases = ((f"forward X.W ({T}x{n_out}x{n_in})", lambda: K.mm(x, w), lambda: torch.matmul(x2, w, out=out)),
                 (f"input gradient dY.W^T ({T}x{n_in}x{n_out})", lambda: K.mm(dy, w.T), lambda: torch.matmul(dy2, w.T, out=out_in)),
                 (f"weight gradient X^T.dY ({n_in}x{n_out}x{T})", lambda: K.mm_dw(x, dy), lambda: torch.matmul(x2.T, dy2, out=out_w)))
        for what, ours, theirs in cases:
            a, b = timed(ours), timed(theirs)
            rows.append(f"| {name} | {what} | {a:.1f} | {flop / a / 1e6:.0f} | {b:.1f} | {flop / b / 1e6:.0f} | {a / b:.2f} |")
    text = "\n".join([
        f"# Dense products of the step against the vendor BLAS library ({workload}, {str(dtype).replace('torch.', '')})", "",
        "Command (on the MI355X box, from the repository root):", "",
        f"    python3 bench.py --workload {workload} --vendor-compare gpurun_out/vendor_compare.md", "",
        f"Each product alone, {iters} back-to-back calls on N(0,1) activations / gradients and N(0,0.02) weights, HIP events around the "
        "calls (a split contraction includes its reduce pass; 16-bit results on both sides).  `torch.matmul` runs the BLAS "
        "library torch is built with (hipBLASLt / rocBLAS).  Back-to-back repeats keep the operands in the caches: both "
        "columns are faster than the same product inside the training step.", "",
        "| layer | product (M x N x K) | this library, us | TFLOP/s | vendor, us | TFLOP/s | ours / vendor |", "|---|---|---:|---:|---:|---:|---:|"] + rows) + "\n"
    with open(path, "w") as fh:
        fh.write(text)
    return {"vendor_compare": path, "products": len(rows)}


def attention_probe(workload, dtype, device, iters=20):
    """The attention kernels of one layer of ``workload`` alone (forward, dQ, dK/dV on the
    packed projection layout the model uses), ``iters`` times: what `rocprofv3 --pmc` is pointed at
    for their counters.  Returns the average time of one forward + backward."""
    import tritonformer_amd as T

    L, d, nh, hd, f, S, B, lin_bias, alibi = WORKLOADS[workload]
    gen = torch.Generator(device="cpu").manual_seed(0)
    qkv = torch.randn(B, S, 3, nh, hd, generator=gen).to(dtype).to(device).requires_grad_(True)
    grad = torch.randn(B, S, nh * hd, generator=gen).to(dtype).to(device)
    bias = None
    if alibi:
        from tritonformer_amd.transformer import get_slopes
        bias = torch.tensor(get_slopes(nh), dtype=torch.float16, device=device)

    def once():
        qkv.grad = None
        T.fast_causal_attention_qkvpacked.apply(qkv, bias).backward(grad)

    for _ in range(3):
        once()
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(iters):
        once()
    e1.record()
    torch.cuda.synchronize()
    us = e0.elapsed_time(e1) / iters * 1e3
    flop = 7.0 * B * S * S * nh * hd  # causal: 2 forward + 5 backward matrix products at half cost
    return {"probe": "attention forward + backward of one layer", "workload": workload,
            "dtype": str(dtype).replace("torch.", ""), "iters": iters, "us_per_layer": round(us, 1),
            "tflops": round(flop / us / 1e6, 1)}


def softmax_probe(device, iters=20):
    """The row softmax kernels alone (tritonformer_amd.Softmax forward and backward), HIP events around `iters`
    back-to-back calls: algorithmic bytes (forward: read x, write y; backward: read dy, y, write dx) per second
    against the HBM peak, for 16-bit and fp32 rows of attention-score and vocabulary length."""
    from tritonformer_amd import kernels as K

    rows_out = []
    for dt, name in ((torch.float16, "fp16"), (torch.bfloat16, "bf16"), (torch.float32, "fp32")):
        for cols, rows in ((2048, 65536), (50304, 4096)):
            es = 4 if dt == torch.float32 else 2
            x = torch.randn(1, rows, cols, device=device).to(dt)
            y = K.softmax_fwd(x)
            dy = torch.randn_like(y)

            def timed(fn):
                for _ in range(2):
                    fn()
                e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                e0.record()
                for _ in range(iters):
                    fn()
                e1.record()
                torch.cuda.synchronize()
                return e0.elapsed_time(e1) / iters * 1e3

            for what, us, nbytes in (("forward", timed(lambda: K.softmax_fwd(x)), 2.0 * es * rows * cols),
                                     ("backward", timed(lambda: K.softmax_bwd(dy, y)), 3.0 * es * rows * cols)):
                gbs = nbytes / us / 1e3
                rows_out.append({"pass": what, "dtype": name, "rows": rows, "cols": cols, "us": round(us, 1),
                                 "GB/s": round(gbs, 1), "frac_of_hbm_peak": round(gbs / PEAK_HBM_GBS, 3)})
            del x, y, dy
    return {"probe": "row softmax forward / backward alone", "iters": iters, "peak_GB/s": PEAK_HBM_GBS, "results": rows_out}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--workload", default="gpt2-410m-ctx2048-bs4", choices=sorted(WORKLOADS))
    ap.add_argument("--dtype", default="fp16", choices=["fp16", "bf16"])
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-roofline", action="store_true")
    ap.add_argument("--no-extras", action="store_true",
                    help="skip the loss-scaled / recast / other-workload timings that follow the headline")
    ap.add_argument("--loss-scale", type=float, default=1024.0, help="scale of the `loss_scaled` extra")
    ap.add_argument("--recast", action="store_true",
                    help="time the headline with the fp32 weights converted to 16 bits in every forward pass")
    ap.add_argument("--gemm-table", metavar="FILE", help="write the per-shape table of the instrumented GEMM calls there")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also run one plain 1 GiB streaming kernel, dst = src + 1 (known traffic: 1 GiB read, "
                         "1 GiB written) so that rocprofv3 FETCH_SIZE / WRITE_SIZE readings can be scaled")
    ap.add_argument("--mfma-probe", action="store_true",
                    help="instead of the step: sustained rate of the GEMM kernel's MFMA stream alone (no memory "
                         "traffic) for constant and for random operand values, one JSON line")
    ap.add_argument("--vendor-compare", metavar="FILE",
                    help="instead of the step: every dense product of the workload timed alone through this library and "
                         "through torch.matmul (the vendor BLAS library); writes a markdown table to FILE")
    ap.add_argument("--softmax-probe", action="store_true",
                    help="instead of the step: the row softmax kernels alone (16-bit and fp32 rows of 2048 and 50304 "
                         "columns), GB/s against the HBM peak, one JSON line")
    ap.add_argument("--attention-probe", action="store_true",
                    help="instead of the step: the attention kernels of one layer of the workload alone, one JSON line")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build runs on ONE GPU; --gpus N with N > 1 is not supported "
                 "(no collectives are part of it)")
    if not torch.cuda.is_available():
        sys.exit("bench.py: needs an MI355X (no CPU path exists for the kernels)")

    dtype = torch.float16 if args.dtype == "fp16" else torch.bfloat16
    device = torch.device("cuda:0")
    if args.mfma_probe:
        print(json.dumps(mfma_probe(dtype, device)))
        return
    if args.attention_probe:
        print(json.dumps(attention_probe(args.workload, dtype, device)))
        return
    if args.softmax_probe:
        print(json.dumps(softmax_probe(device)))
        return
    if args.vendor_compare:
        print(json.dumps(vendor_compare(args.workload, dtype, device, args.vendor_compare)))
        return
    import tritonformer_amd as T

    L, d, nh, hd, f, S, B, lin_bias, alibi = WORKLOADS[args.workload]
    model, tokens = make_model(args.workload, device, dtype)
    T.set_weight_cast_cache(not args.recast)

    ms, loss = time_steps(model, tokens, args.steps, args.warmup, dtype)
    flops = step_flops(L, d, f, S, B)
    tflops = flops / (ms * 1e-3) / 1e12

    out = {
        "metric": metric_name(args.workload),
        "value": round(tflops, 2),
        "unit": "TFLOP/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms, 3),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": args.dtype,
        "data": "synthetic",
        "config": {"workload": args.workload, "layers": L, "d_model": d, "heads": nh, "head_dim": hd, "ffn": f,
                   "seq_len": S, "global_batch": B, "vocab": VOCAB, "linear_bias": lin_bias, "alibi": alibi,
                   "master_weights": "fp32", "autocast": args.dtype, "parallelism": "single GPU",
                   "protocol": "reference README.md:62-77: forward under autocast, loss.backward() unscaled, no optimizer",
                   "weight_gradients": "launched by the model's gradient queue in whole rounds of workgroups, in param.grad "
                                       "when backward() returns (`weight_gradients_in_layer` has the in-layer launches)",
                   "weight_casts": "every forward pass" if args.recast else
                                   "16-bit copies of the unchanged fp32 weights kept between steps (keyed on the "
                                   "parameters' version counters); `recast_each_step` has the other mode"},
        "pct_of_fp16_mfma_peak": round(100.0 * tflops / PEAK_FP16_TFLOPS, 2),
        "tokens_per_s": round(B * S / (ms * 1e-3), 1),
        "step_tflop": round(flops / 1e12, 3),
        "loss": round(loss, 4),
    }

    if not args.no_roofline:
        reps = max(1, min(args.steps, 5))
        from tritonformer_amd import _lib

        gt = GemmTimer()
        # plain steps ahead of the instrumented ones, not synchronised: the host runs several milliseconds ahead
        # of the GPU from here on, so the events of a call bracket its kernels and not the host's launch latency
        run_steps(model, tokens, 3, dtype)
        count0 = _lib.load_diag().tf_diag_gemm_launch_count()
        with gt:
            run_steps(model, tokens, reps, dtype)
        calls = sum(c for c, _ in gt.by_shape.values())
        launches = _lib.load_diag().tf_diag_gemm_launch_count() - count0  # kernels: a product cut along N is two
        total_ms = sum(t for _, t in gt.by_shape.values())
        gflops = gemm_flops(L, d, f, S, B) * reps
        achieved = gflops / (total_ms * 1e-3) / 1e12
        out["roofline"] = {
            "bound": "mfma",
            "kernel": "tfa::gemm_dma_kernel / gemm_dma_group_kernel (all instantiations; fwd X.W, dX = dY.W^T, dW = X^T.dY)",
            "achieved": round(achieved, 2),
            "peak": PEAK_FP16_TFLOPS,
            "unit": "TFLOP/s",
            "frac": round(achieved / PEAK_FP16_TFLOPS, 4),
            "traffic": GEMM_TRAFFIC_BYTES_PER_LAUNCH.get(args.workload),
            "launches_per_step": launches // reps,
            "calls_per_step": calls // reps,
            "flop_per_launch": round(gflops / launches, 1),
            "avg_launch_us": round(total_ms / launches * 1e3, 2),
            "gemm_ms_per_step": round(total_ms / reps, 3),
            "measured": f"HIP events on the launch stream around each tf_gemm / tf_gemm_scaled / tf_gemm_relu_bits / tf_gemm_group call, {reps} instrumented steps "
                        "run after the timed ones (queued behind three plain steps so that the GPU never waits for the host); the event time of a call covers its GEMM kernel(s) and, for a split contraction, "
                        "the reduce kernel; launches = GEMM kernels counted by the library",
        }
        out["roofline"]["other_kernels"] = family_rooflines(gt.by_family, reps)
        out["roofline"]["other_kernels_measured"] = (
            "same instrumented steps: HIP events around every tf_attn_* / tf_*layernorm_* / tf_cross_entropy_* call; "
            "attention: 2 (forward) + 5 (backward) causal tile products; LayerNorm and cross-entropy: operand and result "
            "bytes of the call, each once, against 8 TB/s")
        if args.gemm_table:
            with open(args.gemm_table, "w") as fh:
                fh.write(gemm_table(gt.by_shape, reps, args.workload, args.dtype))
    if not args.no_extras:
        k, w = max(3, args.steps // 2), 2
        ms_s, loss_s = time_steps(model, tokens, k, w, dtype, loss_scale=args.loss_scale)
        out["loss_scaled"] = {"scale": args.loss_scale, "ms_per_step": round(ms_s, 3), "steps": k,
                              "value": round(flops / (ms_s * 1e-3) / 1e12, 2), "loss": round(loss_s, 4)}
        if not args.recast:
            T.set_weight_cast_cache(False)
            ms_r, _ = time_steps(model, tokens, k, w, dtype)
            out["recast_each_step"] = {"ms_per_step": round(ms_r, 3), "steps": k,
                                       "value": round(flops / (ms_r * 1e-3) / 1e12, 2)}
            # what a real training step pays, both at once: loss scaled (real data in the backward GEMMs)
            # AND the fp32 weights converted in every forward pass (an optimizer changes them every step)
            ms_t, loss_t = time_steps(model, tokens, k, w, dtype, loss_scale=args.loss_scale)
            out["training_regime"] = {"loss_scale": args.loss_scale, "weight_casts": "every forward pass",
                                      "ms_per_step": round(ms_t, 3), "steps": k,
                                      "value": round(flops / (ms_t * 1e-3) / 1e12, 2),
                                      "pct_of_fp16_mfma_peak": round(100.0 * flops / (ms_t * 1e-3) / 1e12 / PEAK_FP16_TFLOPS, 2),
                                      "loss": round(loss_t, 4)}
            T.set_weight_cast_cache(True)
        # the reference's graph node for node: every model-level fusion off, so that the step runs through the
        # reference-named Functions only (LinearNoBias x 4 + LinearNoBiasReLU per block, CausalAttention,
        # LayerNorm, `residual + hidden`, nn.Embedding, logits + CrossEntropyLoss); headline protocol otherwise
        import tritonformer_amd.transformer as TM
        # the headline graph with every weight gradient launched inside its layer's backward (no queue across layers)
        TM.DEFER_DW = False
        try:
            ms_i, loss_i = time_steps(model, tokens, k, w, dtype)
        finally:
            TM.DEFER_DW = True
        out["weight_gradients_in_layer"] = {"ms_per_step": round(ms_i, 3), "steps": k,
                                            "value": round(flops / (ms_i * 1e-3) / 1e12, 2), "loss": round(loss_i, 4)}
        flags = ("FUSE_QKV", "FUSE_MLP", "FUSE_ATTN_BLOCK", "FUSE_ADD_LN", "FUSE_EMBED", "FUSE_HEAD")
        saved = {n: getattr(TM, n) for n in flags}
        try:
            for n in flags:
                setattr(TM, n, False)
            ms_d, loss_d = time_steps(model, tokens, k, w, dtype)
            # ... and with every weight gradient launched where the reference launches it, inside its layer's backward
            TM.DEFER_DW = False
            ms_dl, _ = time_steps(model, tokens, k, w, dtype)
        finally:
            TM.DEFER_DW = True
            for n, v in saved.items():
                setattr(TM, n, v)
        out["drop_in_graph"] = {"fusions": "all off (" + ", ".join(flags) + "); weight and LayerNorm-parameter gradients "
                                           "through the gradient queue (DEFER_DW, a launch schedule, not a graph change)",
                                "ms_per_step": round(ms_d, 3), "steps": k,
                                "value": round(flops / (ms_d * 1e-3) / 1e12, 2),
                                "pct_of_fp16_mfma_peak": round(100.0 * flops / (ms_d * 1e-3) / 1e12 / PEAK_FP16_TFLOPS, 2),
                                "loss": round(loss_d, 4),
                                "ms_per_step_weight_gradients_in_layer": round(ms_dl, 3)}
        del model
        others = []
        for name, dts in (("gpt2-160m-ctx2048-bs8", ["fp16"]), ("gpt2-410m-ctx2048-bs4", ["fp16"]),
                          ("gpt2-840m-alibi-ctx4096-bs1", ["fp16"]), ("gpt2-1.4b-ctx2048-bs2", ["fp16", "bf16"])):
            if name == args.workload:
                continue
            torch.cuda.empty_cache()
            m2, tok2 = make_model(name, device, dtype)
            L2, d2, _, _, f2, S2, B2, _, _ = WORKLOADS[name]
            for dn in dts:
                T.clear_weight_cast_cache()
                ms2, loss2 = time_steps(m2, tok2, 5, 2, torch.float16 if dn == "fp16" else torch.bfloat16)
                fl2 = step_flops(L2, d2, f2, S2, B2)
                others.append({"workload": name, "dtype": dn, "ms_per_step": round(ms2, 3), "steps": 5,
                               "value": round(fl2 / (ms2 * 1e-3) / 1e12, 2),
                               "pct_of_fp16_mfma_peak": round(100.0 * fl2 / (ms2 * 1e-3) / 1e12 / PEAK_FP16_TFLOPS, 2),
                               "loss": round(loss2, 4)})
            del m2, tok2
        T.clear_weight_cast_cache()
        torch.cuda.empty_cache()
        out["workloads"] = others
    if args.calibrate_copy:
        src = torch.empty(1 << 28, dtype=torch.float32, device=device).normal_()
        dst = torch.empty_like(src)
        torch.add(src, 1.0, out=dst)  # one elementwise kernel: reads 1 GiB, writes 1 GiB
        torch.cuda.synchronize()
    if not args.no_cpu_baseline:
        out["cpu_baseline"] = cpu_baseline(args.workload)
    print(json.dumps(out))


if __name__ == "__main__":
    main()
