"""C-ABI library: loads, exports every symbol include/tritonformer_amd.h declares,
and rejects bad arguments on the host before anything is launched (so these run
without a GPU).  Mirrors the reference's Python asserts (kernels/gemm.py:370-377,
kernels/attention.py:181-183, 567-570, kernels/biased_attention.py:199-207,
kernels/layernorm.py:68-71) as status codes."""
import ctypes
import os
import re

import pytest

from tritonformer_amd import _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "tritonformer_amd.h")
DIAG_HEADER = os.path.join(ROOT, "include", "tritonformer_amd_diag.h")


def declared_functions(header=HEADER):
    text = open(header).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(tf_[a-z0-9_]+)\s*\(", text)))


def test_header_declares_the_expected_surface():
    names = declared_functions()
    for must in ["tf_gemm", "tf_attn_fwd", "tf_attn_bwd", "tf_layernorm_fwd", "tf_layernorm_bwd", "tf_add_layernorm_fwd",
                 "tf_add_layernorm_bwd", "tf_softmax_fwd",
                 "tf_softmax_bwd", "tf_cross_entropy_fwd", "tf_cross_entropy_bwd", "tf_colsum", "tf_relu_mask",
                 "tf_status_string", "tf_version"]:
        assert must in names


def test_library_exports_every_declared_symbol():
    lib = ctypes.CDLL(_lib.LIB_PATH)
    for name in declared_functions():
        assert hasattr(lib, name), f"{name} declared in the header but not exported"


def test_binding_table_matches_header():
    assert sorted(_lib.SIGNATURES) == declared_functions()


def test_diagnostics_are_declared_apart_and_exported():
    """Diagnostics have a header of their own; the product header names none of them, the two
    libraries export what that header declares, and the binding table mirrors it."""
    names = declared_functions(DIAG_HEADER)
    assert names and all(n.startswith("tf_diag_") for n in names)
    assert not [n for n in declared_functions() if "diag" in n or "probe" in n or "tune" in n or "debug" in n]
    assert sorted(_lib.DIAG_SIGNATURES) == names
    libs = {"main": ctypes.CDLL(_lib.LIB_PATH), "diag": ctypes.CDLL(_lib.DIAG_LIB_PATH)}
    for name, (where, _, _) in _lib.DIAG_SIGNATURES.items():
        assert hasattr(libs[where], name), f"{name} not exported by the {where} library"


def test_library_reads_no_environment_and_reports_its_sources():
    """No getenv in the product sources (tile choice cannot be switched from outside the call), and
    the binary carries the hash of the sources it was built from."""
    from tritonformer_amd import _build

    csrc = os.path.join(ROOT, "tritonformer_amd", "csrc")
    for f in os.listdir(csrc):
        if f.endswith((".hip", ".h")):
            assert "getenv" not in open(os.path.join(csrc, f)).read(), f
    assert _lib.load().tf_source_hash().decode() == _build.source_hash()


def test_device_info_has_a_fallback_without_a_gpu():
    lib = _lib.load()
    cus, xcds = ctypes.c_int(0), ctypes.c_int(0)
    assert lib.tf_device_info(ctypes.byref(cus), ctypes.byref(xcds)) == 0
    assert cus.value > 0 and xcds.value > 0 and cus.value % xcds.value == 0
    assert lib.tf_device_info(None, None) == -1


def test_status_strings():
    lib = _lib.load()
    assert lib.tf_version() >= 100
    assert lib.tf_status_string(0) == b"ok"
    for code in range(-6, 0):
        assert len(lib.tf_status_string(code)) > 3


FAKE = 0x1000  # non-null, 16-byte aligned; never dereferenced because the checks fail first


def test_gemm_rejects_bad_arguments():
    lib = _lib.load()
    g = lib.tf_gemm
    ok_tail = (FAKE, 64, FAKE, 64, FAKE, 64, None, 0, None, 0)
    assert g(None, 0, 0, 1, 64, 64, 64, None, 64, FAKE, 64, FAKE, 64, None, 0, None, 0) == -1   # null A
    assert g(None, 0, 0, 1, 0, 64, 64, *ok_tail) == -1                                          # M = 0
    assert g(None, 2, 0, 1, 64, 64, 64, *ok_tail) == -2                                         # fp32 operands
    assert g(None, 0, 5, 1, 64, 64, 64, *ok_tail) == -1                                         # bad layout
    assert g(None, 0, 0, 1, 64, 64, 64, FAKE, 32, FAKE, 64, FAKE, 64, None, 0, None, 0) == -4   # lda < K
    assert g(None, 0, 0, 1, 64, 64, 64, FAKE + 1, 64, FAKE, 64, FAKE, 64, None, 0, None, 0) == -3  # odd pointer
    # a split contraction without workspace is refused, and the size query says how much is needed
    need = lib.tf_gemm_workspace_bytes(1, 1, 1024, 1024, 8192)
    assert need > 0 and need % (1024 * 1024 * 4) == 0
    assert g(None, 0, 1, 1, 1024, 1024, 8192, FAKE, 1024, FAKE, 1024, FAKE, 1024, None, 0, None, 0) == -5
    assert lib.tf_gemm_workspace_bytes(0, 1, 8192, 4096, 1024) == 0
    scaled = lambda alpha: lib.tf_gemm_scaled(None, 0, 0, 0, 1, 64, 64, 64, FAKE, 64, FAKE, 64, FAKE, 64, alpha, None, 0)
    assert scaled(None) == -1 and scaled(0x1002) == -3     # the factor is a device pointer to one aligned fp32 value
    out_tail = (FAKE, 64, FAKE, 64, FAKE, 64, None, 0, None, 0, None, 0)
    assert lib.tf_gemm_out(None, 0, 1, 0, 1, 64, 64, 64, *out_tail) == -2                       # bf16 out of fp16 in
    assert lib.tf_gemm_out(None, 0, 0, 0, 1, 64, 64, 64, FAKE, 64, FAKE, 64, FAKE, 64, None, 1, FAKE, 64,
                           None, 0) == -1                                                        # mask with ReLU
    # ReLU sign bits: exactly one of bits_out / bits_in, N a multiple of 8, rows of at least N / 8 bytes,
    # and only where the direct-to-LDS kernel runs (K a multiple of 64 among other things)
    rb = lambda n, k, out, inp, ld: lib.tf_gemm_relu_bits(None, 0, 0, 0, 1, 64, n, k, FAKE, k, FAKE, n, FAKE, n, None,
                                                          out, inp, ld)
    assert rb(64, 64, None, None, 8) == -1 and rb(64, 64, FAKE, FAKE, 8) == -1
    assert rb(60, 64, FAKE, None, 8) == -1 and rb(64, 64, FAKE, None, 7) == -1
    # a well-formed product that the bit kernel does not serve has a status of its own (TF_ESHAPE):
    # the launcher falls back to the activation as mask on that one only
    assert rb(64, 72, FAKE, None, 8) == -4 and rb(64, 72, None, FAKE, 8) == -4
    assert lib.tf_gemm_relu_bits(None, 0, 2, 0, 1, 64, 64, 64, FAKE, 64, FAKE, 64, FAKE, 64, None, FAKE, None,
                                 8) == -1                                                        # bits_out with fp32 C
    assert lib.tf_gemm_relu_bits(None, 0, 0, 0, 1, 64, 64, 64, FAKE, 64, FAKE, 64, FAKE, 64, FAKE, None, FAKE,
                                 8) == -1                                                        # bits_in with bias
    # column-block output: blocks must divide N, be multiples of 8 wide and not overlap
    def chunked(chunk_n, chunk_stride, ldc=32):
        return lib.tf_gemm_out_chunked(None, 0, 2, 1, 1, 64, 96, 64, FAKE, 64, FAKE, 96, FAKE, ldc, chunk_n,
                                       chunk_stride, None, 0, None, 0, None, 0)
    assert chunked(36, 64 * 32) == -4 and chunked(32, 63 * 32) == -4 and chunked(32, 64 * 32, ldc=24) == -4
    assert chunked(-1, 0) == -1
    import ctypes
    probs = (_lib.GemmProblem * 2)(_lib.GemmProblem(1024, 4096, 8192, FAKE, 1024, FAKE, 4096, FAKE, 4096, 0, 0),
                                   _lib.GemmProblem(4096, 1024, 8192, FAKE, 4096, FAKE, 1024, FAKE, 1024, 0, 0))
    # two 64-tile weight gradients side by side: 2 contraction slices each instead of 4
    assert lib.tf_gemm_group_workspace_bytes(1, 1, 2, probs) == 2 * 2 * 1024 * 4096 * 4
    assert lib.tf_gemm_workspace_bytes(1, 1, 1024, 4096, 8192) == 4 * 1024 * 4096 * 4
    assert lib.tf_gemm_group(None, 0, 2, 1, 1, 2, probs, None, 0) == -5
    assert lib.tf_gemm_group(None, 0, 2, 1, 1, 17, probs, FAKE, 1 << 40) == -1
    assert lib.tf_gemm_group(None, 2, 2, 1, 1, 2, probs, FAKE, 1 << 40) == -2
    assert lib.tf_gemm_group(None, 0, 1, 1, 1, 2, probs, FAKE, 1 << 40) == -2
    ptrs = (ctypes.c_void_p * 3)(FAKE, FAKE, FAKE)
    assert lib.tf_cast_pack(None, 2, 0, 5, 8, 8, ptrs, 8, FAKE, 40) == -1          # more than 4 sources
    assert lib.tf_cast_pack(None, 2, 0, 3, 8, 8, ptrs, 8, FAKE, 16) == -1          # destination rows too short
    assert lib.tf_cast_pack(None, 1, 0, 3, 8, 8, ptrs, 8, FAKE, 24) == -2          # bf16 -> fp16
    assert lib.tf_cast_pack(None, 2, 2, 3, 8, 8, ptrs, 8, FAKE, 24) == -2          # fp32 destination
    assert lib.tf_cast_pack(None, 2, 0, 3, 0, 8, ptrs, 8, FAKE, 24) == 0           # nothing to do


def test_diagnostics_reject_bad_arguments():
    d = _lib.load_diag()
    assert d.tf_diag_mfma_rate(None, 0, None, 10, 256, FAKE) == -1
    assert d.tf_diag_mfma_rate(None, 0, FAKE, 0, 256, FAKE) == -1
    assert d.tf_diag_mfma_rate(None, 0, FAKE, 10, 0, FAKE) == -1
    assert d.tf_diag_mfma_rate(None, 2, FAKE, 10, 256, FAKE) == -2
    assert d.tf_diag_mfma_rate_flops(10, 256) == 10 * 256 * 2 * 256 * 256 * 64
    g = lambda cfg, splits, flags: d.tf_diag_gemm(None, cfg, splits, flags, 0, 0, 0, 1, 64, 64, 64, None, 64, FAKE, 64,
                                                  FAKE, 64, None, 0, None, 0)
    assert g(99, 0, 0) == -1 and g(2, -1, 0) == -1 and g(2, 0, 8) == -1   # unknown cfg, negative split, refused flag bit
    assert g(2, 0, 0) == -1                                               # then the ordinary checks (null A)
    # a forced split is priced by the size query
    assert d.tf_diag_gemm_workspace_bytes(2, 4, 256, 256, 1024) == 4 * 256 * 256 * 4
    assert d.tf_diag_gemm_workspace_bytes(2, 1, 256, 256, 1024) == 0


def test_embedding_rejects_bad_arguments():
    lib = _lib.load()

    def fwd(T=8, S=4, d=16, V=10, P=4, ids=FAKE, pos=FAKE, pd=2, od=0, ld=16):
        return lib.tf_embedding_fwd(None, pd, od, T, S, d, V, P, ids, FAKE, ld, pos, ld, FAKE, ld)

    assert fwd(ids=None) == -1
    assert fwd(T=7) == -4            # not whole sequences
    assert fwd(P=3) == -4            # position table shorter than the sequence
    assert fwd(pd=0, od=1) == -2     # 16-bit tables give their own dtype only
    assert fwd(ld=8) == -1           # leading dimension shorter than a row

    def bwd(T=8, S=4, d=16, V=10, P=4, ws=FAKE, nbytes=1 << 20, gd=0, pd=2, ldt=16):
        return lib.tf_embedding_bwd(None, gd, pd, T, S, d, V, P, FAKE, FAKE, 16, FAKE, ldt, FAKE, 16, ws, nbytes)

    assert lib.tf_embedding_bwd_workspace_bytes(8) == 64 and lib.tf_embedding_bwd_workspace_bytes(0) == 0
    assert bwd(ws=None) == -5 and bwd(nbytes=63) == -5
    assert bwd(T=6) == -4
    assert bwd(ldt=32) == -1         # token gradient must be contiguous
    assert bwd(gd=0, pd=1) == -2


def test_adamw_rejects_bad_arguments():
    import ctypes

    lib = _lib.load()

    def call(count=1, step=1, beta1=0.9, lr=1e-3, shadow=None, shadow_dtype=0, grad=FAKE, param=FAKE):
        arr = (_lib.AdamTensor * 1)()
        arr[0].param, arr[0].grad, arr[0].exp_avg, arr[0].exp_avg_sq = param, grad, FAKE, FAKE
        arr[0].shadow, arr[0].count = shadow, 16
        return lib.tf_adamw_step(None, shadow_dtype, count, ctypes.cast(arr, ctypes.c_void_p), lr, beta1, 0.999, 1e-8,
                                 0.01, step)

    assert call(step=0) == -1 and call(beta1=1.0) == -1 and call(lr=-1.0) == -1 and call(grad=None) == -1
    assert call(param=0x1002) == -3            # fp32 tensors are 4-byte aligned
    assert call(shadow=FAKE, shadow_dtype=2) == -2   # a 16-bit type for the copies
    assert lib.tf_adamw_step(None, 0, 1, None, 1e-3, 0.9, 0.999, 1e-8, 0.01, 1) == -1
    assert lib.tf_adamw_step(None, 0, 0, None, 1e-3, 0.9, 0.999, 1e-8, 0.01, 1) == 0   # nothing to do


def test_attention_rejects_bad_shapes():
    lib = _lib.load()

    def fwd(S, hd, ss=None, dtype=0, bias=None, bsr=0):
        ss = ss if ss is not None else hd
        row = 2 * hd if ss == hd else ss
        return lib.tf_attn_fwd(None, dtype, 1, 2, S, hd, FAKE, FAKE, FAKE, FAKE, S * 2 * hd, hd, row, S * 2 * hd, hd,
                               2 * hd, FAKE, bias, bsr * bsr if bias else 0, bsr, 0.125)

    assert fwd(100, 64) == -4           # S % 32 != 0
    assert fwd(128, 48) == -4           # head_dim not in {32, 64, 128}
    assert fwd(128, 64, dtype=2) == -2  # fp32
    assert fwd(128, 64, ss=60) == -3    # row stride not a multiple of 8 elements
    assert fwd(128, 64, bias=FAKE, bsr=64) == -3   # bias rows shorter than S
    assert lib.tf_attn_bwd(None, 0, 1, 2, 128, 64, FAKE, FAKE, FAKE, FAKE, FAKE, FAKE, FAKE, None, 16384, 64, 128,
                           16384, 64, 128, FAKE, FAKE, None, 0, 0, 0.125) == -1  # null dv
    # closed-form ALiBi: same checks, plus the slopes pointer
    alibi = lambda S, hd, slopes: lib.tf_attn_alibi_fwd(None, 0, 1, 2, S, hd, FAKE, FAKE, FAKE, FAKE, S * 2 * hd, hd,
                                                        2 * hd, S * 2 * hd, hd, 2 * hd, FAKE, slopes, 0.125)
    assert alibi(128, 64, None) == -1 and alibi(128, 64, 0x1001) == -1
    assert alibi(100, 64, FAKE) == -4 and alibi(128, 48, FAKE) == -4
    assert lib.tf_attn_alibi_bwd(None, 0, 1, 2, 128, 64, FAKE, FAKE, FAKE, FAKE, FAKE, FAKE, FAKE, FAKE, 16384, 64, 128,
                                 16384, 64, 128, FAKE, FAKE, None, 0.125) == -1


def test_row_kernels_reject_bad_arguments():
    lib = _lib.load()
    assert lib.tf_layernorm_fwd(None, 2, 2, 4, 64, FAKE, 64, FAKE, FAKE, 1e-5, FAKE, 64, FAKE, FAKE) == -2
    assert lib.tf_layernorm_fwd(None, 0, 1, 4, 64, FAKE, 64, FAKE, FAKE, 1e-5, FAKE, 64, FAKE, FAKE) == -2   # bf16 params, fp16 x
    assert lib.tf_layernorm_fwd(None, 0, 0, 4, 64, FAKE, 32, FAKE, FAKE, 1e-5, FAKE, 64, FAKE, FAKE) == -1
    assert lib.tf_layernorm_bwd(None, 0, 0, 4, 64, FAKE, 64, FAKE, 64, FAKE, FAKE, FAKE, FAKE, 64, FAKE, FAKE,
                                None, 0) == -5
    assert lib.tf_layernorm_bwd_partial_bytes(8192, 1024) == 512 * 2 * 1024 * 4
    # the second stage by itself: dgamma and dbeta are given together or not at all; partial rows as the row pass cuts them
    assert lib.tf_layernorm_bwd(None, 0, 0, 4, 64, FAKE, 64, FAKE, 64, FAKE, FAKE, FAKE, FAKE, 64, FAKE, None,
                                FAKE, 1 << 20) == -1
    assert lib.tf_layernorm_bwd(None, 0, 0, 4, 64, FAKE, 64, FAKE, 64, FAKE, FAKE, FAKE, FAKE, 64, None, None,
                                None, 0) == -5
    assert lib.tf_layernorm_bwd_parts(8192) == 512 and lib.tf_layernorm_bwd_parts(5) == 2 and lib.tf_layernorm_bwd_parts(0) == 0
    item = (_lib.LnParamGrads * 2)(_lib.LnParamGrads(FAKE, 512, FAKE, FAKE), _lib.LnParamGrads(FAKE, 513, FAKE, FAKE))
    assert lib.tf_layernorm_param_grads(None, 2, 1024, 0, None) == 0            # nothing to do
    assert lib.tf_layernorm_param_grads(None, 2, 1024, 1, None) == -1
    assert lib.tf_layernorm_param_grads(None, 2, 1024, 2, item) == -1           # more partial rows than a row pass writes
    assert lib.tf_layernorm_param_grads(None, 3, 1024, 1, item) == -2
    assert lib.tf_layernorm_param_grads(None, 2, 0, 1, item) == -1
    # fused residual add: missing summand / sum buffer, short leading dimension, missing workspace
    assert lib.tf_add_layernorm_fwd(None, 0, 0, 4, 64, FAKE, 64, None, 64, FAKE, 64, FAKE, FAKE, 1e-5, FAKE, 64, FAKE,
                                    FAKE) == -1
    assert lib.tf_add_layernorm_fwd(None, 0, 0, 4, 64, FAKE, 64, FAKE, 32, FAKE, 64, FAKE, FAKE, 1e-5, FAKE, 64, FAKE,
                                    FAKE) == -1
    assert lib.tf_add_layernorm_fwd(None, 2, 2, 4, 64, FAKE, 64, FAKE, 64, FAKE, 64, FAKE, FAKE, 1e-5, FAKE, 64, FAKE,
                                    FAKE) == -2
    assert lib.tf_add_layernorm_bwd(None, 0, 0, 4, 64, FAKE, 64, None, 64, FAKE, 64, FAKE, FAKE, FAKE, FAKE, 64, FAKE,
                                    FAKE, FAKE, 1 << 20) == -1
    assert lib.tf_add_layernorm_bwd(None, 0, 0, 4, 64, FAKE, 64, FAKE, 64, FAKE, 64, FAKE, FAKE, FAKE, FAKE, 64, FAKE,
                                    FAKE, None, 0) == -5
    assert lib.tf_softmax_fwd(None, 0, 4, 0, FAKE, 64, FAKE, 64) == -1
    assert lib.tf_cross_entropy_fwd(None, 2, 4, 64, FAKE, 64, 0, 0, FAKE, FAKE, FAKE) == -2
    assert lib.tf_cross_entropy_bwd(None, 0, 4, 64, FAKE, 32, 0, 0, FAKE, FAKE, FAKE, 1, FAKE, 64, 0) == -1
    assert lib.tf_cross_entropy_fwd_grad(None, 0, 4, 64, FAKE, 64, 0, 0, FAKE, FAKE, FAKE, None, 64, 0, 1.0, None) == -1
    assert lib.tf_cross_entropy_fwd_grad(None, 0, 4, 64, FAKE, 64, 0, 0, FAKE, FAKE, FAKE, FAKE, 32, 0, 1.0, None) == -1
    assert lib.tf_cross_entropy_fwd_grad(None, 2, 4, 64, FAKE, 64, 0, 0, FAKE, FAKE, FAKE, FAKE, 64, 0, 1.0, None) == -2
    assert lib.tf_cross_entropy_fwd(None, 0, 6, 64, FAKE, 64, 3, 100, FAKE, FAKE, FAKE) == -1   # groups overlap
    assert lib.tf_colsum(None, 0, 0, 16, 64, FAKE, 64, FAKE, None, 0) == -5
    assert lib.tf_colsum(None, 0, 1, 16, 64, FAKE, 64, FAKE, FAKE, 1 << 20) == -2   # bf16 sums of fp16 input
    assert lib.tf_relu_mask(None, 0, 4, 64, None, 64, FAKE, 64, FAKE, 64) == -1
    # empty inputs are accepted and launch nothing
    assert lib.tf_softmax_fwd(None, 0, 0, 64, FAKE, 64, FAKE, 64) == 0
    assert lib.tf_cross_entropy_fwd(None, 0, 0, 64, FAKE, 64, 0, 0, FAKE, FAKE, FAKE) == 0
    assert lib.tf_relu_mask(None, 0, 0, 64, FAKE, 64, FAKE, 64, FAKE, 64) == 0


def test_check_maps_status_to_exceptions():
    with pytest.raises(ValueError):
        _lib.check(-4)
    with pytest.raises(_lib.TritonformerAmdError):
        _lib.check(-5)
    _lib.check(0)
