"""ctypes binding of libtritonformer_amd.so (the C ABI in include/tritonformer_amd.h).

The HIP library is the only execution path of this package: if it cannot be
loaded the import of any operator raises, there is no PyTorch/CPU fallback.
"""
import ctypes
import os

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libtritonformer_amd.so")

TF_F16, TF_BF16, TF_F32 = 0, 1, 2
KMAJOR, KMINOR = 0, 1

_c = ctypes
_vp, _i, _i64, _f = _c.c_void_p, _c.c_int, _c.c_int64, _c.c_float

# name -> (restype, argtypes); mirrors include/tritonformer_amd.h one to one
SIGNATURES = {
    "tf_status_string": (_c.c_char_p, [_i]),
    "tf_version": (_i, []),
    "tf_source_hash": (_c.c_char_p, []),
    "tf_device_info": (_i, [_vp, _vp]),
    "tf_gemm": (_i, [_vp, _i, _i, _i, _i64, _i64, _i64, _vp, _i64, _vp, _i64, _vp, _i64, _vp, _i, _vp, _i64]),
    "tf_gemm_out": (_i, [_vp, _i, _i, _i, _i, _i64, _i64, _i64, _vp, _i64, _vp, _i64, _vp, _i64, _vp, _i, _vp, _i64,
                         _vp, _i64]),
    "tf_gemm_out_chunked": (_i, [_vp, _i, _i, _i, _i, _i64, _i64, _i64, _vp, _i64, _vp, _i64, _vp, _i64, _i64, _i64,
                                 _vp, _i, _vp, _i64, _vp, _i64]),
    "tf_gemm_relu_bits": (_i, [_vp, _i, _i, _i, _i, _i64, _i64, _i64, _vp, _i64, _vp, _i64, _vp, _i64, _vp, _vp, _vp,
                               _i64]),
    "tf_gemm_scaled": (_i, [_vp, _i, _i, _i, _i, _i64, _i64, _i64, _vp, _i64, _vp, _i64, _vp, _i64, _vp, _vp, _i64]),
    "tf_cast_pack": (_i, [_vp, _i, _i, _i, _i64, _i64, _vp, _i64, _vp, _i64]),
    "tf_embedding_fwd": (_i, [_vp, _i, _i, _i64, _i64, _i64, _i64, _i64, _vp, _vp, _i64, _vp, _i64, _vp, _i64]),
    "tf_embedding_bwd_workspace_bytes": (_i64, [_i64]),
    "tf_embedding_bwd": (_i, [_vp, _i, _i, _i64, _i64, _i64, _i64, _i64, _vp, _vp, _i64, _vp, _i64, _vp, _i64, _vp, _i64]),
    "tf_adamw_step": (_i, [_vp, _i, _i, _vp, _f, _f, _f, _f, _f, _i64]),
    "tf_gemm_group": (_i, [_vp, _i, _i, _i, _i, _i, _vp, _vp, _i64]),
    "tf_gemm_group_workspace_bytes": (_i64, [_i, _i, _i, _vp]),
    "tf_gemm_workspace_bytes": (_i64, [_i, _i, _i64, _i64, _i64]),
    "tf_attn_fwd": (_i, [_vp, _i, _i64, _i64, _i64, _i64, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _i64, _i64,
                         _vp, _vp, _i64, _i64, _f]),
    "tf_attn_bwd": (_i, [_vp, _i, _i64, _i64, _i64, _i64, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64,
                         _i64, _i64, _i64, _vp, _vp, _vp, _i64, _i64, _f]),
    "tf_attn_alibi_fwd": (_i, [_vp, _i, _i64, _i64, _i64, _i64, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _i64, _i64,
                               _vp, _vp, _f]),
    "tf_attn_alibi_bwd": (_i, [_vp, _i, _i64, _i64, _i64, _i64, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i64, _i64,
                               _i64, _i64, _i64, _i64, _vp, _vp, _vp, _f]),
    "tf_layernorm_fwd": (_i, [_vp, _i, _i, _i64, _i64, _vp, _i64, _vp, _vp, _f, _vp, _i64, _vp, _vp]),
    "tf_layernorm_bwd": (_i, [_vp, _i, _i, _i64, _i64, _vp, _i64, _vp, _i64, _vp, _vp, _vp, _vp, _i64, _vp, _vp, _vp,
                              _i64]),
    "tf_layernorm_bwd_partial_bytes": (_i64, [_i64, _i64]),
    "tf_layernorm_bwd_parts": (_i64, [_i64]),
    "tf_layernorm_param_grads": (_i, [_vp, _i, _i64, _i, _vp]),
    "tf_add_layernorm_fwd": (_i, [_vp, _i, _i, _i64, _i64, _vp, _i64, _vp, _i64, _vp, _i64, _vp, _vp, _f, _vp, _i64,
                                  _vp, _vp]),
    "tf_add_layernorm_bwd": (_i, [_vp, _i, _i, _i64, _i64, _vp, _i64, _vp, _i64, _vp, _i64, _vp, _vp, _vp, _vp, _i64,
                                  _vp, _vp, _vp, _i64]),
    "tf_softmax_fwd": (_i, [_vp, _i, _i64, _i64, _vp, _i64, _vp, _i64]),
    "tf_softmax_bwd": (_i, [_vp, _i, _i64, _i64, _vp, _i64, _vp, _i64, _vp, _i64]),
    "tf_cross_entropy_fwd": (_i, [_vp, _i, _i64, _i64, _vp, _i64, _i64, _i64, _vp, _vp, _vp]),
    "tf_cross_entropy_fwd_grad": (_i, [_vp, _i, _i64, _i64, _vp, _i64, _i64, _i64, _vp, _vp, _vp, _vp, _i64, _i64, _f,
                                       _vp]),
    "tf_cross_entropy_bwd": (_i, [_vp, _i, _i64, _i64, _vp, _i64, _i64, _i64, _vp, _vp, _vp, _i64, _vp, _i64, _i64]),
    "tf_colsum": (_i, [_vp, _i, _i, _i64, _i64, _vp, _i64, _vp, _vp, _i64]),
    "tf_colsum_partial_bytes": (_i64, [_i64, _i64]),
    "tf_colsum_noalloc": (_i, [_vp, _i, _i, _i64, _i64, _vp, _i64, _vp]),
    "tf_colsum_noalloc_max_partial_bytes": (_i64, []),
    "tf_relu_mask": (_i, [_vp, _i, _i64, _i64, _vp, _i64, _vp, _i64, _vp, _i64]),
}

# include/tritonformer_amd_diag.h: name -> (library, restype, argtypes)
DIAG_SIGNATURES = {
    "tf_diag_gemm": ("main", _i, [_vp, _i, _i, _i, _i, _i, _i, _i, _i64, _i64, _i64, _vp, _i64, _vp, _i64, _vp, _i64,
                                  _vp, _i, _vp, _i64]),
    "tf_diag_gemm_workspace_bytes": ("main", _i64, [_i, _i, _i64, _i64, _i64]),
    "tf_diag_gemm_launch_count": ("main", _i64, []),
    "tf_diag_mfma_rate": ("diag", _i, [_vp, _i, _vp, _i, _i, _vp]),
    "tf_diag_mfma_rate_flops": ("diag", _i64, [_i, _i]),
}


class AdamTensor(ctypes.Structure):
    """tf_adamw_tensor of the C header."""
    _fields_ = [("param", ctypes.c_void_p), ("grad", ctypes.c_void_p), ("exp_avg", ctypes.c_void_p),
                ("exp_avg_sq", ctypes.c_void_p), ("shadow", ctypes.c_void_p), ("count", ctypes.c_int64)]


class GemmProblem(ctypes.Structure):
    """`tf_gemm_problem` of include/tritonformer_amd.h."""
    _fields_ = [("M", _i64), ("N", _i64), ("K", _i64), ("A", _vp), ("lda", _i64), ("B", _vp), ("ldb", _i64),
                ("C", _vp), ("ldc", _i64), ("chunk_n", _i64), ("chunk_stride", _i64)]


class LnParamGrads(ctypes.Structure):
    """`tf_ln_param_grads` of include/tritonformer_amd.h."""
    _fields_ = [("partial", _vp), ("parts", _i64), ("dgamma", _vp), ("dbeta", _vp)]


DIAG_LIB_PATH = os.path.join(_HERE, "libtritonformer_amd_diag.so")

_lib = None
_diag = None


def load():
    """Load the shared library once; raise if it has not been built, or if it was built
    from other sources than the ones lying next to it (a stale binary proves nothing)."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise ImportError(
                f"{LIB_PATH} is missing: build it with `python -m tritonformer_amd._build` "
                "(there is no fallback path)"
            )
        lib = ctypes.CDLL(LIB_PATH)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(lib, name)
            fn.restype = res
            fn.argtypes = args
        if os.path.isdir(os.path.join(_HERE, "csrc")):
            from . import _build

            built, here = lib.tf_source_hash().decode(), _build.source_hash()
            if built != here:
                raise ImportError(
                    f"{LIB_PATH} was built from other sources (hash {built or 'none'}) than csrc/ and include/ hold "
                    f"now ({here}): rebuild it with `python -m tritonformer_amd._build`"
                )
        _lib = lib
    return _lib


class _Diag:
    """The functions of include/tritonformer_amd_diag.h, wherever they live."""


def load_diag():
    """Diagnostics (benchmark, tests, kernel work); no operator of the package calls this."""
    global _diag
    if _diag is None:
        libs = {"main": load()}
        if not os.path.exists(DIAG_LIB_PATH):
            raise ImportError(f"{DIAG_LIB_PATH} is missing: build it with `python -m tritonformer_amd._build`")
        libs["diag"] = ctypes.CDLL(DIAG_LIB_PATH)
        d = _Diag()
        for name, (where, res, args) in DIAG_SIGNATURES.items():
            fn = getattr(libs[where], name)
            fn.restype = res
            fn.argtypes = args
            setattr(d, name, fn)
        _diag = d
    return _diag


class TritonformerAmdError(RuntimeError):
    pass


def check(status):
    if status != 0:
        msg = load().tf_status_string(status).decode()
        if status in (-1, -3, -4):
            raise ValueError(f"tritonformer_amd: {msg}")
        if status == -2:
            raise TypeError(f"tritonformer_amd: {msg}")
        raise TritonformerAmdError(f"tritonformer_amd: {msg}")


def dtype_code(t):
    if t == torch.float16:
        return TF_F16
    if t == torch.bfloat16:
        return TF_BF16
    if t == torch.float32:
        return TF_F32
    raise TypeError(f"tritonformer_amd: unsupported dtype {t}")


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)
_raw_device = getattr(torch._C, "_cuda_getDevice", None)


def stream_ptr():
    """The current stream of the current device as a `hipStream_t` value (the raw query where torch has
    one: a tenth of the cost of building a `torch.cuda.Stream` object per launch)."""
    if _raw_stream is not None and _raw_device is not None:
        return _raw_stream(_raw_device())
    return torch.cuda.current_stream().cuda_stream


def require_cuda(*tensors):
    for t in tensors:
        if t is not None and not t.is_cuda:
            raise ValueError("tritonformer_amd kernels need tensors on the GPU (there is no CPU path)")
