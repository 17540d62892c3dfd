"""ctypes binding of libptj.so (see include/ptj.h for the contract of each symbol).

The library is the only compute path: if it is missing or a call fails, a Python
exception is raised -- there is no fallback.
"""
import ctypes
import os

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libptj.so")

PTJ_F32, PTJ_BF16 = 0, 1
EPI_NONE, EPI_BIAS, EPI_BIAS_GELU, EPI_BIAS_GELU_DERIV, EPI_ACCUMULATE = 0, 1, 2, 3, 4

_c = ctypes
_p, _i64, _int, _sz = _c.c_void_p, _c.c_int64, _c.c_int, _c.c_size_t

# name -> (restype, argtypes); mirrors include/ptj.h declaration by declaration.
SIGNATURES = {
    "ptj_version": (_int, []),
    "ptj_last_error": (_c.c_char_p, []),
    "ptj_init": (_int, []),
    "ptj_layernorm_fwd": (_int, [_p, _p, _p, _p, _i64, _i64, _i64, _i64, _int, _p]),
    "ptj_layernorm_bwd_workspace_bytes": (_sz, [_i64, _i64]),
    "ptj_layernorm_bwd": (_int, [_p, _p, _p, _p, _p, _p, _p, _p, _sz, _i64, _i64, _i64, _i64, _i64, _int, _p]),
    "ptj_layernorm_bwd_dropout": (_int, [_p, _p, _p, _p, _p, _p, _p, _p, _p, _int, _i64, _p, _p, _sz, _i64, _i64, _i64, _i64, _i64,
                                         _int, _p]),
    "ptj_colsum_workspace_bytes": (_sz, [_i64, _i64]),
    "ptj_colsum": (_int, [_p, _p, _p, _sz, _i64, _i64, _i64, _int, _p]),
    "ptj_colsum_static": (_int, [_p, _p, _i64, _i64, _i64, _int, _p]),
    "ptj_gelu_fwd": (_int, [_p, _p, _i64, _int, _p]),
    "ptj_gelu_bwd": (_int, [_p, _p, _p, _i64, _int, _p]),
    "ptj_gelu_bwd_colsum": (_int, [_p, _p, _p, _p, _p, _sz, _i64, _i64, _int, _p]),
    "ptj_dropout": (_int, [_p, _p, _i64, _i64, _i64, _i64, _int, _i64, _int, _p]),
    "ptj_dropout_add": (_int, [_p, _p, _p, _i64, _i64, _int, _i64, _int, _p]),
    "ptj_dropout_add_keep": (_int, [_p, _p, _p, _p, _i64, _i64, _int, _i64, _int, _p]),
    "ptj_embed_fwd": (_int, [_p, _p, _p, _p, _i64, _i64, _i64, _i64, _c.c_float, _int, _i64, _int, _p]),
    "ptj_embed_bwd": (_int, [_p, _p, _p, _p, _i64, _i64, _i64, _c.c_float, _int, _p]),
    "ptj_dropout_add_layernorm": (_int, [_p, _p, _p, _p, _p, _p, _p, _i64, _i64, _int, _i64, _int, _p]),
    "ptj_log_softmax_fwd": (_int, [_p, _p, _i64, _i64, _i64, _i64, _int, _p]),
    "ptj_log_softmax_bwd": (_int, [_p, _p, _p, _i64, _i64, _i64, _i64, _i64, _int, _p]),
    "ptj_ce_workspace_bytes": (_sz, [_i64]),
    "ptj_ce_fwd_bwd": (_int, [_p, _p, _p, _p, _p, _p, _p, _sz, _i64, _i64, _i64, _i64, _int, _p]),
    "ptj_ce_colsum_workspace_bytes": (_sz, [_i64, _i64]),
    "ptj_ce_fwd_bwd_colsum": (_int, [_p, _p, _p, _p, _p, _p, _p, _p, _sz, _i64, _i64, _i64, _i64, _int, _p]),
    "ptj_ce_fwd_bwd_colsum_rows": (_int, [_p, _p, _p, _p, _p, _p, _p, _p, _sz, _i64, _i64, _i64, _i64, _i64, _i64, _int, _p]),
    "ptj_gemm_workspace_bytes": (_sz, [_i64, _i64, _i64, _int]),
    "ptj_gemm_mul_colsum_workspace_bytes": (_sz, [_i64, _i64]),
    "ptj_gemm_mul_colsum": (_int, [_p, _p, _p, _p, _p, _i64, _i64, _i64, _i64, _i64, _i64, _i64, _i64, _i64, _p, _sz, _int,
                                   _p]),
    "ptj_gemm": (_int, [_p, _p, _p, _p, _i64, _i64, _i64, _i64, _i64, _i64, _i64, _i64, _int, _p, _i64, _p, _sz, _int,
                        _p]),
    "ptj_adamw": (_int, [_p, _p, _p, _p, _p, _i64, _c.c_float, _c.c_float, _c.c_float, _c.c_float, _c.c_float, _i64,
                         _int, _int, _p]),
    "ptj_adamw_multi": (_int, [_i64, _p, _p, _p, _p, _p, _p, _p, _c.c_float, _c.c_float, _c.c_float, _c.c_float, _i64,
                               _int, _int, _p]),
    "ptj_attn_workspace_bytes": (_sz, [_i64, _i64, _i64]),
    "ptj_attn_packed_mask_bytes": (_sz, [_i64, _i64]),
    "ptj_attn_pack_mask": (_int, [_p, _p, _i64, _i64, _p]),
    "ptj_attn_fwd": (_int, [_p, _p, _p, _p, _p, _p, _p, _p, _sz] + [_i64] * 16 + [_int, _i64, _int, _p]),
    "ptj_attn_bwd": (_int, [_p] * 11 + [_p, _sz] + [_i64] * 28 + [_int, _i64, _int, _p]),
}

_lib = None


class PtjError(RuntimeError):
    pass


def lib():
    """The loaded library; raises if libptj.so has not been built."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise PtjError("libptj.so not found at %s: build it with `python pre-tjax_amd/build.py` "
                           "(there is no fallback path)" % LIB_PATH)
        l = ctypes.CDLL(LIB_PATH)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(l, name)
            fn.restype = res
            fn.argtypes = args
        _lib = l
    return _lib


def check(rc, what):
    if rc != 0:
        raise PtjError("%s failed (%d): %s" % (what, rc, lib().ptj_last_error().decode()))


def dtype_code(t):
    if t.dtype == torch.float32:
        return PTJ_F32
    if t.dtype == torch.bfloat16:
        return PTJ_BF16
    raise PtjError("unsupported dtype %s (fp32 and bf16 only)" % t.dtype)


def ptr(t):
    return None if t is None else t.data_ptr()


def stream():
    return torch.cuda.current_stream().cuda_stream


def require_gpu(*tensors):
    for t in tensors:
        if t is not None and not t.is_cuda:
            raise PtjError("libptj kernels need GPU tensors; got a %s tensor (no CPU fallback)" % t.device)
