"""Operator wrappers with the reference's names and tensor signatures
(model_triton.py of martin-kukla/pre-tjax), backed by the gfx950 HIP kernels of
libptj.so instead of Triton.

Each ``*_t`` function allocates its outputs, passes raw pointers / strides to the C
ABI and returns tensors shaped like the reference's.  Launches are asynchronous on
torch's current stream; nothing here synchronises.  Inputs are never modified.
"""
import math

import torch

from . import _lib
from ._lib import check, dtype_code, lib, ptr, require_gpu, stream

DROPOUT_RATE = 0.1  # baked into the kernels, as in the reference (model_torch_func.py:2)

_ws_cache = {}


def _workspace(nbytes, device, tag):
    """Reusable scratch buffer per (device, tag); grown on demand.  Kernels that use it
    are ordered on one stream, so sharing between consecutive calls is safe."""
    key = (device, tag)
    buf = _ws_cache.get(key)
    if buf is None or buf.numel() < nbytes:
        buf = torch.empty(max(int(nbytes), 1), dtype=torch.uint8, device=device)
        _ws_cache[key] = buf
    return buf


def _rows2d(x):
    """View as [rows, cols] with unit column stride (copies only when needed)."""
    x2 = x.reshape(-1, x.shape[-1])
    if x2.stride(-1) != 1:
        x2 = x2.contiguous()
    return x2


# ----------------------------------------------------------------------------------
# log-softmax  (reference: model_triton.py:62-72, :153-164)
# ----------------------------------------------------------------------------------
def t_log_softmax_fwd_t(x: torch.Tensor):
    require_gpu(x)
    x2 = _rows2d(x)
    out = torch.empty_like(x2, memory_format=torch.contiguous_format)
    rows, cols = x2.shape
    check(lib().ptj_log_softmax_fwd(ptr(x2), ptr(out), rows, cols, x2.stride(0), out.stride(0),
                                    dtype_code(x2), stream()), "ptj_log_softmax_fwd")
    return out.reshape(x.shape)


def t_log_softmax_bkwd2_t(dloss_dx: torch.Tensor, x: torch.Tensor):
    require_gpu(dloss_dx, x)
    d2, x2 = _rows2d(dloss_dx), _rows2d(x)
    assert d2.shape == x2.shape and d2.dtype == x2.dtype
    out = torch.empty_like(x2, memory_format=torch.contiguous_format)
    rows, cols = x2.shape
    check(lib().ptj_log_softmax_bwd(ptr(d2), ptr(x2), ptr(out), rows, cols, d2.stride(0), x2.stride(0),
                                    out.stride(0), dtype_code(x2), stream()), "ptj_log_softmax_bwd")
    return out.reshape(dloss_dx.shape)


# ----------------------------------------------------------------------------------
# GELU  (reference: model_triton.py:254-260, :296-304)
# ----------------------------------------------------------------------------------
def t_gelu_fwd_t(x: torch.Tensor):
    require_gpu(x)
    xc = x.contiguous()
    out = torch.empty_like(xc)
    check(lib().ptj_gelu_fwd(ptr(xc), ptr(out), xc.numel(), dtype_code(xc), stream()), "ptj_gelu_fwd")
    return out.reshape(x.shape)


def t_gelu_bkwd2_t(dloss_dx: torch.Tensor, x: torch.Tensor):
    require_gpu(dloss_dx, x)
    assert dloss_dx.numel() == x.numel() and dloss_dx.dtype == x.dtype
    dc, xc = dloss_dx.contiguous(), x.contiguous()
    out = torch.empty_like(xc)
    check(lib().ptj_gelu_bwd(ptr(dc), ptr(xc), ptr(out), xc.numel(), dtype_code(xc), stream()), "ptj_gelu_bwd")
    return out.reshape(x.shape)


# ----------------------------------------------------------------------------------
# dropout  (reference: model_triton.py:1496-1506, :1562-1572)
# ----------------------------------------------------------------------------------
def _dropout(x, train, p_gen_aux):
    require_gpu(x)
    if train:
        assert p_gen_aux is not None, "train-mode dropout needs a seed (p_gen_aux)"
    else:
        p_gen_aux = 0
    x2 = _rows2d(x)
    out = torch.empty_like(x2, memory_format=torch.contiguous_format)
    rows, cols = x2.shape
    check(lib().ptj_dropout(ptr(x2), ptr(out), rows, cols, x2.stride(0), out.stride(0), int(bool(train)),
                            int(p_gen_aux), dtype_code(x2), stream()), "ptj_dropout")
    return out.reshape(x.shape)


def t_dropout_fwd_t(x: torch.Tensor, train=True, p_gen_aux=None):
    return _dropout(x, train, p_gen_aux)


def t_dropout_bkwd2_t(dloss_dx: torch.Tensor, x: torch.Tensor, train=True, p_gen_aux=None):
    # The mask depends on (seed, row, column) only; `x` is unused, as in the reference.
    return _dropout(dloss_dx, train, p_gen_aux)


def dropout_add_t(x: torch.Tensor, residual: torch.Tensor, train=True, p_gen_aux=None):
    """residual + dropout(x) in one pass (the `y + t_dropout_fwd_t(y_diff, ...)` of
    model_triton.py:1898 and :2069)."""
    require_gpu(x, residual)
    assert x.shape == residual.shape and x.dtype == residual.dtype
    if not train:
        p_gen_aux = 0
    xc, rc = x.contiguous(), residual.contiguous()
    out = torch.empty_like(xc)
    cols = xc.shape[-1]
    rows = xc.numel() // cols
    check(lib().ptj_dropout_add(ptr(xc), ptr(rc), ptr(out), rows, cols, int(bool(train)), int(p_gen_aux),
                                dtype_code(xc), stream()), "ptj_dropout_add")
    return out


# ----------------------------------------------------------------------------------
# LayerNorm  (reference: model_triton.py:1625-1637, :1710-1726, :1853-1867)
# ----------------------------------------------------------------------------------
def t_layernorm_fwd_t(layer_params, x: torch.Tensor):
    require_gpu(x)
    gamma, beta = layer_params[0].contiguous(), layer_params[1].contiguous()
    x2 = _rows2d(x)
    assert gamma.dtype == x2.dtype and beta.dtype == x2.dtype and gamma.numel() == x2.shape[1]
    out = torch.empty_like(x2, memory_format=torch.contiguous_format)
    rows, cols = x2.shape
    check(lib().ptj_layernorm_fwd(ptr(x2), ptr(gamma), ptr(beta), ptr(out), rows, cols, x2.stride(0), out.stride(0),
                                  dtype_code(x2), stream()), "ptj_layernorm_fwd")
    return out.reshape(x.shape)


def _layernorm_bwd(dloss_dx, layer_params, x, want_dx, want_p):
    require_gpu(dloss_dx, x)
    d2, x2 = _rows2d(dloss_dx), _rows2d(x)
    assert d2.shape == x2.shape and d2.dtype == x2.dtype
    rows, cols = x2.shape
    gamma = layer_params[0].contiguous()
    dx = torch.empty_like(x2, memory_format=torch.contiguous_format) if want_dx else None
    dg = torch.empty_like(gamma) if want_p else None
    db = torch.empty_like(gamma) if want_p else None
    ws, ws_bytes = None, 0
    if want_p:
        ws_bytes = lib().ptj_layernorm_bwd_workspace_bytes(rows, cols)
        ws = _workspace(ws_bytes, x2.device, "ln_bwd")
    check(lib().ptj_layernorm_bwd(ptr(d2), ptr(x2), ptr(gamma), ptr(dx), ptr(dg), ptr(db), ptr(ws), ws_bytes,
                                  rows, cols, d2.stride(0), x2.stride(0), dx.stride(0) if want_dx else 0,
                                  dtype_code(x2), stream()), "ptj_layernorm_bwd")
    return (dx.reshape(dloss_dx.shape) if want_dx else None), dg, db


def t_layernorm_bkwd2_p_t(dloss_dx: torch.Tensor, layer_params, x: torch.Tensor):
    _, dg, db = _layernorm_bwd(dloss_dx, layer_params, x, False, True)
    return dg, db


def t_layernorm_bkwd2_x_t(dloss_dx: torch.Tensor, layer_params, x: torch.Tensor):
    dx, _, _ = _layernorm_bwd(dloss_dx, layer_params, x, True, False)
    return dx


def layernorm_bkwd2_t(dloss_dx: torch.Tensor, layer_params, x: torch.Tensor):
    """dx, (dgamma, dbeta) from one read of dy and x (fusion of the two reference
    launches at model_triton.py:2033-2034)."""
    dx, dg, db = _layernorm_bwd(dloss_dx, layer_params, x, True, True)
    return dx, (dg, db)
