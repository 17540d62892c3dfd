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


# ----------------------------------------------------------------------------------
# GEMM  (reference: model_triton.py:373-398 t_matmul_t, :1258-1313 t_tlayer_ffn_fwd_t)
# ----------------------------------------------------------------------------------
def matmul_t(a: torch.Tensor, b: torch.Tensor, bias=None, gelu=False, out=None):
    """``out[N,M] = a[N,K] @ b[K,M] (+ bias[M]) (tanh-GELU)`` on the MFMA GEMM kernel.

    `a` and `b` are 2-D tensors with arbitrary strides (``.t()`` views are consumed in
    place, never copied); `out`, if given, is a 2-D tensor with unit column stride
    (a column slice of a wider buffer is fine)."""
    require_gpu(a, b, bias, out)
    assert a.dim() == 2 and b.dim() == 2 and a.shape[1] == b.shape[0], (a.shape, b.shape)
    assert a.dtype == b.dtype
    N, K = a.shape
    M = b.shape[1]
    if out is None:
        out = torch.empty((N, M), dtype=a.dtype, device=a.device)
    else:
        assert out.shape == (N, M) and out.dtype == a.dtype and (out.stride(1) == 1 or M == 1)
    epi = _lib.EPI_NONE
    if bias is not None:
        assert bias.dtype == a.dtype and bias.numel() == M
        bias = bias.contiguous()
        epi = _lib.EPI_BIAS_GELU if gelu else _lib.EPI_BIAS
    else:
        assert not gelu, "GELU epilogue is defined on top of the bias epilogue"
    code = dtype_code(a)
    ws_bytes = lib().ptj_gemm_workspace_bytes(N, M, K, code)
    ws = _workspace(ws_bytes, a.device, "gemm") if ws_bytes else None
    check(lib().ptj_gemm(ptr(a), ptr(b), ptr(out), ptr(bias), N, M, K, a.stride(0), a.stride(1), b.stride(0),
                         b.stride(1), out.stride(0), epi, ptr(ws), ws_bytes, code, stream()), "ptj_gemm")
    return out


def t_matmul_t(a: torch.Tensor, b: torch.Tensor):
    """Reference signature (model_triton.py:373): a[N,K] contiguous, b[K,M] any strides."""
    assert a.is_contiguous(), "Matrix A must be contiguous"
    return matmul_t(a, b)


t_matmul = t_matmul_t


def t_gelu_fwd(x):
    """Marker for `activation_fn` arguments (the reference passes its torch GELU here,
    model_triton.py:221); evaluating it runs the HIP kernel."""
    return t_gelu_fwd_t(x)


def t_tlayer_ffn_fwd_t(layer_params, x: torch.Tensor, activation_fn=t_gelu_fwd):
    """Two GEMM launches: bias+GELU epilogue, then bias (model_triton.py:1258-1313)."""
    assert activation_fn in (t_gelu_fwd, t_gelu_fwd_t), "only the tanh-GELU epilogue exists"
    w1, b1, w2, b2 = layer_params
    shape = x.shape
    x2 = _rows2d(x)
    mid = matmul_t(x2, w1.t(), b1, gelu=True)
    out = matmul_t(mid, w2.t(), b2)
    return out.view(shape[:-1] + (w2.shape[0],))


# ----------------------------------------------------------------------------------
# attention  (reference: model_triton.py:706-754 fwd3_t, :951-1003 bkwd3_t)
# ----------------------------------------------------------------------------------
_mask_cache = {}


def _mask_arg(mask, B, T):
    """None when `mask` is exactly the causal (lower-triangular) mask -- the kernel then
    masks by index -- else a contiguous uint8 [B,T,T] tensor.  The comparison reads the
    mask once per distinct tensor (one host sync) and is cached on (storage, version)."""
    if mask is None:
        return None
    assert mask.shape[-2:] == (T, T), mask.shape
    key = (mask.data_ptr(), mask._version, tuple(mask.shape), tuple(mask.stride()), mask.device)
    hit = _mask_cache.get(key)
    if hit is None:
        m = mask.expand(B, T, T) if mask.dim() == 3 else mask.reshape(1, T, T).expand(B, T, T)
        tril = torch.ones(T, T, dtype=torch.bool, device=mask.device).tril_()
        if bool((m.to(torch.bool) == tril).all()):
            hit = ("causal", None)
        else:
            hit = ("mask", m.to(torch.bool).contiguous().view(torch.uint8))
        if len(_mask_cache) > 64:
            _mask_cache.clear()
        _mask_cache[key] = hit
    return hit[1]


def _bhr(t):
    """(batch, head, row) element strides of a [B,H,T,dh] view with unit last stride."""
    assert t.stride(3) == 1, "head dimension must be contiguous"
    return t.stride(0), t.stride(1), t.stride(2)


def attn_fwd_t(q, k, v, mask, train, seed, out=None):
    """Flash-attention forward on [B,H,T,dh] *views* (any batch/head/row strides).
    Returns (O, ms[B,H,T] fp32, ls[B,H,T] fp32).  `out` may be a preallocated view."""
    require_gpu(q, k, v)
    B, H, T, dh = q.shape
    assert k.shape == q.shape and v.shape == q.shape and q.dtype == k.dtype == v.dtype
    assert T % 64 == 0, "sequence length must be a multiple of 64"
    if out is None:
        out = torch.empty((B, H, T, dh), dtype=q.dtype, device=q.device)
    ms = torch.empty((B, H, T), dtype=torch.float32, device=q.device)
    ls = torch.empty_like(ms)
    m = _mask_arg(mask, B, T)
    ws_bytes = lib().ptj_attn_workspace_bytes(B, H, T) if train else 0
    ws = _workspace(ws_bytes, q.device, "attn") if train else None
    check(lib().ptj_attn_fwd(ptr(q), ptr(k), ptr(v), ptr(m), ptr(out), ptr(ms), ptr(ls), ptr(ws), ws_bytes,
                             B, H, T, dh, *_bhr(q), *_bhr(k), *_bhr(v), *_bhr(out),
                             int(bool(train)), int(seed if train else 0), dtype_code(q), stream()), "ptj_attn_fwd")
    return out, ms, ls


def attn_bwd_t(d_o, q, k, v, o, ms, ls, mask, train, seed, out=None):
    """Flash-attention backward on [B,H,T,dh] views; returns (dq, dk, dv) (views of `out`
    = (dq, dk, dv) when given)."""
    require_gpu(d_o, q, k, v, o)
    B, H, T, dh = q.shape
    if out is None:
        out = tuple(torch.empty((B, H, T, dh), dtype=q.dtype, device=q.device) for _ in range(3))
    dq, dk, dv = out
    m = _mask_arg(mask, B, T)
    ws_bytes = lib().ptj_attn_workspace_bytes(B, H, T)
    ws = _workspace(ws_bytes, q.device, "attn")
    ms = ms.contiguous()
    ls = ls.contiguous()
    check(lib().ptj_attn_bwd(ptr(d_o), ptr(q), ptr(k), ptr(v), ptr(o), ptr(ms), ptr(ls), ptr(m), ptr(dq), ptr(dk),
                             ptr(dv), ptr(ws), ws_bytes, B, H, T, dh, *_bhr(d_o), *_bhr(q), *_bhr(k), *_bhr(v),
                             *_bhr(o), *_bhr(dq), *_bhr(dk), *_bhr(dv), int(bool(train)),
                             int(seed if train else 0), dtype_code(q), stream()), "ptj_attn_bwd")
    return dq, dk, dv


def _aligned_view(t):
    """Kernel operand requirements: 16-byte aligned base, strides multiple of 16 bytes."""
    vec = 16 // t.element_size()
    if t.stride(3) != 1 or t.data_ptr() % 16 or any(s % vec for s in t.stride()[:3]):
        return t.contiguous()
    return t


def t_scaled_dot_prod_attn_fwd3_t(qkv: torch.Tensor, mask: torch.Tensor, train=True, p_gen_aux=None):
    """qkv [B,H,3,T,dh], mask [B,T,T] bool -> (O [B,H,T,dh], [ms, ls, O])."""
    q, k, v = (_aligned_view(t) for t in torch.unbind(qkv, dim=2))
    if train:
        assert p_gen_aux is not None
    o, ms, ls = attn_fwd_t(q, k, v, mask, train, p_gen_aux)
    return o, [ms, ls, o]


def t_scaled_dot_prod_attn_bkwd3_t(dloss_dx, acts, qkv: torch.Tensor, mask: torch.Tensor, train=True, p_gen_aux=None):
    """-> (dq, dk, dv), each [B,H,T,dh]."""
    q, k, v = (_aligned_view(t) for t in torch.unbind(qkv, dim=2))
    ms, ls, o = acts
    return attn_bwd_t(_aligned_view(dloss_dx), q, k, v, _aligned_view(o), ms, ls, mask, train, p_gen_aux)
