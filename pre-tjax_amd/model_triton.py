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
# plain-torch twins of the wrappers (the reference's names without `_t`); not used below
# except `t_gelu_fwd`, which callers pass as the `activation_fn` marker
from .spec_torch import (t_dropout_bkwd2, t_dropout_fwd, t_gelu_bkwd2, t_gelu_fwd,  # noqa: F401
                         t_layernorm_bkwd2_p, t_layernorm_bkwd2_x, t_layernorm_fwd, t_linear_fwd,
                         t_log_softmax_bkwd2, t_log_softmax_fwd, t_proj_fwd, t_scaled_dot_prod_attn_bkwd3,
                         t_scaled_dot_prod_attn_fwd, t_scaled_dot_prod_attn_fwd3, t_softmax_attn_bkwd2,
                         t_softmax_attn_fwd, t_tlayer_ffn_fwd)

DROPOUT_RATE = 0.1  # baked into the kernels, as in the reference (model_torch_func.py:2)

_ws_cache = {}


def _workspace(nbytes, device, tag):
    """Reusable scratch buffer per (device, stream, tag); grown on demand.  Kernels that use
    it are ordered on one stream, so sharing between consecutive calls is safe."""
    key = (device, stream(), tag)
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


def t_gelu_bkwd2_colsum_t(dloss_dx: torch.Tensor, x: torch.Tensor):
    """GELU backward plus the column sums of its result in one pass:
    ``(t_gelu_bkwd2_t(dloss_dx, x), colsum_t(of that))`` -- dx and the gradient of the bias
    in front of the activation (model_triton.py:296-304, :426)."""
    require_gpu(dloss_dx, x)
    assert dloss_dx.shape == x.shape and dloss_dx.dtype == x.dtype
    dc, xc = _rows2d(dloss_dx).contiguous(), _rows2d(x).contiguous()
    rows, cols = xc.shape
    out = torch.empty_like(xc)
    sums = torch.empty(cols, dtype=xc.dtype, device=xc.device)
    ws_bytes = lib().ptj_colsum_workspace_bytes(rows, cols)
    ws = _workspace(ws_bytes, xc.device, "colsum")
    check(lib().ptj_gelu_bwd_colsum(ptr(dc), ptr(xc), ptr(out), ptr(sums), ptr(ws), ws_bytes, rows, cols,
                                    dtype_code(xc), stream()), "ptj_gelu_bwd_colsum")
    return out.reshape(x.shape), sums


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


def _keep_bytes_ok(t):
    """Keep bytes (one per 8 columns) exist for 2-byte element types with 8-column rows."""
    return t.element_size() == 2 and t.shape[-1] % 8 == 0 and t.data_ptr() % 16 == 0


def dropout_add_t(x: torch.Tensor, residual: torch.Tensor, train=True, p_gen_aux=None, want_keep=False):
    """residual + dropout(x) in one pass (the `y + t_dropout_fwd_t(y_diff, ...)` of
    model_triton.py:1898 and :2069).  With ``want_keep`` the result is (out, keep) where
    `keep` holds the keep mask as one byte per 8 columns (None when the mask is not
    recorded: eval mode, or a layout without keep bytes); the backward reads it instead
    of recomputing the Philox stream."""
    require_gpu(x, residual)
    assert x.shape == residual.shape and x.dtype == residual.dtype
    if not train:
        p_gen_aux = 0
    xc, rc = x.contiguous(), residual.contiguous()
    out = torch.empty_like(xc)
    cols = xc.shape[-1]
    rows = xc.numel() // cols
    if want_keep and train and _keep_bytes_ok(xc) and _keep_bytes_ok(rc):
        keep = torch.empty(rows * (cols // 8), dtype=torch.uint8, device=xc.device)
        check(lib().ptj_dropout_add_keep(ptr(xc), ptr(rc), ptr(out), ptr(keep), rows, cols, 1, int(p_gen_aux),
                                         dtype_code(xc), stream()), "ptj_dropout_add_keep")
        return out, keep
    check(lib().ptj_dropout_add(ptr(xc), ptr(rc), ptr(out), rows, cols, int(bool(train)), int(p_gen_aux),
                                dtype_code(xc), stream()), "ptj_dropout_add")
    return (out, None) if want_keep else out


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


def dropout_add_layernorm_t(x: torch.Tensor, residual: torch.Tensor, layer_params, train=True, p_gen_aux=None,
                            want_keep=False):
    """``y = residual + dropout(x)`` and ``h = layernorm(y)`` in one pass: dropout_add_t followed
    by t_layernorm_fwd_t without re-reading y (model_triton.py:1898 / :2069 then :1625-1637).
    Returns (y, h, keep) with `keep` as in dropout_add_t (None unless recorded)."""
    require_gpu(x, residual)
    assert x.shape == residual.shape and x.dtype == residual.dtype
    if not train:
        p_gen_aux = 0
    xc, rc = x.contiguous(), residual.contiguous()
    gamma, beta = layer_params[0].contiguous(), layer_params[1].contiguous()
    cols = xc.shape[-1]
    rows = xc.numel() // cols
    assert gamma.dtype == xc.dtype and beta.dtype == xc.dtype and gamma.numel() == cols
    y, h = torch.empty_like(xc), torch.empty_like(xc)
    keep = None
    if want_keep and train and _keep_bytes_ok(xc) and _keep_bytes_ok(rc):
        keep = torch.empty(rows * (cols // 8), dtype=torch.uint8, device=xc.device)
    check(lib().ptj_dropout_add_layernorm(ptr(xc), ptr(rc), ptr(gamma), ptr(beta), ptr(y), ptr(h), ptr(keep), rows, cols,
                                          int(bool(train)), int(p_gen_aux), dtype_code(xc), stream()),
          "ptj_dropout_add_layernorm")
    return y, h, keep


def _layernorm_bwd(dloss_dx, layer_params, x, want_dx, want_p, residual=None, drop=None, drop_sum=False):
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
    if residual is not None:
        assert want_dx and residual.shape == x.shape and residual.dtype == x2.dtype
        residual = residual.contiguous()
    dropped, d_train, d_seed = None, 0, 0
    keep = None
    if drop is not None:                         # (train, seed[, keep bytes]): also emit dropout_bkwd(dx)
        assert want_dx
        d_train, d_seed = int(bool(drop[0])), int(drop[1] if drop[0] else 0)
        keep = drop[2] if len(drop) > 2 and drop[0] else None
        dropped = torch.empty_like(dx)
    dsum = None
    if drop_sum:
        assert drop is not None and want_p
        dsum = torch.empty_like(gamma)
    check(lib().ptj_layernorm_bwd_dropout(ptr(d2), ptr(x2), ptr(gamma), ptr(residual), ptr(dx), ptr(dg), ptr(db),
                                          ptr(dropped), ptr(dsum), d_train, d_seed, ptr(keep), ptr(ws), ws_bytes, rows,
                                          cols, d2.stride(0), x2.stride(0), dx.stride(0) if want_dx else 0,
                                          dtype_code(x2), stream()),
          "ptj_layernorm_bwd")
    dx_out = dx.reshape(dloss_dx.shape) if want_dx else None
    if drop_sum:
        return dx_out, dg, db, dropped.reshape(dloss_dx.shape), dsum
    if drop is not None:
        return dx_out, dg, db, dropped.reshape(dloss_dx.shape)
    return dx_out, dg, db


def t_layernorm_bkwd2_p_t(dloss_dx: torch.Tensor, layer_params, x: torch.Tensor):
    _, dg, db = _layernorm_bwd(dloss_dx, layer_params, x, False, True)
    return dg, db


def t_layernorm_bkwd2_x_t(dloss_dx: torch.Tensor, layer_params, x: torch.Tensor):
    dx, _, _ = _layernorm_bwd(dloss_dx, layer_params, x, True, False)
    return dx


def layernorm_bkwd2_t(dloss_dx: torch.Tensor, layer_params, x: torch.Tensor, residual=None, drop=None,
                      drop_sum=False):
    """dx (+ residual), (dgamma, dbeta) from one read of dy and x (fusion of the two
    reference launches at model_triton.py:2033-2034 and of the residual add at :2036).
    With ``drop=(train, seed[, keep])`` a third result is t_dropout_bkwd2_t(dx, None, train,
    seed) (the dropout backward the block applies next, :2021-2024), written in the same
    pass; `keep` are the keep bytes recorded by dropout_add_t for that seed, if any.  With
    ``drop_sum=True`` a fourth result is colsum_t of that third one (the bias gradient of
    the linear layer whose output gradient it is, :426)."""
    if drop_sum:
        dx, dg, db, dropped, dsum = _layernorm_bwd(dloss_dx, layer_params, x, True, True, residual, drop, True)
        return dx, (dg, db), dropped, dsum
    if drop is not None:
        dx, dg, db, dropped = _layernorm_bwd(dloss_dx, layer_params, x, True, True, residual, drop)
        return dx, (dg, db), dropped
    dx, dg, db = _layernorm_bwd(dloss_dx, layer_params, x, True, True, residual)
    return dx, (dg, db)


def colsum_t(x: torch.Tensor, out=None):
    """Sum over all leading dimensions: the bias gradient `.sum(dim=0)` of the reference's
    t_linear_bkwd2_p (model_triton.py:426), deterministic.  `out`, if given, is a contiguous
    tensor of `cols` elements that receives the sums."""
    require_gpu(x)
    x2 = _rows2d(x)
    rows, cols = x2.shape
    if out is None:
        out = torch.empty(cols, dtype=x2.dtype, device=x2.device)
    else:
        assert out.numel() == cols and out.dtype == x2.dtype and out.is_contiguous()
    ws_bytes = lib().ptj_colsum_workspace_bytes(rows, cols)
    ws = _workspace(ws_bytes, x2.device, "colsum")
    check(lib().ptj_colsum(ptr(x2), ptr(out), ptr(ws), ws_bytes, rows, cols, x2.stride(0), dtype_code(x2), stream()),
          "ptj_colsum")
    return out


# ----------------------------------------------------------------------------------
# GEMM  (reference: model_triton.py:373-398 t_matmul_t, :1258-1313 t_tlayer_ffn_fwd_t)
# ----------------------------------------------------------------------------------
def matmul_t(a: torch.Tensor, b: torch.Tensor, bias=None, gelu=False, out=None, pre_out=None, deriv_out=None,
             accumulate=False):
    """``out[N,M] = a[N,K] @ b[K,M] (+ bias[M]) (tanh-GELU)`` on the MFMA GEMM kernel.

    `a` and `b` are 2-D tensors with arbitrary strides (``.t()`` views are consumed in
    place, never copied); `out`, if given, is a 2-D tensor with unit column stride
    (a column slice of a wider buffer is fine).  `pre_out` (with ``gelu=True``) also
    receives ``a @ b + bias`` before the activation; `deriv_out` (instead) receives the
    GELU's derivative there, which is all the backward pass needs of it.  With
    ``accumulate=True`` the product is added onto the given `out` (the accumulators start from
    it): a weight gradient summed over row chunks."""
    require_gpu(a, b, bias, out)
    assert a.dim() == 2 and b.dim() == 2 and a.shape[1] == b.shape[0], (a.shape, b.shape)
    assert a.dtype == b.dtype
    N, K = a.shape
    M = b.shape[1]
    if out is None:
        assert not accumulate, "accumulate needs the tensor to add onto"
        out = torch.empty((N, M), dtype=a.dtype, device=a.device)
    else:
        assert out.shape == (N, M) and out.dtype == a.dtype and (out.stride(1) == 1 or M == 1)
    if accumulate:
        assert bias is None and not gelu and pre_out is None and deriv_out is None
        check(lib().ptj_gemm(ptr(a), ptr(b), ptr(out), None, N, M, K, a.stride(0), a.stride(1), b.stride(0),
                             b.stride(1), out.stride(0), _lib.EPI_ACCUMULATE, None, 0, None, 0, dtype_code(a), stream()),
              "ptj_gemm")
        return out
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
    if deriv_out is not None:
        assert pre_out is None, "one second output"
        pre_out, epi = deriv_out, _lib.EPI_BIAS_GELU_DERIV
    if pre_out is not None:
        assert gelu and pre_out.shape == (N, M) and pre_out.dtype == a.dtype and pre_out.stride(1) == 1
    check(lib().ptj_gemm(ptr(a), ptr(b), ptr(out), ptr(bias), N, M, K, a.stride(0), a.stride(1), b.stride(0),
                         b.stride(1), out.stride(0), epi, ptr(pre_out), pre_out.stride(0) if pre_out is not None else 0,
                         ptr(ws), ws_bytes, code, stream()), "ptj_gemm")
    return out


def matmul_mul_colsum_t(a: torch.Tensor, b: torch.Tensor, mul: torch.Tensor):
    """``c = (a @ b) * mul`` element-wise and the column sums of c, from one GEMM launch whose
    epilogue multiplies and sums (plus a small fixed-order reduction): with `mul` the GELU
    derivative kept by the forward pass this is d(pre-activation) and the gradient of the bias
    in front of the activation (model_triton.py:495-508, :274-294, :426).  Returns (c, sums)."""
    require_gpu(a, b, mul)
    assert a.dim() == 2 and b.dim() == 2 and a.shape[1] == b.shape[0], (a.shape, b.shape)
    N, K = a.shape
    M = b.shape[1]
    assert a.dtype == b.dtype == mul.dtype and mul.shape == (N, M) and (mul.stride(1) == 1 or M == 1)
    out = torch.empty((N, M), dtype=a.dtype, device=a.device)
    sums = torch.empty(M, dtype=a.dtype, device=a.device)
    ws_bytes = lib().ptj_gemm_mul_colsum_workspace_bytes(N, M)
    ws = _workspace(ws_bytes, a.device, "gemm_colsum") if ws_bytes else None
    check(lib().ptj_gemm_mul_colsum(ptr(a), ptr(b), ptr(mul), ptr(out), ptr(sums), N, M, K, a.stride(0), a.stride(1),
                                    b.stride(0), b.stride(1), mul.stride(0), out.stride(0), ptr(ws), ws_bytes,
                                    dtype_code(a), stream()), "ptj_gemm_mul_colsum")
    return out, sums


def t_matmul_t(a: torch.Tensor, b: torch.Tensor):
    """Reference signature (model_triton.py:373): a[N,K] contiguous, b[K,M] any strides."""
    assert a.is_contiguous(), "Matrix A must be contiguous"
    return matmul_t(a, b)


t_matmul = t_matmul_t


def _is_gelu_marker(fn):
    """The reference passes its own `t_gelu_fwd` function object as a marker for "tanh-GELU"
    (model_triton.py:1259, :2184); after an attribute-level install that object is the
    reference module's, not this package's twin, so the marker is recognised by name."""
    return getattr(fn, "__name__", "") in ("t_gelu_fwd", "t_gelu_fwd_t")


def t_tlayer_ffn_fwd_t(layer_params, x: torch.Tensor, activation_fn=t_gelu_fwd):
    """Two GEMM launches: bias+GELU epilogue, then bias (model_triton.py:1258-1313).
    `activation_fn` is the reference's marker argument: its torch GELU (`t_gelu_fwd`)."""
    assert _is_gelu_marker(activation_fn), "only the tanh-GELU epilogue exists"
    w1, b1, w2, b2 = layer_params
    shape = x.shape
    x2 = _rows2d(x)
    mid = matmul_t(x2, w1.t(), b1, gelu=True)
    out = matmul_t(mid, w2.t(), b2)
    return out.view(shape[:-1] + (w2.shape[0],))


def t_tlayer_ffn_bkwd2_t(dloss_dx, layer_params, x: torch.Tensor, activation_fn=t_gelu_fwd):
    """VJP of the feed-forward block without saved activations (model_triton.py:1410-1428):
    the first linear layer is recomputed (bias+GELU epilogue that also keeps the GELU's
    derivative), then dW2, db2, d(mid) times that derivative with db1 from the same launch,
    dW1 and dx.
    Returns (dx shaped like x, (dW1, db1, dW2, db2))."""
    assert _is_gelu_marker(activation_fn), "only the tanh-GELU backward exists"
    w1, b1, w2, b2 = layer_params
    x2 = _rows2d(x)
    d2 = _rows2d(dloss_dx)
    dgelu = torch.empty((x2.shape[0], w1.shape[0]), dtype=x2.dtype, device=x2.device)
    mid = matmul_t(x2, w1.t(), b1, gelu=True, deriv_out=dgelu)
    db2 = colsum_t(d2)
    dw2 = matmul_t(d2.t(), mid)
    dpre, db1 = matmul_mul_colsum_t(d2, w2, dgelu)
    dw1 = matmul_t(dpre.t(), x2)
    dx = matmul_t(dpre, w1)
    return dx.reshape(x.shape), (dw1, db1, dw2, db2)


# ----------------------------------------------------------------------------------
# attention  (reference: model_triton.py:706-754 fwd3_t, :951-1003 bkwd3_t)
# ----------------------------------------------------------------------------------
_mask_cache = {}


def _mask_arg(mask, B, T):
    """The attention kernels' mask argument.  ``mask=None`` is the plain causal mask: the
    kernels then mask by index.  Any tensor is bit-packed on the device for the kernels
    (ptj_attn_pack_mask, both orientations) and applied as ``mask AND (key <= query)``; no
    host comparison, no synchronisation.  The packed words are cached for the tensor they
    were made from (address, version, layout, stream), so the 2L attention calls of a step
    that share one mask pack it once; at most two entries live, each keeping its mask tensor
    alive so that its address cannot be reused while the entry exists."""
    if mask is None:
        return None
    assert mask.shape[-2:] == (T, T), mask.shape
    key = (mask.data_ptr(), mask._version, tuple(mask.shape), tuple(mask.stride()), mask.dtype, mask.device, B, T,
           stream())
    hit = _mask_cache.get(key)
    if hit is None:
        m = mask.expand(B, T, T) if mask.dim() == 3 else mask.reshape(1, T, T).expand(B, T, T)
        bytes_ = m.to(torch.bool).contiguous().view(torch.uint8)
        packed = torch.empty(lib().ptj_attn_packed_mask_bytes(B, T) // 4, dtype=torch.int32, device=mask.device)
        check(lib().ptj_attn_pack_mask(ptr(bytes_), ptr(packed), B, T, stream()), "ptj_attn_pack_mask")
        hit = (packed, mask)
        while len(_mask_cache) >= 2:
            _mask_cache.pop(next(iter(_mask_cache)))
        _mask_cache[key] = hit
    return hit[0]


def _bhr(t):
    """(batch, head, row) element strides of a [B,H,T,dh] view with unit last stride."""
    assert t.stride(3) == 1, "head dimension must be contiguous"
    return t.stride(0), t.stride(1), t.stride(2)


ATTN_DH = 64   # head dimension of the attention kernels


def _pad_heads(t, scale=None):
    """[..., dh] -> [..., 64] with zero columns (optionally times `scale`): zero columns add
    nothing to q.k and produce zero output columns."""
    out = torch.zeros(t.shape[:-1] + (ATTN_DH,), dtype=t.dtype, device=t.device)
    out[..., :t.shape[-1]] = t if scale is None else t * scale
    return out


def _aligned_view(t):
    """Kernel operand requirements: 16-byte aligned base, strides multiple of 16 bytes."""
    vec = 16 // t.element_size()
    if t.stride(3) != 1 or t.data_ptr() % 16 or any(s % vec for s in t.stride()[:3]):
        return t.contiguous()
    return t


def attn_fwd_t(q, k, v, mask, train, seed, out=None):
    """Flash-attention forward on [B,H,T,dh] *views* (any batch/head/row strides).
    Returns (O, ms[B,H,T] fp32, ls[B,H,T] fp32).  `out` may be a preallocated view.

    The kernels are written for dh = 64.  Smaller head sizes (the reference takes any power of
    two, model_triton.py:716) are run on zero-padded copies: q is scaled by sqrt(64/dh) so that
    the kernels' 1/sqrt(64) gives 1/sqrt(dh), and O is cut back to dh columns."""
    require_gpu(q, k, v)
    B, H, T, dh = q.shape
    assert k.shape == q.shape and v.shape == q.shape and q.dtype == k.dtype == v.dtype
    assert T % 64 == 0, "sequence length must be a multiple of 64"
    assert dh <= ATTN_DH, "head dimension %d > %d is not supported" % (dh, ATTN_DH)
    if dh < ATTN_DH:
        o, ms, ls = attn_fwd_t(_pad_heads(q, math.sqrt(ATTN_DH / dh)), _pad_heads(k), _pad_heads(v), mask, train, seed)
        if out is None:
            return o[..., :dh].contiguous(), ms, ls
        out.copy_(o[..., :dh])
        return out, ms, ls
    if out is None:
        out = torch.empty((B, H, T, dh), dtype=q.dtype, device=q.device)
    q, k, v = _aligned_view(q), _aligned_view(k), _aligned_view(v)
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
    = (dq, dk, dv) when given).  Head sizes below 64 run on zero-padded copies as in the forward
    (q' = f q with f = sqrt(64/dh), so dq = f dq')."""
    require_gpu(d_o, q, k, v, o)
    B, H, T, dh = q.shape
    assert dh <= ATTN_DH, "head dimension %d > %d is not supported" % (dh, ATTN_DH)
    if dh < ATTN_DH:
        f = math.sqrt(ATTN_DH / dh)
        dq, dk, dv = attn_bwd_t(_pad_heads(d_o), _pad_heads(q, f), _pad_heads(k), _pad_heads(v), _pad_heads(o), ms, ls,
                                mask, train, seed)
        if out is None:
            return dq[..., :dh] * f, dk[..., :dh].contiguous(), dv[..., :dh].contiguous()
        out[0].copy_(dq[..., :dh] * f)
        out[1].copy_(dk[..., :dh])
        out[2].copy_(dv[..., :dh])
        return out
    if out is None:
        out = tuple(torch.empty((B, H, T, dh), dtype=q.dtype, device=q.device) for _ in range(3))
    dq, dk, dv = out
    d_o, q, k, v, o = (_aligned_view(t) for t in (d_o, q, k, v, o))
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


def t_scaled_dot_prod_attn_fwd3_t(qkv: torch.Tensor, mask: torch.Tensor, train=True, p_gen_aux=None):
    """qkv [B,H,3,T,dh], mask [B,T,T] bool -> (O [B,H,T,dh], [ms, ls, O]) (model_triton.py:706-754)."""
    if train:
        assert p_gen_aux is not None
    q, k, v = torch.unbind(qkv, dim=2)
    o, ms, ls = attn_fwd_t(q, k, v, mask, train, p_gen_aux)
    return o, [ms, ls, o]


def t_scaled_dot_prod_attn_bkwd3_t(dloss_dx, acts, qkv: torch.Tensor, mask: torch.Tensor, train=True, p_gen_aux=None):
    """-> (dq, dk, dv), each [B,H,T,dh] (model_triton.py:951-1003)."""
    ms, ls, o = acts
    q, k, v = torch.unbind(qkv, dim=2)
    return attn_bwd_t(dloss_dx, q, k, v, o, ms, ls, mask, train, p_gen_aux)


def _masked_scores(q, k, mask):
    s = torch.matmul(q, k.transpose(-2, -1)) * (1.0 / math.sqrt(q.shape[-1]))
    return s.masked_fill(~mask.unsqueeze(1), -1e9)


def t_softmax_attn_fwd_t(q, k, mask, train, p_gen_aux=None):
    """Materialised dropped attention probabilities [B,H,T,T] (model_triton.py:519-526): the
    row-wise kernels (log-softmax, dropout) on torch's batched q.k^T.  Not on the training path
    (the flash kernels never form this tensor); kept because callers import the name."""
    return t_dropout_fwd_t(torch.exp(t_log_softmax_fwd_t(_masked_scores(q, k, mask))), train, p_gen_aux)


def t_softmax_attn_bkwd2_t(dloss_dx, q, k, mask, train, p_gen_aux=None):
    """VJP of t_softmax_attn_fwd_t with respect to (q, k) (model_triton.py:579-606)."""
    scale = 1.0 / math.sqrt(q.shape[-1])
    s = _masked_scores(q, k, mask)
    p = torch.exp(t_log_softmax_fwd_t(s))
    d = t_dropout_bkwd2_t(dloss_dx, p, train, p_gen_aux) * p
    d = t_log_softmax_bkwd2_t(d, s).masked_fill(~mask.unsqueeze(1), 0.0)
    return torch.matmul(d, k) * scale, torch.matmul(d.transpose(-2, -1), q) * scale


# ----------------------------------------------------------------------------------
# GPT-2 composites  (reference: model_triton.py:2334-2351 t_gpt2_tlayers_fwd3_t,
# :2535-2539 t_gpt2_forward_with_acts_t, :2489-2521 / :2583-2593 backward)
#
# Same call order and arithmetic as the reference's fwd3_t / bkwd3_t chain, with the
# host-side "linking" restated for the hardware:
#   * Q, K and V of all heads come from ONE [N,D]x[D,3D] product (the reference stacks
#     the LayerNorm output three times and runs a broadcast matmul, :1051-1053); the
#     attention kernels read/write strided slices of that buffer and of the [N,D]
#     head-merged output, so no head transposes or stack/sum copies exist;
#   * residual + dropout, and LayerNorm dx + dgamma/dbeta + residual, are single passes;
#   * the FFN pre-activation is saved instead of recomputed (:1415-1418 recomputes it);
#   * the LM-head logits live in a row-padded buffer (pitch = V rounded up to 64) so
#     that every row is 16-byte aligned; the loss gradient overwrites it in place.
# ----------------------------------------------------------------------------------
VOCAB_PAD = 64


def _padded_logits(n_rows, vocab, dtype, device):
    pitch = (vocab + VOCAB_PAD - 1) // VOCAB_PAD * VOCAB_PAD
    buf = torch.empty((n_rows, pitch), dtype=dtype, device=device)
    return buf[:, :vocab]


def t_embed_fwd(layer_params, x):
    """model_triton.py:166-167 (torch gather, as in the reference)."""
    return layer_params[0][x] * math.sqrt(layer_params[0].shape[1])


def embed_pos_dropout_t(wemb, pos, y, train=True, p_gen_aux=None):
    """dropout(t_embed_fwd((wemb,), y) + pos[:T]) in one pass: y int [B,T] -> [B,T,D]
    (the first three steps of model_triton.py:2334-2351)."""
    require_gpu(wemb, pos, y)
    B, T = y.shape
    V, D = wemb.shape
    assert pos.shape[0] >= T and pos.shape[1] == D and pos.dtype == wemb.dtype
    wc, pc = wemb.contiguous(), pos.contiguous()
    tok = y.reshape(-1).to(torch.int64).contiguous()
    out = torch.empty((B, T, D), dtype=wemb.dtype, device=wemb.device)
    check(lib().ptj_embed_fwd(ptr(wc), ptr(pc), ptr(tok), ptr(out), B * T, D, T, V, math.sqrt(D), int(bool(train)),
                              int(p_gen_aux if train else 0), dtype_code(wc), stream()), "ptj_embed_fwd")
    return out


def embed_bkwd_add_t(dwemb, d, y):
    """dwemb[tok] += sqrt(D) * (sum of the rows of d [N,D] whose token is tok), in place and
    deterministic (model_triton.py:2489-2521 scatter-add, accumulated onto the tied LM-head
    gradient as at :2591)."""
    require_gpu(dwemb, d, y)
    V, D = dwemb.shape
    assert dwemb.is_contiguous() and d.dtype == dwemb.dtype
    d2 = d.reshape(-1, D).contiguous()
    stok, order = torch.sort(y.reshape(-1).to(torch.int64), stable=True)
    check(lib().ptj_embed_bwd(ptr(d2), ptr(stok), ptr(order), ptr(dwemb), d2.shape[0], D, V, math.sqrt(D),
                              dtype_code(dwemb), stream()), "ptj_embed_bwd")
    return dwemb


def t_gpt2_tlayer_fwd3_t(layer_params, y, mask, train=True, p_gen_aux=None, h1=None, next_ln=None):
    """One block (model_triton.py:2214-2223).  y [B,T,D] -> (y_out, acts).

    `h1`, if given, is t_layernorm_fwd_t((ln1g, ln1b), y) already computed by the producer
    of y; `next_ln` = (gamma, beta) of the LayerNorm that consumes y_out asks for the same
    service: the result is then (y_out, acts, layernorm(y_out)), the norm coming out of the
    pass that forms y_out."""
    if not train:
        p_gen_aux = [0, 0, 0]
    ln1g, ln1b, wqkv, wo, ln2g, ln2b, w1, b1, w2, b2 = layer_params
    B, T, D = y.shape
    H, _, dh, _ = wqkv.shape
    N = B * T
    x_in = y.reshape(N, D)
    if h1 is None:
        h1 = t_layernorm_fwd_t((ln1g, ln1b), x_in)
    else:
        h1 = h1.reshape(N, D)
    qkv = matmul_t(h1, wqkv.view(H * 3 * dh, D).t())                     # [N, H*3*dh]
    v5 = qkv.view(B, T, H, 3, dh)
    q, k, v = (v5[:, :, :, c].permute(0, 2, 1, 3) for c in range(3))     # [B,H,T,dh] views
    o2 = torch.empty((N, D), dtype=y.dtype, device=y.device)
    o4 = o2.view(B, T, H, dh).permute(0, 2, 1, 3)
    _, ms, ls = attn_fwd_t(q, k, v, mask, train, p_gen_aux[0], out=o4)
    a_out = matmul_t(o2, wo.t())
    x_mid, h2, keep1 = dropout_add_layernorm_t(a_out, x_in, (ln2g, ln2b), train, p_gen_aux[1], want_keep=True)
    f1 = torch.empty((N, w1.shape[0]), dtype=y.dtype, device=y.device)  # gelu'(h2 @ W1^T + b1)
    g1 = matmul_t(h2, w1.t(), b1, gelu=True, deriv_out=f1)             # bias + GELU epilogue; its derivative kept
    f2 = matmul_t(g1, w2.t(), b2)
    if next_ln is not None:
        x_out, h_next, keep2 = dropout_add_layernorm_t(f2, x_mid, next_ln, train, p_gen_aux[2], want_keep=True)
    else:
        x_out, keep2 = dropout_add_t(f2, x_mid, train, p_gen_aux[2], want_keep=True)
    acts = (x_in, h1, qkv, o2, ms, ls, x_mid, h2, f1, g1, keep1, keep2)
    if next_ln is not None:
        return x_out.view(B, T, D), acts, h_next.view(B, T, D)
    return x_out.view(B, T, D), acts


def t_gpt2_tlayer_bkwd3_t(dloss_dx, acts, layer_params, y, mask, train=True, p_gen_aux=None, *, dropped_in=None,
                          drop_out=None, db2_in=None, drop_out_sum=False):
    """Backward of one block (model_triton.py:2291-2299 and the sub-block VJPs :2021-2039,
    :2175-2193).  dloss_dx [N,D] -> (dx [N,D], grads in parameter order).  `y` is the block's
    input, in the reference's argument position; `acts` already holds it, so it is not read.

    `dropped_in`, if given, is t_dropout_bkwd2_t(dloss_dx, None, train, p_gen_aux[2]) already
    computed by the producer of dloss_dx; `drop_out=(train, seed)` asks for the same service
    for the consumer of dx: the result is then (dx, grads, dropout_bkwd(dx)).  `db2_in` is
    colsum_t(dropped_in) if the producer also summed it; `drop_out_sum` appends the column
    sums of the dropped dx to the result."""
    if not train:
        p_gen_aux = [0, 0, 0]
    ln1g, ln1b, wqkv, wo, ln2g, ln2b, w1, b1, w2, b2 = layer_params
    x_in, h1, qkv, o2, ms, ls, x_mid, h2, f1, g1, keep1, _ = acts
    H, _, dh, D = wqkv.shape
    N = x_in.shape[0]
    T = ms.shape[2]
    B = N // T
    # ---- sub-block 2: x_out = x_mid + dropout(ffn(ln2(x_mid)))
    d = dropped_in if dropped_in is not None else t_dropout_bkwd2_t(dloss_dx, None, train, p_gen_aux[2])
    db2 = db2_in if (db2_in is not None and dropped_in is not None) else colsum_t(d)
    dw2 = matmul_t(d.t(), g1)                                           # [D,F]
    df1, db1 = matmul_mul_colsum_t(d, w2, f1)                           # [N,F] = (d @ W2) * gelu', and its column sums
    dw1 = matmul_t(df1.t(), h2)                                         # [F,D]
    dh2 = matmul_t(df1, w1)                                             # [N,D]
    dx_mid, (dln2g, dln2b), d = layernorm_bkwd2_t(dh2, (ln2g, ln2b), x_mid, residual=dloss_dx,
                                                  drop=(train, p_gen_aux[1], keep1))
    # ---- sub-block 1: x_mid = x_in + dropout(attn(ln1(x_in))); d = dropout_bkwd(dx_mid) came with dx_mid
    dwo = matmul_t(d.t(), o2)                                           # [D,D]
    do2 = matmul_t(d, wo)                                               # [N,D] = [B,T,H,dh]
    v5 = qkv.view(B, T, H, 3, dh)
    q, k, v = (v5[:, :, :, c].permute(0, 2, 1, 3) for c in range(3))
    dqkv = torch.empty_like(qkv)
    d5 = dqkv.view(B, T, H, 3, dh)
    outs = tuple(d5[:, :, :, c].permute(0, 2, 1, 3) for c in range(3))
    o4 = o2.view(B, T, H, dh).permute(0, 2, 1, 3)
    do4 = do2.view(B, T, H, dh).permute(0, 2, 1, 3)
    attn_bwd_t(do4, q, k, v, o4, ms, ls, mask, train, p_gen_aux[0], out=outs)
    dwqkv = matmul_t(dqkv.t(), h1).view(H, 3, dh, D)                    # [H*3*dh, D]
    dh1 = matmul_t(dqkv, wqkv.view(H * 3 * dh, D))                      # [N,D]
    dsum = None
    if drop_out is not None and drop_out_sum:
        dx_in, (dln1g, dln1b), dropped, dsum = layernorm_bkwd2_t(dh1, (ln1g, ln1b), x_in, residual=dx_mid,
                                                                 drop=drop_out, drop_sum=True)
    elif drop_out is not None:
        dx_in, (dln1g, dln1b), dropped = layernorm_bkwd2_t(dh1, (ln1g, ln1b), x_in, residual=dx_mid, drop=drop_out)
    else:
        dx_in, (dln1g, dln1b) = layernorm_bkwd2_t(dh1, (ln1g, ln1b), x_in, residual=dx_mid)
    grads = [dln1g, dln1b, dwqkv, dwo, dln2g, dln2b, dw1, db1, dw2, db2]
    if drop_out is not None and drop_out_sum:
        return dx_in, grads, dropped, dsum
    if drop_out is not None:
        return dx_in, grads, dropped
    return dx_in, grads


def t_gpt2_tlayers_fwd3_t(params, y, mask, indices, train=True, p_gen_aux=None):
    """model_triton.py:2334-2351.  y int [B,T] -> (h [B,T,D], acts)."""
    L = len(params) - 3
    if not train:
        p_gen_aux = [0] * (1 + 3 * L)
    T = y.shape[1]
    assert T <= params[1][0].shape[0], "sequence longer than the positional table"
    x = embed_pos_dropout_t(params[0][0], params[1][0], y, train, p_gen_aux[0])
    layer_acts = []
    layers = params[2:-1]
    h = None                                   # layernorm of x by the LayerNorm that reads it next
    for i, lp in enumerate(layers):
        # the pass that forms a block's output also applies the next norm (the next block's
        # first one, or the final one)
        nxt = (layers[i + 1][0], layers[i + 1][1]) if i + 1 < len(layers) else params[-1]
        x, a, h = t_gpt2_tlayer_fwd3_t(lp, x, mask, train, p_gen_aux[1 + 3 * i:4 + 3 * i], h1=h, next_ln=nxt)
        layer_acts.append(a)
    if h is None:
        h = t_layernorm_fwd_t(params[-1], x)
    return h, [layer_acts, x]


def t_gpt2_forward_with_acts_t(params, y, y_mask, y_indices, train, p_gen_aux=None):
    """model_triton.py:2535-2539: -> (logits [B,T,V], acts).  The logits are a view of a
    row-padded buffer (unit column stride)."""
    h, acts = t_gpt2_tlayers_fwd3_t(params, y, y_mask, y_indices, train, p_gen_aux)
    B, T, D = h.shape
    wemb, bemb = params[0]
    V = wemb.shape[0]
    logits = _padded_logits(B * T, V, h.dtype, h.device)
    matmul_t(h.view(B * T, D), wemb.t(), bemb, out=logits)
    return logits.view(B, T, V), [acts, h]


def t_gpt2_forward_t(params, y, y_mask, y_indices, train, p_gen_aux=None):
    return t_gpt2_forward_with_acts_t(params, y, y_mask, y_indices, train, p_gen_aux)[0]


def t_gpt2_bkwd3_p_t(dloss_dx, acts, params, y, y_mask, y_indices, train, p_gen_aux=None, *, dbemb=None):
    """model_triton.py:2583-2593 + :2489-2521: gradient nest shaped like `params`.
    `dbemb`, if given, is colsum_t(dloss_dx) already computed by the producer of dloss_dx."""
    L = len(params) - 3
    if not train:
        p_gen_aux = [0] * (1 + 3 * L)
    (layer_acts, x_last), h = acts
    wemb, bemb = params[0]
    V, D = wemb.shape
    B, T = y.shape
    N = B * T
    dlog = dloss_dx.reshape(N, V)                                       # view for padded buffers
    if dlog.stride(1) != 1:
        dlog = dlog.contiguous()
    h2d = h.view(N, D)
    if dbemb is None:
        dbemb = colsum_t(dlog)
    dwemb = matmul_t(dlog.t(), h2d)                                     # [V,D]  LM-head weight grad
    dh = matmul_t(dlog, wemb)                                           # [N,D]
    return gpt2_bkwd_below_head_t(dh, dwemb, dbemb, acts, params, y, y_mask, train, p_gen_aux)


def gpt2_bkwd_below_head_t(dh, dwemb, dbemb, acts, params, y, y_mask, train, p_gen_aux=None):
    """t_gpt2_bkwd3_p_t from the gradient of the final LayerNorm's output on (model_triton.py:2583-2593
    after the LM head's own three products): `dh` [N,D] = dlogits @ Wemb, `dwemb` [V,D] = the head's
    weight gradient (the embedding's is added onto it), `dbemb` [V] its bias gradient."""
    L = len(params) - 3
    if not train:
        p_gen_aux = [0] * (1 + 3 * L)
    (layer_acts, x_last), _ = acts
    D = dh.shape[1]
    B, T = y.shape
    N = B * T
    # Every dropout backward acts on a gradient that a LayerNorm backward has just produced,
    # so each LayerNorm backward also writes the dropped copy its consumer needs: the final
    # norm for the last block's FFN dropout (seed 3L), block i's first norm for block i-1's
    # FFN dropout (seed 3i) or, for block 0, for the embedding dropout (seed 0).
    dsum = None                                                         # colsum_t(dropped): block i's db2
    if L > 0:
        dx, (dlnfg, dlnfb), dropped, dsum = layernorm_bkwd2_t(dh, params[-1], x_last.reshape(N, D),
                                                             drop=(train, p_gen_aux[3 * L], layer_acts[L - 1][-1]),
                                                             drop_sum=True)
    else:
        dx, (dlnfg, dlnfb), dropped = layernorm_bkwd2_t(dh, params[-1], x_last.reshape(N, D),
                                                       drop=(train, p_gen_aux[0]))
    layer_grads = [None] * L
    for i in reversed(range(L)):
        res = t_gpt2_tlayer_bkwd3_t(dx, layer_acts[i], params[2 + i], layer_acts[i][0], y_mask, train,
                                    p_gen_aux[1 + 3 * i:4 + 3 * i],
                                    dropped_in=dropped, db2_in=dsum,
                                    drop_out=(train, p_gen_aux[3 * i], layer_acts[i - 1][-1] if i > 0 else None),
                                    drop_out_sum=i > 0)
        dx, layer_grads[i], dropped = res[:3]
        dsum = res[3] if i > 0 else None
    d = dropped                                                         # [N,D] = dropout_bkwd(dx, seed 0)
    # positional table: sum over the batch (model_triton.py:2518 with indices = arange(T))
    table_rows = params[1][0].shape[0]
    dpos = torch.empty_like(params[1][0])
    colsum_t(d.view(B, T * D), out=dpos[:T])                            # the sums land in the table gradient itself
    if T < table_rows:
        dpos[T:].zero_()
    # embedding: scatter-add rows by token id, times sqrt(D); tied with the LM head (:2591)
    dwemb = embed_bkwd_add_t(dwemb, d, y)
    return [[dwemb, dbemb], [dpos]] + layer_grads + [[dlnfg, dlnfb]]
