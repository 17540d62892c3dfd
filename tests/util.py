"""Shared helpers for the GPU parity tests."""
import torch

DTYPES = [torch.float32, torch.bfloat16]


def gen(seed):
    return torch.Generator(device="cpu").manual_seed(seed)


def randn(g, *shape, dtype=torch.float32, mean=0.0, std=1.0):
    """Seeded CPU draw in fp32, rounded to `dtype` (so GPU and oracle see the same bits)."""
    return (torch.randn(*shape, generator=g, dtype=torch.float32) * std + mean).to(dtype)


def f64(t):
    return t.detach().to("cpu").to(torch.float64)


def tol(dtype):
    """(rtol, atol) per dtype: fp32 1e-5 relative; bf16 2e-2 relative (north-star bars)."""
    return (1e-5, 1e-6) if dtype == torch.float32 else (2e-2, 2e-3)


def assert_close(got, want64, dtype, rtol=None, atol=None, what=""):
    r, a = tol(dtype)
    rtol = r if rtol is None else rtol
    atol = a if atol is None else atol
    g = f64(got)
    assert g.shape == want64.shape, (what, g.shape, want64.shape)
    err = (g - want64).abs()
    bound = atol + rtol * want64.abs()
    bad = err > bound
    if bad.any():
        i = torch.argmax(err - bound)
        raise AssertionError("%s: %d/%d outside tol (rtol=%g atol=%g); worst |err|=%.3e want=%.6e got=%.6e"
                             % (what, int(bad.sum()), bad.numel(), rtol, atol, err.flatten()[i].item(),
                                want64.flatten()[i].item(), g.flatten()[i].item()))


def rel_l2(got, want64):
    g = f64(got)
    return ((g - want64).norm() / want64.norm().clamp_min(1e-30)).item()


GEMM_ACC = 1e-5       # fp32 accumulation error of a product, relative to sum_k |a_ik b_kj|
OUT_BF16 = 2.0 ** -8  # rounding of a result to bf16 (2^-9) with a factor two of slack, relative to the value


def gemm_bound(want64, scale64, dtype, factor=1.0):
    """Element-wise error bound of a matrix product with fp32 accumulation stored as `dtype`:
    `scale64` = |a| @ |b| (+ |bias|), `want64` the exact result."""
    out = OUT_BF16 if dtype == torch.bfloat16 else 0.0
    return factor * GEMM_ACC * scale64 + out * want64.abs() + (1e-6 if dtype == torch.bfloat16 else 1e-30)
