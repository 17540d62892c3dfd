"""ptj_colsum_static -- the entry point that allocates nothing -- against ptj_colsum through
the C ABI: bit-equal results on two calls in a row, the second on a smaller input (the
library's built-in scratch still holds the first call's partial sums), for both storage
types, plus the size limit (checked without a launch).  Collected last on purpose."""
import ctypes
import importlib

import pytest
import torch

from util import gen, randn

pytestmark = pytest.mark.gpu
DEV = "cuda"


def _both(l, x, rows, cols, stride, code, stream):
    out_ws = torch.empty(cols, dtype=x.dtype, device=DEV)
    out_st = torch.full((cols,), float("nan"), dtype=x.dtype, device=DEV)
    nbytes = l.ptj_colsum_workspace_bytes(rows, cols)
    ws = torch.empty(nbytes, dtype=torch.uint8, device=DEV)
    assert l.ptj_colsum(x.data_ptr(), out_ws.data_ptr(), ws.data_ptr(), nbytes, rows, cols, stride, code, stream) == 0
    rc = l.ptj_colsum_static(x.data_ptr(), out_st.data_ptr(), rows, cols, stride, code, stream)
    assert rc == 0, l.ptj_last_error()
    return out_ws, out_st


def test_colsum_static_after_init_takes_no_device_memory():
    """With ptj_init() done, a ptj_colsum_static call changes neither the free device memory nor
    torch's allocator state (inputs and output are allocated before the measurement)."""
    _lib = importlib.import_module("pre-tjax_amd._lib")
    l = _lib.lib()
    assert l.ptj_init() == 0, l.ptj_last_error()
    rows, cols = 2048, 768
    x = torch.randn(rows, cols, device=DEV)
    out = torch.empty(cols, device=DEV)
    torch.cuda.synchronize()
    free0, _ = torch.cuda.mem_get_info()
    stats0 = torch.cuda.memory_stats()["allocation.all.allocated"]
    assert l.ptj_colsum_static(x.data_ptr(), out.data_ptr(), rows, cols, cols, 0, torch.cuda.current_stream().cuda_stream) == 0
    torch.cuda.synchronize()
    free1, _ = torch.cuda.mem_get_info()
    assert free1 == free0 and torch.cuda.memory_stats()["allocation.all.allocated"] == stats0
    assert torch.allclose(out.double(), x.double().sum(0), rtol=1e-5, atol=1e-3)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_colsum_static_equals_colsum_twice_second_call_smaller(dtype):
    _lib = importlib.import_module("pre-tjax_amd._lib")
    l = _lib.lib()
    code = _lib.dtype_code(torch.empty(0, dtype=dtype))
    stream = torch.cuda.current_stream().cuda_stream
    g = gen(17)
    # first call: a wide input whose partial sums fill several MB of the scratch; second: fewer
    # rows AND fewer columns, a row pitch larger than the width, a width that is not a vector multiple
    for rows, cols, pitch in ((4096, 3072, 3072), (777, 1001, 1024)):
        x = randn(g, rows, pitch, dtype=dtype).to(DEV)
        a, b = _both(l, x, rows, cols, pitch, code, stream)
        torch.cuda.synchronize()
        assert torch.equal(a, b), (rows, cols)
        want = x[:, :cols].double().sum(0)
        tol = 1e-5 if dtype == torch.float32 else 2e-2
        assert ((a.double() - want).abs().max() <= tol * want.abs().max().clamp_min(1.0)).item()


def test_colsum_static_rejects_what_does_not_fit():
    _lib = importlib.import_module("pre-tjax_amd._lib")
    l = _lib.lib()
    rows, cols = 64, 6_000_000
    assert l.ptj_colsum_workspace_bytes(rows, cols) > (16 << 20)
    x = torch.zeros(8, device=DEV)
    assert l.ptj_colsum_static(x.data_ptr(), x.data_ptr(), rows, cols, cols, 0, None) == -1
    assert b"scratch" in l.ptj_last_error()
