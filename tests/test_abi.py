"""CPU-only: libptj.so loads and exports every symbol include/ptj.h declares, the
ctypes table covers exactly those symbols, and argument errors are reported without
touching a GPU."""
import ctypes
import importlib
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared():
    src = open(os.path.join(ROOT, "include", "ptj.h")).read()
    src = re.sub(r"/\*.*?\*/", "", src, flags=re.S)
    return sorted(set(re.findall(r"\b(ptj_[a-z0-9_]+)\s*\(", src)))


def test_header_symbols_exported_and_bound():
    _lib = importlib.import_module("pre-tjax_amd._lib")
    names = _declared()
    assert len(names) >= 15
    assert sorted(_lib.SIGNATURES) == names
    l = ctypes.CDLL(_lib.LIB_PATH)
    for n in names:
        assert hasattr(l, n), n
    assert _lib.lib().ptj_version() >= 1


def test_argument_errors_do_not_launch():
    _lib = importlib.import_module("pre-tjax_amd._lib")
    l = _lib.lib()
    assert l.ptj_layernorm_fwd(None, None, None, None, 4, 8, 8, 8, 0, None) == -1
    assert b"null" in l.ptj_last_error()
    assert l.ptj_gelu_fwd(1, 1, 16, 7, None) == -1          # unknown dtype
    assert b"dtype" in l.ptj_last_error()
    assert l.ptj_layernorm_bwd_workspace_bytes(8192, 768) > 0
    assert l.ptj_ce_workspace_bytes(8192) == 8192 * 4


def test_wrappers_refuse_cpu_tensors():
    import torch
    mt = importlib.import_module("pre-tjax_amd.model_triton")
    _lib = importlib.import_module("pre-tjax_amd._lib")
    with pytest.raises(_lib.PtjError):
        mt.t_gelu_fwd_t(torch.zeros(8))
