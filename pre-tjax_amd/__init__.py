"""MI355X-native replacement of the pre-tjax Triton kernel path.

Modules keep the reference's flat module names so that code written against it
(`from model_triton import t_layernorm_fwd_t`, ...) can be pointed here:
`model_triton`, `loss_and_optimizer_triton`.
"""
from . import _lib  # noqa: F401
