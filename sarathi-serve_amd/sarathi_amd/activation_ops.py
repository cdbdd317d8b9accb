"""Counterpart of the reference's ``sarathi.activation_ops`` (csrc/activation.cpp:15-28)."""
from ._ext import C as _C

silu_and_mul = _C.silu_and_mul
gelu_new = _C.gelu_new
gelu_fast = _C.gelu_fast

__all__ = ["silu_and_mul", "gelu_new", "gelu_fast"]
