"""Counterpart of the reference's ``sarathi.layernorm_ops`` (csrc/layernorm.cpp:9-14)."""
from ._ext import C as _C

rms_norm = _C.rms_norm
fused_add_rms_norm = _C.fused_add_rms_norm

__all__ = ["rms_norm", "fused_add_rms_norm"]
