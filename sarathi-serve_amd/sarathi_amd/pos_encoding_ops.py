"""Counterpart of the reference's ``sarathi.pos_encoding_ops`` (csrc/pos_encoding.cpp:11-16)."""
from ._ext import C as _C

rotary_embedding = _C.rotary_embedding

__all__ = ["rotary_embedding"]
