"""Rotary position embedding layers (reference: sarathi/model_executor/layers/rotary_embedding.py).

The kernel is the same for every variant; the variants differ only in how the cos || sin table is
built.  Tables are computed in fp32 and cast to the model dtype, on the device the layer is created
for (the reference always builds them on "cuda"; pass ``device="cpu"`` to build one on the host).
"""
import math
from typing import Any, Dict, Optional, Tuple, Union

import torch
import torch.nn as nn

from .. import pos_encoding_ops


def _default_device() -> torch.device:
    return torch.device("cuda" if torch.cuda.is_available() else "cpu")


def base_inv_freq(base: Union[int, float], rotary_dim: int, device) -> torch.Tensor:
    """1 / base^(2i / rotary_dim), i = 0 .. rotary_dim/2 - 1 (rotary_embedding.py:55-64)."""
    exponents = torch.arange(0, rotary_dim, 2, dtype=torch.float, device=device) / rotary_dim
    return 1.0 / (base ** exponents)


def cos_sin_table(t: torch.Tensor, inv_freq: torch.Tensor, scale: float = 1.0) -> torch.Tensor:
    """[len(t), rotary_dim] = cos(t x inv_freq) || sin(t x inv_freq), times ``scale``."""
    angles = torch.outer(t, inv_freq)
    cos, sin = angles.cos(), angles.sin()
    if scale != 1.0:
        cos, sin = cos * scale, sin * scale
    return torch.cat((cos, sin), dim=-1)


class RotaryEmbedding(nn.Module):
    """Plain rotary embedding; ``forward`` rotates query and key in place."""

    def __init__(self, head_size: int, rotary_dim: int, max_position_embeddings: int, base: int,
                 is_neox_style: bool, *, device=None, dtype: Optional[torch.dtype] = None) -> None:
        super().__init__()
        self.head_size = head_size
        self.rotary_dim = rotary_dim
        self.max_position_embeddings = max_position_embeddings
        self.base = base
        self.is_neox_style = is_neox_style
        self._device = torch.device(device) if device is not None else _default_device()
        cache = self._compute_cos_sin_cache().to(dtype or torch.get_default_dtype())
        self.register_buffer("cos_sin_cache", cache, persistent=False)

    def _compute_inv_freq(self, base: Union[int, float]) -> torch.Tensor:
        return base_inv_freq(base, self.rotary_dim, self._device)

    def _positions(self, count) -> torch.Tensor:
        return torch.arange(count, dtype=torch.float, device=self._device)

    def _compute_cos_sin_cache(self) -> torch.Tensor:
        return cos_sin_table(self._positions(self.max_position_embeddings),
                             self._compute_inv_freq(self.base))

    def forward(self, positions: torch.Tensor, query: torch.Tensor,
                key: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor]:
        pos_encoding_ops.rotary_embedding(positions, query, key, self.head_size, self.cos_sin_cache,
                                          self.is_neox_style)
        return query, key


class LinearScalingRotaryEmbedding(RotaryEmbedding):
    """Position interpolation: the table covers max_position * factor positions, position p
    using the angle of p / factor (rotary_embedding.py:105-139)."""

    def __init__(self, head_size, rotary_dim, max_position_embeddings, base, is_neox_style,
                 scaling_factor: float, **kw) -> None:
        self.scaling_factor = scaling_factor
        super().__init__(head_size, rotary_dim, max_position_embeddings, base, is_neox_style, **kw)

    def _compute_cos_sin_cache(self) -> torch.Tensor:
        t = self._positions(self.max_position_embeddings * self.scaling_factor)
        return cos_sin_table(t / self.scaling_factor, self._compute_inv_freq(self.base))


class DynamicNTKScalingRotaryEmbedding(RotaryEmbedding):
    """NTK-aware base rescaling evaluated at the extended length
    (rotary_embedding.py:142-179)."""

    def __init__(self, head_size, rotary_dim, max_position_embeddings, base, is_neox_style,
                 scaling_factor: float, **kw) -> None:
        self.scaling_factor = scaling_factor
        super().__init__(head_size, rotary_dim, max_position_embeddings, base, is_neox_style, **kw)

    def _compute_cos_sin_cache(self) -> torch.Tensor:
        max_len = self.max_position_embeddings * self.scaling_factor
        stretch = self.scaling_factor * max_len / self.max_position_embeddings \
            - (self.scaling_factor - 1)
        base = self.base * stretch ** (self.rotary_dim / (self.rotary_dim - 2))
        return cos_sin_table(self._positions(max_len), self._compute_inv_freq(base))


def yarn_correction_dim(num_rotations: float, dim: int, base: float,
                        max_position_embeddings: int) -> float:
    """Dimension index whose wavelength makes ``num_rotations`` turns over the original context."""
    return dim * math.log(max_position_embeddings / (num_rotations * 2 * math.pi)) \
        / (2 * math.log(base))


def yarn_correction_range(low_rot: float, high_rot: float, dim: int, base: float,
                          max_position_embeddings: int) -> Tuple[int, int]:
    low = math.floor(yarn_correction_dim(low_rot, dim, base, max_position_embeddings))
    high = math.ceil(yarn_correction_dim(high_rot, dim, base, max_position_embeddings))
    return max(low, 0), min(high, dim - 1)


def yarn_mscale(scale: float = 1.0) -> float:
    return 1.0 if scale <= 1 else 0.1 * math.log(scale) + 1.0


class YaRNScalingRotaryEmbedding(RotaryEmbedding):
    """YaRN (Peng et al.): per-dimension blend of interpolated and original frequencies plus a
    magnitude correction (rotary_embedding.py:182-298).  ``max_position_embeddings`` is the
    ORIGINAL context length; the table covers it times ``scaling_factor``."""

    def __init__(self, head_size, rotary_dim, max_position_embeddings, base, is_neox_style,
                 scaling_factor: float, *, extrapolation_factor: float = 1, attn_factor: float = 1,
                 beta_fast: float = 32, beta_slow: float = 1, **kw) -> None:
        self.scaling_factor = scaling_factor
        self.extrapolation_factor = extrapolation_factor
        self.attn_factor = attn_factor
        self.beta_fast = beta_fast
        self.beta_slow = beta_slow
        self.mscale = float(yarn_mscale(scaling_factor) * attn_factor)
        super().__init__(head_size, rotary_dim, max_position_embeddings, base, is_neox_style, **kw)

    def _compute_inv_freq(self, scaling_factor: float) -> torch.Tensor:
        pos_freqs = self.base ** (
            torch.arange(0, self.rotary_dim, 2, dtype=torch.float, device=self._device)
            / self.rotary_dim)
        original = 1.0 / pos_freqs                          # extrapolation: keep the frequency
        interpolated = 1.0 / (scaling_factor * pos_freqs)   # interpolation: stretch it
        low, high = yarn_correction_range(self.beta_fast, self.beta_slow, self.rotary_dim, self.base,
                                          self.max_position_embeddings)
        hi = high + 0.001 if low == high else high
        ramp = ((torch.arange(self.rotary_dim // 2, dtype=torch.float, device=self._device) - low)
                / (hi - low)).clamp(0, 1)
        keep_original = (1 - ramp) * self.extrapolation_factor
        return interpolated * (1 - keep_original) + original * keep_original

    def _compute_cos_sin_cache(self) -> torch.Tensor:
        t = self._positions(self.max_position_embeddings * self.scaling_factor)
        return cos_sin_table(t, self._compute_inv_freq(self.scaling_factor), self.mscale)


def get_rope(head_size: int, rotary_dim: int, max_position: int, base: int, is_neox_style: bool,
             rope_scaling: Optional[Dict[str, Any]], **kw) -> RotaryEmbedding:
    """Factory with the reference's signature (rotary_embedding.py:301-344)."""
    if rope_scaling is None:
        return RotaryEmbedding(head_size, rotary_dim, max_position, base, is_neox_style, **kw)
    kind, factor = rope_scaling["type"], rope_scaling["factor"]
    if kind == "linear":
        return LinearScalingRotaryEmbedding(head_size, rotary_dim, max_position, base,
                                            is_neox_style, factor, **kw)
    if kind == "dynamic":
        return DynamicNTKScalingRotaryEmbedding(head_size, rotary_dim, max_position, base,
                                                is_neox_style, factor, **kw)
    if kind == "yarn":
        original = rope_scaling["original_max_position_embeddings"]
        assert max_position == original * factor
        extra = {k: rope_scaling[k] for k in ("extrapolation_factor", "attn_factor", "beta_fast",
                                              "beta_slow") if k in rope_scaling}
        return YaRNScalingRotaryEmbedding(head_size, rotary_dim, original, base, is_neox_style,
                                          factor, **extra, **kw)
    raise ValueError(f"Unknown RoPE scaling type {kind}")
