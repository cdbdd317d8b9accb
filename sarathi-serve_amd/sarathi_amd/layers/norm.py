"""RMSNorm layer (reference: sarathi/model_executor/layers/layernorm.py:12-40)."""
from typing import Optional, Tuple

import torch
import torch.nn as nn

from .. import layernorm_ops


class RMSNorm(nn.Module):
    """x -> w * x / sqrt(mean(x^2) + eps).

    ``forward(x)`` matches the reference layer: a new tensor is returned and ``x`` is left alone.
    ``forward(x, residual)`` is the fused form of the decoder layer's
    ``x = residual + x; residual = x; x = norm(x)`` (sarathi/model_executor/models/llama.py:248-252):
    both tensors are updated in place and returned.

    ``norm_name`` / ``layer_id`` are the reference's per-op timer labels
    (sarathi/metrics/constants.py); they are accepted and kept but nothing is timed here.
    """

    def __init__(self, hidden_size: int, eps: float = 1e-6, norm_name: Optional[str] = None,
                 layer_id: Optional[int] = None) -> None:
        super().__init__()
        self.weight = nn.Parameter(torch.ones(hidden_size))
        self.variance_epsilon = eps
        self.norm_name = norm_name
        self.layer_id = layer_id

    def forward(self, x: torch.Tensor, residual: Optional[torch.Tensor] = None):
        if residual is None:
            out = torch.empty_like(x)
            layernorm_ops.rms_norm(out, x, self.weight.data, self.variance_epsilon)
            return out
        layernorm_ops.fused_add_rms_norm(x, residual, self.weight.data, self.variance_epsilon)
        return x, residual
