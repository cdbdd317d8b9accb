"""RMSNorm layer (reference: sarathi/model_executor/layers/layernorm.py:12-40)."""
from typing import Optional, Tuple

import torch
import torch.nn as nn

from .. import layernorm_ops
from .op_timer import op_timer


class RMSNorm(nn.Module):
    """x -> w * x / sqrt(mean(x^2) + eps).

    ``forward(x)`` matches the reference layer: a new tensor is returned and ``x`` is left alone.
    ``forward(x, residual)`` is the fused form of the decoder layer's
    ``x = residual + x; residual = x; x = norm(x)`` (sarathi/model_executor/models/llama.py:248-252):
    both tensors are updated in place and returned.

    ``norm_name`` / ``layer_id`` are the reference's per-op timer labels
    (sarathi/metrics/constants.py:9-34); the op runs inside the timer that
    ``layers.set_op_timer_factory`` provides for them (a no-op unless a factory is installed), where
    the reference enters its ``CudaTimer`` (layers/layernorm.py:29-32).
    """

    def __init__(self, hidden_size: int, eps: float = 1e-6, norm_name: Optional[str] = None,
                 layer_id: Optional[int] = None) -> None:
        super().__init__()
        self.weight = nn.Parameter(torch.ones(hidden_size))
        self.variance_epsilon = eps
        self.norm_name = norm_name
        self.layer_id = layer_id
        self._norm_timer = op_timer(norm_name, layer_id)

    def forward(self, x: torch.Tensor, residual: Optional[torch.Tensor] = None):
        with self._norm_timer:
            if residual is None:
                out = torch.empty_like(x)
                layernorm_ops.rms_norm(out, x, self.weight.data, self.variance_epsilon)
                return out
            layernorm_ops.fused_add_rms_norm(x, residual, self.weight.data, self.variance_epsilon)
            return x, residual
