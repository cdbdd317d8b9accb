"""Activation layers (reference: sarathi/model_executor/layers/activation.py:9-61)."""
import torch
import torch.nn as nn

from .. import activation_ops


class SiluAndMul(nn.Module):
    """x [num_tokens, 2*d] -> silu(x[:, :d]) * x[:, d:]  [num_tokens, d]"""

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        out = torch.empty((x.shape[0], x.shape[1] // 2), dtype=x.dtype, device=x.device)
        activation_ops.silu_and_mul(out, x)
        return out


class NewGELU(nn.Module):
    def forward(self, x: torch.Tensor) -> torch.Tensor:
        out = torch.empty_like(x)
        activation_ops.gelu_new(out, x)
        return out


class FastGELU(nn.Module):
    def forward(self, x: torch.Tensor) -> torch.Tensor:
        out = torch.empty_like(x)
        activation_ops.gelu_fast(out, x)
        return out


def get_act_fn(act_fn: str) -> nn.Module:
    """Activation by its HF config name; same registry keys as the reference
    (layers/activation.py:47-61)."""
    table = {
        "gelu": lambda: nn.GELU(),
        "gelu_fast": FastGELU,
        "gelu_new": NewGELU,
        "gelu_pytorch_tanh": lambda: nn.GELU(approximate="tanh"),
        "relu": lambda: nn.ReLU(),
    }
    key = act_fn.lower()
    if key not in table:
        raise ValueError(f"Activation function {act_fn!r} is not supported.")
    return table[key]()
