"""RMSNorm with optional fused residual add (reference: tinyvllm/layers/layernorm.py:10-54)."""
import torch
from torch import nn

from .. import ops


class RMSNorm(nn.Module):
    def __init__(self, hidden_size: int, eps: float = 1e-6):
        super().__init__()
        self.hidden_size = hidden_size
        self.eps = eps
        self.weight = nn.Parameter(torch.ones(hidden_size))

    def rms_forward(self, x: torch.Tensor) -> torch.Tensor:
        return ops.rms_norm(x, self.weight.data, self.eps)

    def add_rms_forward(self, x: torch.Tensor, residual: torch.Tensor):
        return ops.add_rms_norm(x, residual, self.weight.data, self.eps)

    def forward(self, x: torch.Tensor, residual: torch.Tensor | None = None):
        if residual is None:
            return self.rms_forward(x)
        return self.add_rms_forward(x, residual)
