"""Rotary position embedding (reference: tinyvllm/layers/rotary_embedding.py:21-70).

The cos/sin table is computed on the host in fp32 with the reference's formula and uploaded,
so its bits are the same as a CPU restatement's; the rotation runs in the HIP kernel.
"""
from functools import lru_cache

import torch
from torch import nn

from .. import ops


def build_cos_sin_cache(rotary_dim: int, max_position: int, base: float) -> torch.Tensor:
    """fp32 ``[max_position, rotary_dim]`` = cos || sin (rotary_embedding.py:31-36), on the CPU."""
    inv_freq = 1.0 / (base ** (torch.arange(0, rotary_dim, 2, dtype=torch.float32, device="cpu") / rotary_dim))
    t = torch.arange(max_position, dtype=torch.float32, device="cpu")
    freqs = torch.einsum("i,j -> ij", t, inv_freq)
    return torch.cat((freqs.cos(), freqs.sin()), dim=-1)


class RotaryEmbedding(nn.Module):
    def __init__(self, head_size: int, rotary_dim: int, max_position_embedding: int, base: float):
        super().__init__()
        assert rotary_dim == head_size
        self.head_size = head_size
        cache = build_cos_sin_cache(rotary_dim, max_position_embedding, base)
        self.register_buffer("cos_sin_cache", cache, persistent=False)

    def forward(self, positions: torch.Tensor, query: torch.Tensor, key: torch.Tensor):
        return ops.rope(positions, query, key, self.cos_sin_cache, self.head_size)


@lru_cache(1)
def get_rope(head_size: int, rotary_dim: int, max_position: int, base: float, rope_scaling=None):
    assert rope_scaling is None
    return RotaryEmbedding(head_size, rotary_dim, max_position, base)
