"""Token sampler (reference: tinyvllm/layers/sampler.py:8-21).

All-greedy batches use the argmax kernel.  Batches with a positive temperature use the sampling
kernel: greedy rows as before, the others one draw from ``softmax(logits / T)`` by the reference's
exponential-race formula.  The reference takes its noise from torch's device generator; the kernel
draws it from Philox4x32-10 keyed by ``seed`` with a call counter as offset, so a run is
reproducible from its seed but follows a stream of its own.
"""
import torch
from torch import nn

from .. import ops


class Sampler(nn.Module):
    def __init__(self, seed: int = 0):
        super().__init__()
        self.seed = seed
        self.calls = 0          # Philox offset: one per sampled batch

    def forward(self, logits: torch.Tensor, temperatures: torch.Tensor, all_greedy: bool | None = None):
        """``all_greedy`` lets the caller (who built ``temperatures`` on the host) skip a device sync."""
        if all_greedy is None:
            all_greedy = bool((temperatures == 0).all().item())
        if all_greedy:
            return ops.argmax(logits)
        self.calls += 1
        return ops.sample(logits, temperatures, self.seed, self.calls)
