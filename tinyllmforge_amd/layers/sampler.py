"""Token sampler (reference: tinyvllm/layers/sampler.py:8-21).

Greedy rows (temperature 0) use the HIP argmax kernel.  Rows with a positive temperature keep
the reference's Gumbel-max formula in torch: it depends on the device RNG stream, which no
kernel of this library reproduces, so it stays a torch composition.
"""
import torch
from torch import nn

from .. import ops


class Sampler(nn.Module):
    def forward(self, logits: torch.Tensor, temperatures: torch.Tensor, all_greedy: bool | None = None):
        """``all_greedy`` lets the caller (who built ``temperatures`` on the host) skip a device sync."""
        if all_greedy is None:
            all_greedy = bool((temperatures == 0).all().item())
        greedy = ops.argmax(logits)
        if all_greedy:
            return greedy
        l32 = logits.to(torch.float32)
        safe_t = torch.where(temperatures == 0, torch.ones_like(temperatures), temperatures)
        probs = torch.softmax(l32 / safe_t.unsqueeze(1), dim=-1, dtype=torch.float32)
        sampled = probs.div_(torch.empty_like(probs).exponential_(1) + 1e-10).argmax(dim=-1)
        return torch.where(temperatures == 0, greedy, sampled)
