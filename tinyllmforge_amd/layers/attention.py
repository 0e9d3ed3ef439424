"""KV-cache write and attention (reference: tinyvllm/layers/attention.py:33-111)."""
import torch
from torch import nn

from .. import ops
from ..utils.context import get_context


def store_kvcache(key, value, k_cache, v_cache, slot_mapping, k_scale=None, v_scale=None):
    """``cache.view(-1, D)[slot_mapping[i]] = key[i] / value[i]`` (attention.py:33-48)."""
    ops.store_kvcache(key, value, k_cache, v_cache, slot_mapping, k_scale, v_scale)


class Attention(nn.Module):
    def __init__(self, num_heads: int, head_dim: int, scale: float, num_kv_heads: int):
        super().__init__()
        self.num_heads = num_heads
        self.head_dim = head_dim
        self.scale = scale
        self.num_kv_heads = num_kv_heads
        self.k_cache = self.v_cache = torch.tensor([])      # bound by the model runner
        self.k_scale = self.v_scale = None                  # fp32 [Hkv] for an e4m3 cache

    def has_cache(self) -> bool:
        return self.k_cache.numel() > 0 and self.v_cache.numel() > 0

    def forward(self, q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, kv_stored: bool = False):
        """``q [N, Hq*Dh]``, ``k``/``v`` ``[N, Hkv*Dh]`` -> ``[N, Hq*Dh]``.

        ``kv_stored`` says the caller already wrote K/V to the cache (the fused
        q/k-norm + RoPE + store kernel does).
        """
        q = q.view(-1, self.num_heads, self.head_dim)
        ctx = get_context()
        if self.has_cache() and not kv_stored:
            store_kvcache(k.view(-1, self.num_kv_heads, self.head_dim), v.view(-1, self.num_kv_heads, self.head_dim),
                          self.k_cache, self.v_cache, ctx.slot_mapping, self.k_scale, self.v_scale)
        if ctx.is_prefill:
            if ctx.block_tables is not None:                 # prefix hit: every sequence reads the paged cache
                return ops.varlen_prefill_attention(q, self.k_cache, self.v_cache, ctx.cu_seqlens_q, ctx.cu_seqlens_k,
                                                    ctx.max_seqlen_q, self.scale, block_tables=ctx.block_tables,
                                                    k_scale=self.k_scale, v_scale=self.v_scale)
            return ops.varlen_prefill_attention(q, k.view(-1, self.num_kv_heads, self.head_dim),
                                                v.view(-1, self.num_kv_heads, self.head_dim),
                                                ctx.cu_seqlens_q, ctx.cu_seqlens_k, ctx.max_seqlen_q, self.scale)
        return ops.paged_decode_attention(q, self.k_cache, self.v_cache, ctx.context_lens, ctx.block_tables,
                                          self.scale, self.k_scale, self.v_scale, plan=ctx.decode_plan)
