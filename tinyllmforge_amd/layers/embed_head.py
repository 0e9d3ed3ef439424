"""Token embedding and LM head (reference: tinyvllm/layers/embed_head.py:9-70), one GPU."""
import torch
from torch import nn

from .. import ops
from ..utils.context import get_context


class VocabParallelEmbedding(nn.Module):
    def __init__(self, num_embeddings: int, embedding_dim: int):
        super().__init__()
        self.tp_rank, self.tp_size = 0, 1
        self.num_embeddings = num_embeddings
        self.num_embeddings_per_partition = num_embeddings
        self.weight = nn.Parameter(torch.empty(num_embeddings, embedding_dim))
        self.weight.weight_loader = self.weight_loader

    def weight_loader(self, param: nn.Parameter, loaded_weight: torch.Tensor):
        assert param.data.size() == loaded_weight.size()
        param.data.copy_(loaded_weight)

    def forward(self, x: torch.Tensor):
        return ops.embedding(x, self.weight.data)


class ParallelLMHead(VocabParallelEmbedding):
    def __init__(self, num_embeddings: int, embedding_dim: int, bias: bool = False):
        super().__init__(num_embeddings, embedding_dim)
        assert not bias

    def forward(self, x: torch.Tensor):
        ctx = get_context()
        if ctx.is_prefill:                                   # only the last token of each sequence
            last = (ctx.cu_seqlens_q[1:] - 1).long()
            x = x[last].contiguous()
        return ops.bf16_linear(x, self.weight.data)

    def forward_greedy(self, x: torch.Tensor):
        """``argmax(self(x), -1)``: the greedy branch of the sampler (sampler.py:13-14,21) applied to this
        layer's logits, in one call that never stores them."""
        ctx = get_context()
        if ctx.is_prefill:
            last = (ctx.cu_seqlens_q[1:] - 1).long()
            x = x[last].contiguous()
        return ops.bf16_linear_argmax(x, self.weight.data)
