"""Qwen3 decoder wiring (reference: tinyvllm/models/qwen3.py:14-234), one GPU.

Same module tree, parameter names and op order as the reference.  With ``fused=True`` (default)
the q/k-norm, RoPE and KV-cache store of a layer run as one kernel, and each row-parallel
projection (o_proj, down_proj) runs together with the add-RMSNorm that consumes it; every
rounding of the unfused sequence is kept, so both paths give identical bits.
"""
import torch
from torch import nn

from .. import ops
from ..config import ModelConfig
from ..layers.activation import SiluAndMul
from ..layers.attention import Attention
from ..layers.embed_head import ParallelLMHead, VocabParallelEmbedding
from ..layers.layernorm import RMSNorm
from ..layers.linear import MergedColumnParallelLinear, QKVParallelLinear, RowParallelLinear
from ..layers.rotary_embedding import get_rope
from ..utils.context import get_context


class QWen3Attention(nn.Module):
    def __init__(self, hidden_size, num_heads, num_kv_heads, max_position=4096 * 32, head_dim=None,
                 rms_norm_eps=1e-6, qkv_bias=False, rope_theta=10000, rope_scaling=None, fused=True):
        super().__init__()
        self.total_num_heads = self.num_heads = num_heads
        self.total_num_kv_heads = self.num_kv_heads = num_kv_heads
        self.head_dim = head_dim or hidden_size // num_heads
        self.q_size = self.num_heads * self.head_dim
        self.kv_size = self.num_kv_heads * self.head_dim
        self.scaling = self.head_dim ** (-0.5)
        self.fused = fused and self.head_dim == 128
        self.qkv_proj = QKVParallelLinear(hidden_size, self.head_dim, num_heads, num_kv_heads, bias=qkv_bias)
        self.o_proj = RowParallelLinear(num_heads * self.head_dim, hidden_size, bias=False)
        self.rotary_emb = get_rope(self.head_dim, rotary_dim=self.head_dim, max_position=max_position,
                                   base=rope_theta, rope_scaling=rope_scaling)
        self.attn = Attention(self.num_heads, self.head_dim, self.scaling, self.num_kv_heads)
        self.q_norm = RMSNorm(self.head_dim, eps=rms_norm_eps)
        self.k_norm = RMSNorm(self.head_dim, eps=rms_norm_eps)

    def forward(self, positions: torch.Tensor, hidden_states: torch.Tensor, residual=None, norm=None):
        """``o_proj(attention(...))``; with ``norm`` (the RMSNorm that follows, and its ``residual``) the
        projection and the add-norm are one call and ``(normed, residual)`` is returned."""
        if self.fused:
            ctx = get_context()
            attn = self.attn
            has_cache = attn.has_cache()
            # prefill without a prefix hit attends over this step's own K/V rows
            want_kv = ctx.is_prefill and ctx.block_tables is None
            # projection, q/k norm, RoPE and cache store in one call (one kernel fewer when the projection's
            # plan splits K across workgroups, which is the rule at decode sizes)
            q, k, v = self.qkv_proj.forward_qknorm_rope_store(
                hidden_states, self.q_norm, self.k_norm, positions, self.rotary_emb.cos_sin_cache,
                attn.k_cache if has_cache else None, attn.v_cache if has_cache else None,
                ctx.slot_mapping if has_cache else None, attn.k_scale, attn.v_scale, want_kv)
            o = attn(q, k, v, kv_stored=True)
        else:
            qkv = self.qkv_proj(hidden_states)
            q, k, v = qkv.split([self.q_size, self.kv_size, self.kv_size], dim=-1)
            q = self.q_norm(q.view(-1, self.num_heads, self.head_dim)).view(-1, self.q_size)
            k = self.k_norm(k.view(-1, self.num_kv_heads, self.head_dim)).view(-1, self.kv_size)
            q, k = self.rotary_emb(positions, q, k)
            o = self.attn(q, k, v)
        if norm is not None:
            return self.o_proj.forward_add_rmsnorm(o, residual, norm)
        return self.o_proj(o)


class Qwen3MLP(nn.Module):
    def __init__(self, hidden_size: int, intermediate_size: int, hidden_act: str):
        super().__init__()
        assert hidden_act == "silu"
        self.gate_up_proj = MergedColumnParallelLinear(hidden_size, [intermediate_size] * 2, bias=False)
        self.down_proj = RowParallelLinear(intermediate_size, hidden_size, bias=False)
        self.act_fn = SiluAndMul()

    def forward(self, x: torch.Tensor, residual=None, norm=None):
        # gate_up projection and activation in one kernel when the weights are int8 (qwen3.py:123-130)
        act = self.gate_up_proj.forward_silu_mul(x)
        if norm is not None:   # down_proj together with the add-norm that follows the layer
            return self.down_proj.forward_add_rmsnorm(act, residual, norm)
        return self.down_proj(act)


class Qwen3DecoderLayer(nn.Module):
    def __init__(self, config: ModelConfig, fused: bool = True):
        super().__init__()
        self.self_attn = QWen3Attention(
            hidden_size=config.hidden_size, num_heads=config.num_attention_heads,
            num_kv_heads=config.num_key_value_heads, max_position=config.max_position_embeddings,
            rms_norm_eps=config.rms_norm_eps, qkv_bias=config.attention_bias, head_dim=config.head_dim,
            rope_theta=config.rope_theta, rope_scaling=config.rope_scaling, fused=fused)
        self.mlp = Qwen3MLP(config.hidden_size, config.intermediate_size, config.hidden_act)
        self.input_layernorm = RMSNorm(config.hidden_size, eps=config.rms_norm_eps)
        self.post_attention_layernorm = RMSNorm(config.hidden_size, eps=config.rms_norm_eps)
        self.fused = fused

    def forward_normed(self, positions, normed, residual, next_norm):
        """The layer from after its input norm to after the NEXT norm (the following layer's
        ``input_layernorm`` or the model's final norm): each row-parallel projection runs together with
        the add-norm that consumes it.  Same ops and rounding points as ``forward`` chained with that norm."""
        hidden_states, residual = self.self_attn(positions, normed, residual, self.post_attention_layernorm)
        return self.mlp(hidden_states, residual, next_norm)

    def forward(self, positions, hidden_states, residual):
        if residual is None:                                   # first layer: the embedding is the residual
            residual = hidden_states
            hidden_states = self.input_layernorm(hidden_states)
        else:
            hidden_states, residual = self.input_layernorm(hidden_states, residual)
        hidden_states = self.self_attn(positions, hidden_states)
        hidden_states, residual = self.post_attention_layernorm(hidden_states, residual)
        hidden_states = self.mlp(hidden_states)
        return hidden_states, residual


class Qwen3Model(nn.Module):
    def __init__(self, config: ModelConfig, fused: bool = True):
        super().__init__()
        self.embed_tokens = VocabParallelEmbedding(config.vocab_size, config.hidden_size)
        self.layers = nn.ModuleList([Qwen3DecoderLayer(config, fused) for _ in range(config.num_hidden_layers)])
        self.norm = RMSNorm(config.hidden_size, config.rms_norm_eps)
        self.fused = fused

    def forward(self, input_ids: torch.Tensor, positions: torch.Tensor) -> torch.Tensor:
        hidden_states = self.embed_tokens(input_ids)
        if self.fused:
            residual = hidden_states                      # the embedding is the first residual
            hidden_states = self.layers[0].input_layernorm(hidden_states)
            for i, layer in enumerate(self.layers):
                nxt = self.layers[i + 1].input_layernorm if i + 1 < len(self.layers) else self.norm
                hidden_states, residual = layer.forward_normed(positions, hidden_states, residual, nxt)
            return hidden_states
        residual = None
        for layer in self.layers:
            hidden_states, residual = layer(positions, hidden_states, residual)
        hidden_states, _ = self.norm(hidden_states, residual)
        return hidden_states


class Qwen3ForCausalLM(nn.Module):
    packed_modules_mapping = {
        "q_proj": ("qkv_proj", "q"),
        "k_proj": ("qkv_proj", "k"),
        "v_proj": ("qkv_proj", "v"),
        "gate_proj": ("gate_up_proj", 0),
        "up_proj": ("gate_up_proj", 1),
    }

    def __init__(self, config: ModelConfig, fused: bool = True):
        super().__init__()
        self.config = config
        self.model = Qwen3Model(config, fused)
        self.lm_head = ParallelLMHead(config.vocab_size, config.hidden_size)
        if config.tie_word_embeddings:
            self.lm_head.weight.data = self.model.embed_tokens.weight.data

    def forward(self, input_ids: torch.Tensor, positions: torch.Tensor) -> torch.Tensor:
        return self.model(input_ids, positions)

    def compute_logits(self, hidden_states: torch.Tensor) -> torch.Tensor:
        return self.lm_head(hidden_states)

    def compute_greedy_ids(self, hidden_states: torch.Tensor) -> torch.Tensor:
        """Token ids of an all-greedy batch: LM head and argmax in one call, no logits in memory."""
        return self.lm_head.forward_greedy(hidden_states)

    def quantize_linears_(self):
        """Weight-only int8 for the four projections of every layer (embedding and LM head stay bf16)."""
        for layer in self.model.layers:
            for lin in (layer.self_attn.qkv_proj, layer.self_attn.o_proj, layer.mlp.gate_up_proj, layer.mlp.down_proj):
                lin.quantize_()
        return self

    def checkpoint_parameters(self):
        """name -> tensor of every parameter with rows in checkpoint order: a bf16 gate_up weight that
        ``pack_linears_`` re-ordered for the fused kernel is handed out as ``[gate; up]`` again."""
        out = {k: v.data for k, v in self.named_parameters()}
        for name, m in self.named_modules():
            if getattr(m, "interleaved", False) and hasattr(m, "natural_weight") and (name + ".weight") in out:
                out[name + ".weight"] = m.natural_weight()
        return out

    def pack_linears_(self):
        """int8 weights into the GEMM kernels' tile order, and a bf16 gate_up weight into the row order of the fused
        projection + SiLU-and-mul kernel (on the GPU, once, after loading / quantising)."""
        for m in self.modules():
            if hasattr(m, "interleave_") and not getattr(m, "is_quantized", False) and m.weight.is_cuda:
                m.interleave_()
            if hasattr(m, "pack_") and getattr(m, "is_quantized", False):
                m.pack_()
        return self
