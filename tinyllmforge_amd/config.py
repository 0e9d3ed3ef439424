"""Engine configuration (reference: tinyvllm/config.py:5-26).

The reference needs a local HuggingFace directory and ``transformers.AutoConfig``.  Here
``model`` may also be a plain dict (or a ``ModelConfig``) of architecture numbers, so that
random-init benchmarks and tests need no files; a directory is read through its
``config.json`` only.
"""
from __future__ import annotations

import json
import os
from dataclasses import dataclass, field, fields
from typing import Any

import torch


@dataclass
class ModelConfig:
    """The architecture fields the reference reads from ``hf_config`` (models/qwen3.py:139-153)."""
    hidden_size: int
    num_hidden_layers: int
    num_attention_heads: int
    num_key_value_heads: int
    intermediate_size: int
    vocab_size: int = 151936
    head_dim: int | None = None
    rms_norm_eps: float = 1e-6
    rope_theta: float = 1e6
    max_position_embeddings: int = 40960
    tie_word_embeddings: bool = False
    hidden_act: str = "silu"
    attention_bias: bool = False
    rope_scaling: Any = None
    torch_dtype: Any = torch.bfloat16

    def __post_init__(self):
        if self.head_dim is None:
            self.head_dim = self.hidden_size // self.num_attention_heads
        if isinstance(self.torch_dtype, str):
            self.torch_dtype = getattr(torch, self.torch_dtype.replace("torch.", ""))

    @classmethod
    def from_any(cls, src) -> "ModelConfig":
        if isinstance(src, cls):
            return src
        if isinstance(src, str):
            with open(os.path.join(src, "config.json")) as f:
                src = json.load(f)
        names = {f.name for f in fields(cls)}
        return cls(**{k: v for k, v in dict(src).items() if k in names})


# Architectures named by the benchmark configurations (Qwen3 family shapes).
QWEN3_SHAPES = {
    "qwen3-0.6b": dict(hidden_size=1024, num_hidden_layers=28, num_attention_heads=16, num_key_value_heads=8,
                       head_dim=128, intermediate_size=3072, tie_word_embeddings=True),
    "qwen3-8b": dict(hidden_size=4096, num_hidden_layers=36, num_attention_heads=32, num_key_value_heads=8,
                     head_dim=128, intermediate_size=12288, tie_word_embeddings=False),
    "qwen3-32b": dict(hidden_size=5120, num_hidden_layers=64, num_attention_heads=64, num_key_value_heads=8,
                      head_dim=128, intermediate_size=25600, tie_word_embeddings=False),
}


@dataclass
class Config:
    model: Any                              # directory, dict, ModelConfig or a key of QWEN3_SHAPES
    max_num_batched_tokens: int = 16384
    max_num_seqs: int = 512
    max_model_len: int = 4096
    gpu_memory_utilization: float = 0.9
    tensor_parallel_size: int = 1
    enforce_eager: bool = False
    hf_config: ModelConfig | None = None
    eos: int = -1
    kvcache_block_size: int = 256
    num_kvcache_blocks: int = -1
    # additions of this build (the reference has neither)
    quantization: str | None = None         # None (bf16 linears) or "w8a16"
    kv_cache_dtype: str = "bf16"            # "bf16" or "fp8_e4m3"
    # static scales of an e4m3 cache, c = e4m3(sat(x / scale)): a float, [Hkv] values or [L][Hkv] values.
    # 1/16 represents |x| <= 28 (448 / 16); larger K or V entries saturate.
    kv_k_scale: Any = 1.0 / 16
    kv_v_scale: Any = 1.0 / 16
    seed: int = 0                           # random-init seed when no weights are given
    decode_position_quirk: bool = True      # reference feeds positions = len(seq) in decode (model_runner.py:219)
    # Decode steps of sequences that can only end by length (ignore_eos) are launched before the token ids of
    # the step before them have been read back: the ids stay on the device as the next step's input, the host
    # keeps two steps in flight and patches the values into its sequences as they arrive.  Same tokens, same
    # block ids and step counts as the step-by-step loop; False restores that loop.
    run_ahead: bool = True
    # The decode attention kernel's split of the step's work over the workgroups is made once per step (one small
    # kernel at the head of the step) instead of by every layer's call: same results, a shorter start per layer.
    decode_plan: bool = True

    def __post_init__(self):
        if isinstance(self.model, str) and self.model.lower() in QWEN3_SHAPES:
            self.hf_config = ModelConfig.from_any(QWEN3_SHAPES[self.model.lower()])
        elif isinstance(self.model, str):
            assert os.path.isdir(self.model), f"{self.model} is neither a known shape nor a directory"
            self.hf_config = ModelConfig.from_any(self.model)
        else:
            self.hf_config = ModelConfig.from_any(self.model)
        assert self.kvcache_block_size % 256 == 0
        assert self.tensor_parallel_size == 1, "this build runs one GPU, no tensor parallelism"
        assert self.quantization in (None, "w8a16")
        assert self.kv_cache_dtype in ("bf16", "fp8_e4m3")
        self.max_model_len = min(self.max_model_len, self.hf_config.max_position_embeddings)
        assert self.max_num_batched_tokens >= self.max_model_len
