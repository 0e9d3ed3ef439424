"""Public entry point (reference: tinyvllm/llm.py:4).

    llm = LLM("qwen3-8b", quantization="w8a16", max_model_len=4096)
    outputs = llm.generate(prompts, SamplingParams(temperature=0.0, max_tokens=64))

``model`` is a checkpoint directory (``config.json`` + safetensors, bf16 or written by
``utils.loader.quantize_checkpoint``), a shape name from ``config.QWEN3_SHAPES``, a dict of
architecture fields or a ``ModelConfig``; the keyword arguments are the fields of ``Config``.
Prompts are lists of token ids, or strings when a tokenizer is available.  The engine behind it is
``engine.llm_engine.LLMEngine``; the reference exposes it under this name and so does this package.
"""
from .engine.llm_engine import LLMEngine

__all__ = ["LLM"]


class LLM(LLMEngine):
    """Name under which the reference publishes its engine; adds nothing to it."""
