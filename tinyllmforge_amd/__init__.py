"""MI355X-native hot path of a TinyLLMForge (tinyvllm) engine.

``LLM`` / ``SamplingParams`` mirror the reference's public surface (tinyvllm/__init__.py:1-2); the
per-token kernels live in ``libtlf_hip.so`` (C ABI in ``include/tlf_hip.h``) and are reached
through ``tinyllmforge_amd.ops`` and the ``tinyllmforge_amd.layers`` modules.
"""
from .sampling_params import SamplingParams


def __getattr__(name):
    if name == "LLM":
        from .llm import LLM
        return LLM
    raise AttributeError(name)


__all__ = ["LLM", "SamplingParams"]
