"""Per-request sampling options (reference: tinyvllm/sampling_params.py:3-11)."""
from dataclasses import dataclass


@dataclass
class SamplingParams:
    temperature: float = 1.0   # 0 selects greedy decoding (the HIP argmax kernel)
    max_tokens: int = 64
    ignore_eos: bool = False

    def __post_init__(self):
        if self.temperature < 0:
            raise ValueError("temperature must be >= 0")
        if self.max_tokens < 1:
            raise ValueError("max_tokens must be >= 1")
