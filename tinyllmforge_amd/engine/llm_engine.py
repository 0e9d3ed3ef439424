"""Request loop (reference: tinyvllm/engine/llm_engine.py:15-101), one process, one GPU.

The tokenizer is optional: prompts given as token-id lists need none (the benchmark and parity
configurations are random-init models without tokenizer files)."""
from __future__ import annotations

import atexit
from dataclasses import fields
from time import perf_counter

from ..config import Config
from ..sampling_params import SamplingParams
from .model_runner import ModelRunner
from .scheduler import Scheduler
from .sequence import Sequence


class LLMEngine:
    def __init__(self, model, **kwargs):
        names = {f.name for f in fields(Config)}
        state_dict = kwargs.pop("state_dict", None)
        config = Config(model, **{k: v for k, v in kwargs.items() if k in names})
        self.config = config
        Sequence.block_size = config.kvcache_block_size
        self.model_runner = ModelRunner(config, 0, None, state_dict=state_dict)
        self.tokenizer = None
        if isinstance(config.model, str):
            import os
            if os.path.isdir(config.model) and os.path.exists(os.path.join(config.model, "tokenizer.json")):
                from transformers import AutoTokenizer
                self.tokenizer = AutoTokenizer.from_pretrained(config.model, use_fast=True)
                config.eos = self.tokenizer.eos_token_id
        self.scheduler = Scheduler(config)
        self.last_stats = {}
        atexit.register(self.exit)

    def exit(self):
        if getattr(self, "model_runner", None) is not None:
            self.model_runner.call("exit")
            self.model_runner = None

    def add_request(self, prompt, sampling_params: SamplingParams):
        if isinstance(prompt, str):
            if self.tokenizer is None:
                raise ValueError("string prompts need a tokenizer; pass token-id lists instead")
            prompt = self.tokenizer.encode(prompt)
        if len(prompt) > self.config.hf_config.max_position_embeddings:
            raise ValueError(f"prompt of {len(prompt)} tokens exceeds max_position_embeddings "
                             f"({self.config.hf_config.max_position_embeddings}): no RoPE row for its tail")
        self.scheduler.add(Sequence(prompt, sampling_params))

    def step(self):
        seqs, is_prefill = self.scheduler.schedule()
        token_ids = self.model_runner.call("run", seqs, is_prefill)
        self.scheduler.postprocess(seqs, token_ids)
        outputs = [(s.seq_id, s.completion_token_ids) for s in seqs if s.is_finished]
        num_tokens = sum(len(s) for s in seqs) if is_prefill else -len(seqs)
        # for the statistics of generate(): cached prompt tokens of a prefill step, context tokens a
        # decode step's attention reads (the token stored in this step included)
        self._step_info = (sum(s.num_cached_tokens for s in seqs) if is_prefill else 0,
                           0 if is_prefill else sum(len(s) - 1 for s in seqs))
        return outputs, num_tokens

    def is_finished(self):
        return self.scheduler.is_finished()

    def generate(self, prompts, sampling_params, use_tqdm: bool = False):
        if not isinstance(sampling_params, list):
            sampling_params = [sampling_params] * len(prompts)
        for prompt, sp in zip(prompts, sampling_params):
            self.add_request(prompt, sp)
        done = {}
        stats = dict(prefill_steps=0, decode_steps=0, prefill_tokens=0, decode_tokens=0,
                     prefill_time=0.0, decode_time=0.0, cached_prompt_tokens=0, decode_context_tokens=0)
        while not self.is_finished():
            t0 = perf_counter()
            finished, num_tokens = self.step()
            dt = perf_counter() - t0
            kind = "prefill" if num_tokens > 0 else "decode"
            stats[f"{kind}_steps"] += 1
            stats[f"{kind}_tokens"] += abs(num_tokens)
            stats[f"{kind}_time"] += dt
            stats["cached_prompt_tokens"] += self._step_info[0]
            stats["decode_context_tokens"] += self._step_info[1]
            for seq_id, toks in finished:
                done[seq_id] = toks
        self.last_stats = stats
        ordered = [done[k] for k in sorted(done)]
        decode = self.tokenizer.decode if self.tokenizer is not None else (lambda ids: "")
        return [{"text": decode(t), "token_ids": t} for t in ordered]
