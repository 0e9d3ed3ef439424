"""Request loop (reference: tinyvllm/engine/llm_engine.py:15-101), one process, one GPU.

The tokenizer is optional: prompts given as token-id lists need none (the benchmark and parity
configurations are random-init models without tokenizer files)."""
from __future__ import annotations

import atexit
from collections import deque
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
        # decode steps whose token ids have not been read back yet, oldest first:
        # (sequences, device ids, pinned landing buffer, arrival event, seq_id -> row)
        self._ahead = deque()
        self.steps_ahead = 0     # decode steps launched without waiting for the ids of the step before
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

    AHEAD = 2    # decode steps in flight before the oldest one's token ids are waited for

    def _retire(self):
        """Read back the oldest step that ran ahead; the sequences it finished, now that their ids are known."""
        seqs, _, landing, arrived, _ = self._ahead.popleft()
        arrived.synchronize()
        self.scheduler.patch(seqs, landing.tolist())
        return [(s.seq_id, s.completion_token_ids) for s in seqs if s.is_finished and s.num_unknown == 0]

    def _drain(self):
        outputs = []
        while self._ahead:
            outputs += self._retire()
        return outputs

    def step(self):
        """One engine step (llm_engine.py:53-59).  A decode step of sequences that can only end by length
        does not wait for its token ids (Config.run_ahead): it is launched with the ids of the step before it
        still on the device, and the sequences finished by a step are reported when its ids have arrived -
        at the latest by the step that finishes the last sequence."""
        runner, sched = self.model_runner, self.scheduler
        ahead = self.config.run_ahead and sched.can_run_ahead() and bool(runner.graph_bs) and not runner.enforce_eager
        outputs = [] if ahead else self._drain()
        seqs, is_prefill = sched.schedule()
        if ahead and not is_prefill and runner.graph_ready(seqs):
            while len(self._ahead) >= self.AHEAD:
                outputs += self._retire()
            feed = None
            if self._ahead:      # the ids this step feeds on are those of the newest step in flight
                _, tokens, _, _, rows = self._ahead[-1]
                feed = (tokens, [rows[s.seq_id] for s in seqs])
            tokens, landing, arrived = runner.run_ahead(seqs, feed)
            self._ahead.append((seqs, tokens, landing, arrived, {s.seq_id: i for i, s in enumerate(seqs)}))
            sched.postprocess_ahead(seqs)
            self.steps_ahead += 1
            if sched.is_finished():
                outputs += self._drain()
        else:
            outputs += self._drain()
            token_ids = runner.call("run", seqs, is_prefill)
            sched.postprocess(seqs, token_ids)
            outputs += [(s.seq_id, s.completion_token_ids) for s in seqs if s.is_finished]
        num_tokens = sum(len(s) for s in seqs) if is_prefill else -len(seqs)
        # for the statistics of generate(): cached prompt tokens of a prefill step, context tokens a
        # decode step's attention reads (the token stored in this step included)
        self._step_info = (sum(s.num_cached_tokens for s in seqs) if is_prefill else 0,
                           0 if is_prefill else sum(len(s) - 1 for s in seqs))
        return outputs, num_tokens

    def is_finished(self):
        return self.scheduler.is_finished() and not self._ahead

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
