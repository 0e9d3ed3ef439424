"""One request's token state and its block arithmetic (reference: tinyvllm/engine/sequence.py:11-71)."""
from __future__ import annotations

import itertools
from enum import Enum

from ..sampling_params import SamplingParams


class SequenceStatus(Enum):
    WAITING = 1
    RUNNING = 2
    FINISHED = 3


class Sequence:
    # Set from Config.kvcache_block_size by the engine (the reference hard-codes 256 here,
    # sequence.py:12, while the runner reads the config value).
    block_size = 256
    _ids = itertools.count()

    def __init__(self, token_ids: list[int], sampling_params: SamplingParams | None = None):
        sp = sampling_params or SamplingParams()
        if not token_ids:
            raise ValueError("a sequence needs at least one prompt token")
        self.seq_id = next(Sequence._ids)
        self.status = SequenceStatus.WAITING
        self.token_ids = list(token_ids)
        self.num_prompt_tokens = len(self.token_ids)
        self.num_tokens = self.num_prompt_tokens
        self.last_token = self.token_ids[-1]
        self.num_cached_tokens = 0
        # tokens at the tail whose values are not on the host yet (a decode step that runs ahead of the
        # read-back of the step before it appends a stand-in and patches the value in later)
        self.num_unknown = 0
        self.block_table: list[int] = []
        self.temperature = sp.temperature
        self.max_tokens = sp.max_tokens
        self.ignore_eos = sp.ignore_eos

    def __len__(self):
        return self.num_tokens

    def __getitem__(self, key):
        return self.token_ids[key]

    @property
    def is_finished(self):
        return self.status is SequenceStatus.FINISHED

    @property
    def num_completion_tokens(self):
        return self.num_tokens - self.num_prompt_tokens

    @property
    def prompt_token_ids(self):
        return self.token_ids[:self.num_prompt_tokens]

    @property
    def completion_token_ids(self):
        return self.token_ids[self.num_prompt_tokens:]

    @property
    def num_cached_blocks(self):
        return self.num_cached_tokens // self.block_size

    @property
    def num_blocks(self):
        return -(-self.num_tokens // self.block_size)

    @property
    def last_block_num_tokens(self):
        return self.num_tokens - (self.num_blocks - 1) * self.block_size

    def block(self, i: int) -> list[int]:
        assert 0 <= i < self.num_blocks
        return self.token_ids[i * self.block_size:(i + 1) * self.block_size]

    def append_token(self, token_id: int):
        self.token_ids.append(token_id)
        self.last_token = token_id
        self.num_tokens += 1

    def append_unknown(self):
        """Lengthen the sequence by a token whose value arrives later (``patch_oldest_unknown``)."""
        self.token_ids.append(0)
        self.last_token = 0
        self.num_tokens += 1
        self.num_unknown += 1

    def patch_oldest_unknown(self, token_id: int):
        assert self.num_unknown > 0
        at = self.num_tokens - self.num_unknown
        self.token_ids[at] = token_id
        if at == self.num_tokens - 1:
            self.last_token = token_id
        self.num_unknown -= 1

    @property
    def num_known_tokens(self):
        return self.num_tokens - self.num_unknown
