"""Continuous batching: prefill first, decode with preemption from the tail
(reference: tinyvllm/engine/scheduler.py:8-72)."""
from __future__ import annotations

from collections import deque

from ..config import Config
from .block_manager import BlockManager
from .sequence import Sequence, SequenceStatus


class Scheduler:
    def __init__(self, config: Config):
        self.max_num_seqs = config.max_num_seqs
        self.max_num_batched_tokens = config.max_num_batched_tokens
        self.eos = config.eos
        # The RoPE table has max_position_embeddings rows and a decode step feeds position len(seq)
        # (len(seq) - 1 without the reference's quirk): a sequence that would step past the table
        # is finished instead (the reference indexes out of range there).
        self.max_len = config.hf_config.max_position_embeddings + (0 if config.decode_position_quirk else 1)
        self.block_manager = BlockManager(config.num_kvcache_blocks, config.kvcache_block_size)
        self.waiting: deque[Sequence] = deque()
        self.running: deque[Sequence] = deque()

    def is_finished(self) -> bool:
        return not self.waiting and not self.running

    def add(self, seq: Sequence):
        self.waiting.append(seq)

    def schedule(self) -> tuple[list[Sequence], bool]:
        """The next step's sequences and whether it is a prefill step.  Prefill has priority: a step
        never mixes the two kinds (scheduler.py:22-57)."""
        admitted = self._admit_waiting()
        if admitted:
            return admitted, True
        return self._step_running(), False

    def _admit_waiting(self) -> list[Sequence]:
        # admission looks at the full length, the budget is charged the uncached part (scheduler.py:29,33)
        batch: list[Sequence] = []
        charged = 0
        while self.waiting and len(batch) < self.max_num_seqs:
            head = self.waiting[0]
            fits = charged + len(head) <= self.max_num_batched_tokens and self.block_manager.can_allocate(head)
            if not fits:
                break
            self.block_manager.allocate(head)
            charged += len(head) - head.num_cached_tokens
            head.status = SequenceStatus.RUNNING
            self.running.append(self.waiting.popleft())
            batch.append(head)
        return batch

    def _step_running(self) -> list[Sequence]:
        # every running sequence gets one token; when no block is left for one of them, the newest
        # running sequence is preempted (freed, back to the head of the waiting queue) until it fits,
        # the sequence itself if it is the last one left
        batch: list[Sequence] = []
        while self.running and len(batch) < self.max_num_seqs:
            seq = self.running.popleft()
            while not self.block_manager.can_append(seq) and self.running:
                self.preempt(self.running.pop())
            if self.block_manager.can_append(seq):
                self.block_manager.may_append(seq)
                batch.append(seq)
            else:
                self.preempt(seq)
        assert batch
        self.running.extendleft(reversed(batch))
        return batch

    def preempt(self, seq: Sequence):
        seq.status = SequenceStatus.WAITING
        self.block_manager.deallocate(seq)
        self.waiting.appendleft(seq)

    def postprocess(self, seqs: list[Sequence], token_ids: list[int]):
        for seq, tok in zip(seqs, token_ids):
            seq.append_token(tok)
            hit_eos = (not seq.ignore_eos) and tok == self.eos
            if hit_eos or seq.num_completion_tokens == seq.max_tokens or len(seq) >= self.max_len:
                seq.status = SequenceStatus.FINISHED
                self.block_manager.deallocate(seq)
                self.running.remove(seq)

    # -- a decode step that runs ahead of the read-back of its tokens (no counterpart in the reference, whose
    #    step waits for its token ids): legal while no sequence of the step can end on a token VALUE
    def can_run_ahead(self) -> bool:
        """The next step is a decode step (nothing waits, or the head of the queue does not fit now: the same test
        as in ``_admit_waiting``) of sequences that ignore EOS."""
        if not self.running or not all(s.ignore_eos for s in self.running):
            return False
        if self.waiting and self.max_num_seqs > 0:
            head = self.waiting[0]
            if len(head) <= self.max_num_batched_tokens and self.block_manager.can_allocate(head):
                return False
        return True

    def postprocess_ahead(self, seqs: list[Sequence]):
        """``postprocess`` without the token values: lengths, finishing by length and block release as there;
        the values follow through ``patch``."""
        for seq in seqs:
            assert seq.ignore_eos
            seq.append_unknown()
            if seq.num_completion_tokens == seq.max_tokens or len(seq) >= self.max_len:
                seq.status = SequenceStatus.FINISHED
                self.block_manager.deallocate(seq)
                self.running.remove(seq)

    def patch(self, seqs: list[Sequence], token_ids: list[int]):
        """The token values of the oldest step that ran ahead, then the seals that waited for them."""
        for seq, tok in zip(seqs, token_ids):
            seq.patch_oldest_unknown(tok)
        self.block_manager.seal_known()
