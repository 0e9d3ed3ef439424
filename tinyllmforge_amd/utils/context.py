"""Attention metadata side channel (reference: tinyvllm/utils/context.py:5-27).

``Attention`` and ``ParallelLMHead`` do not take the step's metadata as arguments: the model runner
publishes it here before each forward pass and the layers read it back, which keeps the layer
signatures those of the reference.  One ``Context`` object lives for the whole process and is
rewritten in place (a decode step publishes three tensors a thousand times per request batch;
nothing is allocated for that), so a caller must not hold on to ``get_context()`` across steps.
"""
from __future__ import annotations

# field -> value after reset_context(), in the positional order of set_context()
_FIELDS = (
    ("is_prefill", False),      # prefill or decode step
    ("cu_seqlens_q", None),     # prefill: int32 [B + 1] prefix sums of the query lengths
    ("cu_seqlens_k", None),     # prefill: the same for the key lengths (cached prefix included)
    ("max_seqlen_q", 0),        # prefill
    ("max_seqlen_k", 0),        # prefill
    ("slot_mapping", None),     # both: int32 [N] cache slot of every token of the step
    ("context_lens", None),     # decode: int32 [B] tokens per sequence, the new one included
    ("block_tables", None),     # decode, and prefill with a prefix hit: int32 [B, max blocks]
    ("decode_plan", None),      # decode (no counterpart in the reference): the step's work split for the attention
                                # kernel, made once by the model runner for all layers (ops.paged_decode_plan)
)


class Context:
    __slots__ = tuple(name for name, _ in _FIELDS)

    def __init__(self):
        self.clear()

    def clear(self):
        for name, default in _FIELDS:
            setattr(self, name, default)

    def __repr__(self):
        return "Context(" + ", ".join(f"{n}={getattr(self, n)!r}" for n, _ in _FIELDS) + ")"


_CURRENT = Context()


def get_context() -> Context:
    return _CURRENT


def set_context(is_prefill, cu_seqlens_q=None, cu_seqlens_k=None, max_seqlen_q=0, max_seqlen_k=0, slot_mapping=None,
                context_lens=None, block_tables=None, decode_plan=None):
    """Publish one step's metadata; every argument after the first is optional, positional or by name
    (the parameter list of tinyvllm/utils/context.py:21, then ``decode_plan``)."""
    c = _CURRENT
    c.is_prefill = is_prefill
    c.cu_seqlens_q, c.cu_seqlens_k = cu_seqlens_q, cu_seqlens_k
    c.max_seqlen_q, c.max_seqlen_k = max_seqlen_q, max_seqlen_k
    c.slot_mapping, c.context_lens, c.block_tables = slot_mapping, context_lens, block_tables
    c.decode_plan = decode_plan


def reset_context():
    _CURRENT.clear()
