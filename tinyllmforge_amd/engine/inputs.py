"""Integer inputs of the hot path, built on the host from the scheduler's sequences.

Pure functions (numpy in, numpy out) so that slot mapping and block indexing can be checked
bit-exactly without a GPU.  They restate the reference's list-building loops
(tinyvllm/engine/model_runner.py:155-159, 164-205, 210-228) with vectorised index arithmetic.
"""
from __future__ import annotations

import numpy as np


def block_tables_array(seqs, pad: int = -1, width: int | None = None) -> np.ndarray:
    """int32 ``[len(seqs), width]``; rows padded with ``pad`` (reference pads with -1 to the batch max)."""
    w = max(len(s.block_table) for s in seqs)
    if width is not None:
        assert width >= w
        w = width
    out = np.full((len(seqs), w), pad, dtype=np.int32)
    for i, s in enumerate(seqs):
        out[i, :len(s.block_table)] = s.block_table
    return out


def prefill_inputs(seqs, block_size: int) -> dict:
    """Inputs of one prefill step (model_runner.py:164-205).

    input_ids / positions cover the uncached tail of every prompt; the slot of token ``t`` of a
    sequence is ``block_table[t // block_size] * block_size + t % block_size`` for every token
    from the first uncached *block* on; ``block_tables`` is only built when some sequence has
    a cached prefix (then the attention reads K/V of every sequence from the paged cache).
    """
    ids, pos, slots = [], [], []
    cu_q, cu_k = [0], [0]
    max_q = max_k = 0
    for s in seqs:
        n, c = len(s), s.num_cached_tokens
        ids.append(np.asarray(s.token_ids[c:n], dtype=np.int64))
        pos.append(np.arange(c, n, dtype=np.int64))
        cu_q.append(cu_q[-1] + (n - c))
        cu_k.append(cu_k[-1] + n)
        max_q, max_k = max(max_q, n - c), max(max_k, n)
        if not s.block_table:
            continue                                # warm-up sequences have no blocks
        t = np.arange(s.num_cached_blocks * block_size, n, dtype=np.int64)
        table = np.asarray(s.block_table, dtype=np.int64)
        slots.append(table[t // block_size] * block_size + t % block_size)
    cat = lambda xs, dt: np.concatenate(xs).astype(dt) if xs else np.zeros(0, dtype=dt)
    out = dict(
        input_ids=cat(ids, np.int64), positions=cat(pos, np.int64), slot_mapping=cat(slots, np.int32),
        cu_seqlens_q=np.asarray(cu_q, dtype=np.int32), cu_seqlens_k=np.asarray(cu_k, dtype=np.int32),
        max_seqlen_q=max_q, max_seqlen_k=max_k, block_tables=None,
    )
    if cu_k[-1] > cu_q[-1]:
        out["block_tables"] = block_tables_array(seqs)
    return out


def decode_inputs(seqs, block_size: int, position_quirk: bool = True) -> dict:
    """Inputs of one decode step (model_runner.py:210-228).

    The fed token is the last one (index ``len - 1``); its K/V go to slot
    ``block_table[-1] * block_size + last_block_num_tokens - 1``; ``context_lens = len``.
    The reference feeds ``positions = len(seq)`` (one past the token's index, model_runner.py:219);
    ``position_quirk=False`` gives ``len - 1`` instead.
    """
    n = np.asarray([len(s) for s in seqs], dtype=np.int64)
    last_blk = np.asarray([s.block_table[-1] for s in seqs], dtype=np.int64)
    nblocks = -(-n // block_size)
    last_cnt = n - (nblocks - 1) * block_size
    return dict(
        input_ids=np.asarray([s.last_token for s in seqs], dtype=np.int64),
        positions=(n if position_quirk else n - 1).astype(np.int64),
        slot_mapping=(last_blk * block_size + last_cnt - 1).astype(np.int32),
        context_lens=n.astype(np.int32),
        block_tables=block_tables_array(seqs),
    )
