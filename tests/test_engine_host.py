"""Host logic (CPU): sequence block math, block manager order and hashing, scheduler policy,
and the integer inputs of the hot path (slot mapping, block tables, positions) - bit exact.

Pins: closed forms on hand-built states (block boundaries len % 256 in {0, 1, 255}), the
xxh64 library as known answer, and the invariants slot // bs == block_table[pos // bs],
slot % bs == pos % bs.
"""
import numpy as np
import pytest
import xxhash

from tinyllmforge_amd.config import Config, ModelConfig, QWEN3_SHAPES
from tinyllmforge_amd.engine import inputs as I
from tinyllmforge_amd.engine.block_manager import BlockManager
from tinyllmforge_amd.engine.scheduler import Scheduler
from tinyllmforge_amd.engine.sequence import Sequence, SequenceStatus
from tinyllmforge_amd.sampling_params import SamplingParams

BS = 256


@pytest.fixture(autouse=True)
def _bs():
    Sequence.block_size = BS
    yield


def seq(n, start=0, **kw):
    return Sequence(list(range(start, start + n)), SamplingParams(**kw) if kw else None)


@pytest.mark.parametrize("n,blocks,last", [(1, 1, 1), (255, 1, 255), (256, 1, 256), (257, 2, 1), (512, 2, 256), (513, 3, 1)])
def test_sequence_block_math(n, blocks, last):
    s = seq(n)
    assert (len(s), s.num_blocks, s.last_block_num_tokens) == (n, blocks, last)
    assert s.block(blocks - 1) == list(range((blocks - 1) * BS, n))
    s.append_token(7)
    assert len(s) == n + 1 and s.last_token == 7 and s.num_completion_tokens == 1 and s.completion_token_ids == [7]


def test_block_hash_known_answers():
    assert xxhash.xxh64(b"").intdigest() == 0xEF46DB3751D8E999            # published xxh64 vector (seed 0)
    toks = [5, 0, 2 ** 40, 9]
    raw = np.array(toks, dtype=np.int64).tobytes()
    assert len(raw) == 32 and raw[:8] == (5).to_bytes(8, "little")
    assert BlockManager.compute_hash(toks) == xxhash.xxh64(raw).intdigest()
    pre = 0x1234567890ABCDEF
    assert BlockManager.compute_hash(toks, pre) == xxhash.xxh64(pre.to_bytes(8, "little") + raw).intdigest()
    assert BlockManager.compute_hash(toks, pre) != BlockManager.compute_hash(toks)


def test_block_manager_fifo_order_prefix_hits_and_revival():
    bm = BlockManager(8, BS)
    a = seq(600)                                     # 3 blocks: two full, one partial
    assert bm.can_allocate(a)
    bm.allocate(a)
    assert a.block_table == [0, 1, 2] and a.num_cached_tokens == 0
    assert bm.blocks[0].hash != -1 and bm.blocks[2].hash == -1        # only full blocks are hashed
    b = Sequence(list(range(512)) + [9999] * 10)                      # shares two full blocks
    bm.allocate(b)
    assert b.block_table == [0, 1, 3] and b.num_cached_tokens == 512
    assert bm.blocks[0].ref_count == 2
    bm.deallocate(a)
    assert list(bm.free_block_ids) == [4, 5, 6, 7, 2]                 # freed to the right, shared blocks stay
    bm.deallocate(b)
    assert list(bm.free_block_ids) == [4, 5, 6, 7, 2, 3, 1, 0]        # reversed table order
    c = seq(300)                                                      # first block revived by its hash
    bm.allocate(c)
    assert c.block_table == [0, 4] and c.num_cached_tokens == 256
    d = Sequence([1] + list(range(1, 600)))                           # first block differs: all fresh
    bm.allocate(d)
    assert d.num_cached_tokens == 0 and d.block_table == [5, 6, 7]


def test_block_manager_full_hit_recomputes_last_block():
    bm = BlockManager(4, BS)
    a = seq(512)
    bm.allocate(a)
    b = seq(512)
    bm.allocate(b)
    assert b.block_table == [0, 1]
    assert b.num_cached_tokens == 256           # never equal to len: at least the last block is prefilled


def test_block_manager_append_protocol():
    bm = BlockManager(4, BS)
    s = seq(255)
    bm.allocate(s)
    s.append_token(1)                            # len 256: block becomes full on may_append
    assert bm.can_append(s)
    bm.may_append(s)
    assert bm.blocks[s.block_table[-1]].hash == BlockManager.compute_hash(s.block(0))
    s.append_token(2)                            # len 257: needs a new block
    assert bm.can_append(s) == (len(bm.free_block_ids) >= 1)
    bm.may_append(s)
    assert s.block_table == [0, 1]
    s.append_token(3)
    bm.may_append(s)                             # nothing to do in the middle of a block
    assert s.block_table == [0, 1]


def _cfg(**kw):
    base = dict(model=QWEN3_SHAPES["qwen3-0.6b"], num_kvcache_blocks=8, max_num_seqs=4, max_num_batched_tokens=4096,
                max_model_len=2048)
    base.update(kw)
    return Config(**base)


def test_scheduler_prefill_first_then_decode_and_finish():
    sch = Scheduler(_cfg())
    seqs = [seq(100, max_tokens=2, ignore_eos=True) for _ in range(3)]
    for s in seqs:
        sch.add(s)
    batch, is_prefill = sch.schedule()
    assert is_prefill and batch == seqs and all(s.status is SequenceStatus.RUNNING for s in seqs)
    sch.postprocess(batch, [1, 2, 3])
    batch, is_prefill = sch.schedule()
    assert not is_prefill and batch == seqs
    sch.postprocess(batch, [4, 5, 6])
    assert sch.is_finished() and all(s.is_finished for s in seqs)
    assert len(sch.block_manager.free_block_ids) == 8
    assert seqs[1].completion_token_ids == [2, 5]


def test_scheduler_token_budget_and_seq_limit():
    sch = Scheduler(_cfg(max_num_batched_tokens=2048, max_num_seqs=2, num_kvcache_blocks=32))
    for n in (1500, 600, 100):
        sch.add(seq(n, max_tokens=1))
    batch, _ = sch.schedule()
    assert [len(s) for s in batch] == [1500]           # 1500 + 600 > 2048
    sch.postprocess(batch, [0])
    batch, _ = sch.schedule()
    assert [len(s) for s in batch] == [600, 100]       # limited by max_num_seqs = 2


def test_scheduler_preempts_newest_when_out_of_blocks():
    sch = Scheduler(_cfg(num_kvcache_blocks=2))
    a, b = seq(256, max_tokens=8, ignore_eos=True), seq(256, start=1000, max_tokens=8, ignore_eos=True)
    sch.add(a); sch.add(b)
    batch, is_prefill = sch.schedule()
    assert is_prefill and len(batch) == 2
    sch.postprocess(batch, [1, 1])                      # both at 257 tokens: each needs a new block, none free
    batch, is_prefill = sch.schedule()
    assert not is_prefill and batch == [a]              # b (newest) preempted, its block goes to a
    assert b.status is SequenceStatus.WAITING and not b.block_table and sch.waiting[0] is b
    assert a.block_table == [0, 1]


def test_eos_stops_unless_ignored():
    cfg = _cfg(); cfg.eos = 42
    sch = Scheduler(cfg)
    a, b = seq(10, max_tokens=5), seq(10, max_tokens=5, ignore_eos=True)
    sch.add(a); sch.add(b)
    batch, _ = sch.schedule()
    sch.postprocess(batch, [42, 42])
    assert a.is_finished and not b.is_finished


def test_sequence_is_finished_before_its_position_leaves_the_rope_table():
    """A decode step feeds position len(seq) (len(seq) - 1 without the reference's quirk) into a RoPE table of
    max_position_embeddings rows: the scheduler ends a sequence whose next step would index past it."""
    for quirk, last_len in ((True, 512), (False, 513)):
        cfg = _cfg(model=dict(QWEN3_SHAPES["qwen3-0.6b"], max_position_embeddings=512), max_model_len=512,
                   decode_position_quirk=quirk)
        sch = Scheduler(cfg)
        s = seq(508, max_tokens=100, ignore_eos=True)
        sch.add(s)
        positions = []
        while not sch.is_finished():
            batch, is_prefill = sch.schedule()
            if not is_prefill:
                positions.append(int(I.decode_inputs(batch, 256, quirk)["positions"][0]))
            sch.postprocess(batch, [7])
        assert len(s) == last_len and max(positions) == 511, (quirk, len(s), positions)


# ----------------------------------------------------------------------------- integer inputs
def test_prefill_inputs_closed_form_no_prefix():
    bm = BlockManager(16, BS)
    seqs = [seq(300), seq(256, start=5000), seq(1, start=9000)]
    for s in seqs:
        bm.allocate(s)
    d = I.prefill_inputs(seqs, BS)
    assert d["input_ids"].dtype == np.int64 and d["positions"].dtype == np.int64
    assert d["slot_mapping"].dtype == np.int32 and d["cu_seqlens_q"].dtype == np.int32
    assert d["cu_seqlens_q"].tolist() == [0, 300, 556, 557] == d["cu_seqlens_k"].tolist()
    assert (d["max_seqlen_q"], d["max_seqlen_k"]) == (300, 300) and d["block_tables"] is None
    assert d["input_ids"].tolist() == list(range(300)) + list(range(5000, 5256)) + [9000]
    assert d["positions"].tolist() == list(range(300)) + list(range(256)) + [0]
    # blocks were handed out in order 0,1 | 2 | 3
    expect = list(range(0, 300)) + list(range(2 * 256, 3 * 256)) + [3 * 256]
    assert d["slot_mapping"].tolist() == expect
    # invariants: slot // bs is the table entry of the token's block, slot % bs its offset
    off = 0
    for s in seqs:
        n = len(s)
        sl = d["slot_mapping"][off:off + n]
        t = np.arange(n)
        assert (sl // BS == np.asarray(s.block_table)[t // BS]).all() and (sl % BS == t % BS).all()
        off += n


def test_prefill_inputs_with_prefix_hit():
    bm = BlockManager(16, BS)
    a = seq(700)
    bm.allocate(a)
    b = Sequence(list(range(512)) + [7] * 100)           # 512 cached tokens
    bm.allocate(b)
    c = seq(50, start=3000)
    bm.allocate(c)
    d = I.prefill_inputs([b, c], BS)
    assert d["cu_seqlens_q"].tolist() == [0, 100, 150] and d["cu_seqlens_k"].tolist() == [0, 612, 662]
    assert d["positions"].tolist() == list(range(512, 612)) + list(range(50))
    assert d["input_ids"][:100].tolist() == [7] * 100
    assert d["slot_mapping"].tolist() == [b.block_table[2] * BS + i for i in range(100)] + [c.block_table[0] * BS + i for i in range(50)]
    assert d["block_tables"].tolist() == [b.block_table, c.block_table + [-1, -1]]
    assert d["block_tables"].dtype == np.int32


@pytest.mark.parametrize("n", [1, 255, 256, 257, 511, 512, 513])
def test_decode_inputs_closed_form(n):
    bm = BlockManager(16, BS)
    s = seq(n)
    bm.allocate(s)
    other = seq(300, start=777)
    bm.allocate(other)
    for q in (s, other):
        q.append_token(11)
        bm.may_append(q)
    d = I.decode_inputs([s, other], BS)
    L = n + 1
    assert d["input_ids"].tolist() == [11, 11]
    assert d["positions"].tolist() == [L, 301]                      # the reference feeds len(seq), not len - 1
    assert I.decode_inputs([s], BS, position_quirk=False)["positions"].tolist() == [L - 1]
    assert d["context_lens"].tolist() == [L, 301]
    t = L - 1                                                       # index of the fed token
    assert d["slot_mapping"][0] == s.block_table[t // BS] * BS + t % BS
    assert d["slot_mapping"][1] == other.block_table[300 // BS] * BS + 300 % BS
    w = max(len(s.block_table), len(other.block_table))
    assert d["block_tables"].shape == (2, w)
    assert d["block_tables"][0, :len(s.block_table)].tolist() == s.block_table
    assert (d["block_tables"][0, len(s.block_table):] == -1).all()


def test_config_accepts_shape_names_and_dicts():
    c = Config("qwen3-8b")
    assert c.hf_config.hidden_size == 4096 and c.hf_config.head_dim == 128 and not c.hf_config.tie_word_embeddings
    c2 = Config(dict(hidden_size=256, num_hidden_layers=2, num_attention_heads=2, num_key_value_heads=1,
                     intermediate_size=512, max_position_embeddings=1024), max_model_len=4096, max_num_batched_tokens=4096)
    assert c2.max_model_len == 1024 and c2.hf_config.head_dim == 128
    with pytest.raises(AssertionError):
        Config("qwen3-8b", kvcache_block_size=100)
    with pytest.raises(AssertionError):
        Config("qwen3-8b", tensor_parallel_size=2)


def test_gate_up_interleave_index_is_the_stated_permutation():
    """Rows 16 j .. 16 j + 7 of the fused gate_up weight are gate channels 8 j .., rows 16 j + 8 .. 16 j + 15
    the matching up channels (ops.gate_up_interleave_index)."""
    import torch
    from tinyllmforge_amd import ops as P
    for n in (16, 32, 6144, 24576):
        idx = P.gate_up_interleave_index(n)
        assert sorted(idx.tolist()) == list(range(n))
        half = n // 2
        for j in range(0, n, 16):
            assert idx[j:j + 8].tolist() == list(range(j // 2, j // 2 + 8))
            assert idx[j + 8:j + 16].tolist() == list(range(half + j // 2, half + j // 2 + 8))


def test_safetensors_loader_and_offline_int8_checkpoint(tmp_path):
    """Weights on disk (loader.py:11-30): an HF-style checkpoint with q/k/v and gate/up stored apart loads
    into the packed parameters; the offline quantiser's int8 checkpoint loads to exactly the int8 weights,
    scales and gate/up row order that quantising the loaded bf16 model in memory gives."""
    import torch
    from safetensors.torch import save_file
    from tinyllmforge_amd.models.qwen3 import Qwen3ForCausalLM
    from tinyllmforge_amd.utils.loader import load_model, quantize_checkpoint, random_init_
    cfg = ModelConfig.from_any(dict(hidden_size=128, num_hidden_layers=2, num_attention_heads=2, num_key_value_heads=1,
                                     head_dim=64, intermediate_size=96, vocab_size=200, max_position_embeddings=64,
                                     tie_word_embeddings=False))
    torch.set_default_dtype(torch.bfloat16)
    try:
        src = random_init_(Qwen3ForCausalLM(cfg), seed=3)
        a, b = Qwen3ForCausalLM(cfg), Qwen3ForCausalLM(cfg)
    finally:
        torch.set_default_dtype(torch.float32)
    # unpack the way a HF checkpoint stores it, split over two files
    hf = {}
    for name, p in src.named_parameters():
        t = p.data
        if "qkv_proj" in name:
            attn = src.get_submodule(name.rsplit(".", 2)[0])
            q, k, v = t.split([attn.q_size, attn.kv_size, attn.kv_size], 0)
            for key, part in (("q_proj", q), ("k_proj", k), ("v_proj", v)):
                hf[name.replace("qkv_proj", key)] = part.contiguous()
        elif "gate_up_proj" in name:
            gate, up = t.chunk(2, 0)
            hf[name.replace("gate_up_proj", "gate_proj")] = gate.contiguous()
            hf[name.replace("gate_up_proj", "up_proj")] = up.contiguous()
        else:
            hf[name] = t.contiguous()
    names = sorted(hf)
    d16, d8 = tmp_path / "bf16", tmp_path / "int8"
    d16.mkdir()
    save_file({n: hf[n] for n in names[::2]}, str(d16 / "model-00001-of-00002.safetensors"))
    save_file({n: hf[n] for n in names[1::2]}, str(d16 / "model-00002-of-00002.safetensors"))
    load_model(a, str(d16))
    for (n1, p1), (n2, p2) in zip(src.named_parameters(), a.named_parameters()):
        assert n1 == n2 and torch.equal(p1.data, p2.data), n1
    quantize_checkpoint(str(d16), str(d8))
    load_model(b, str(d8))
    a.quantize_linears_()
    b.quantize_linears_()                       # nothing left to do for a checkpoint that is int8 already
    for la, lb in zip(a.model.layers, b.model.layers):
        for get in (lambda l: l.self_attn.qkv_proj, lambda l: l.self_attn.o_proj,
                    lambda l: l.mlp.gate_up_proj, lambda l: l.mlp.down_proj):
            ma, mb = get(la), get(lb)
            assert mb.qweight.dtype == torch.int8 and mb.weight.numel() == 0
            assert torch.equal(ma.qweight, mb.qweight) and torch.equal(ma.qscale, mb.qscale)
        assert la.mlp.gate_up_proj.interleaved and lb.mlp.gate_up_proj.interleaved
    assert torch.equal(a.model.embed_tokens.weight, b.model.embed_tokens.weight)
    assert torch.equal(a.lm_head.weight, b.lm_head.weight) and torch.equal(a.model.norm.weight, b.model.norm.weight)


# ----------------------------------------------------------------------------- decode steps that run ahead
def _simulate(ahead, depth, nblk, seed, block_size=16, arrivals=False):
    """The engine loop without a model: a step's tokens are a fixed function of (sequence, length), and in the
    run-ahead form they reach the scheduler ``depth`` steps late (postprocess_ahead now, patch later).
    ``arrivals``: five of the twelve requests are added while the loop runs (after a given number of steps, or when
    the engine falls idle), two of them may end on EOS, and one of those does."""
    import itertools
    import random
    from collections import deque
    from tinyllmforge_amd.config import Config
    from tinyllmforge_amd.engine.block_manager import BlockManager
    from tinyllmforge_amd.engine.scheduler import Scheduler
    from tinyllmforge_amd.engine.sequence import Sequence
    from tinyllmforge_amd.sampling_params import SamplingParams
    rnd = random.Random(seed)
    cfg = Config("qwen3-0.6b", num_kvcache_blocks=nblk, max_num_seqs=8, max_num_batched_tokens=4096, max_model_len=2048)
    old_bs, old_ids = Sequence.block_size, Sequence._ids
    Sequence.block_size, Sequence._ids = block_size, itertools.count(1000)
    try:
        sch = Scheduler(cfg)
        sch.block_manager = BlockManager(nblk, block_size)
        seqs = [Sequence([rnd.randint(0, 99) for _ in range(rnd.randint(3, 60))],
                         SamplingParams(temperature=0.0, max_tokens=rnd.randint(5, 90), ignore_eos=True)) for _ in range(12)]
        tok = lambda s, n: (s.seq_id * 7919 + n * 31) % 1000
        pending = []
        if arrivals:
            for s in (seqs[8], seqs[10]):
                s.ignore_eos = False
            sch.eos = tok(seqs[8], len(seqs[8]) + 4)      # the fifth token of seqs[8]
            pending = list(zip((10, 25, 25, 60, 100), seqs[7:]))
            seqs_at_start = seqs[:7]
        else:
            seqs_at_start = seqs
        for s in seqs_at_start:
            sch.add(s)
        inflight, trace, ran_ahead = deque(), [], 0
        while True:
            while pending and (pending[0][0] <= len(trace) or sch.is_finished()):
                sch.add(pending.pop(0)[1])
            if sch.is_finished():
                if not inflight:
                    break
                sch.patch(*inflight.popleft())
                continue
            if ahead and sch.can_run_ahead():
                while len(inflight) >= depth:
                    sch.patch(*inflight.popleft())
                batch, prefill = sch.schedule()
                assert not prefill
                trace.append(("d", [s.seq_id for s in batch], [list(s.block_table) for s in batch]))
                inflight.append((batch, [tok(s, len(s)) for s in batch]))
                sch.postprocess_ahead(batch)
                ran_ahead += 1
            else:
                while inflight:
                    sch.patch(*inflight.popleft())
                batch, prefill = sch.schedule()
                trace.append(("p" if prefill else "d", [s.seq_id for s in batch], [list(s.block_table) for s in batch]))
                sch.postprocess(batch, [tok(s, len(s)) for s in batch])
        bm = sch.block_manager
        assert not bm.unsealed and not bm.used_block_ids and all(s.num_unknown == 0 for s in seqs)
        return dict(trace=trace, tokens=[s.token_ids for s in seqs], hashes=dict(bm.hash_to_block_id),
                    free=list(bm.free_block_ids), blocks=[(b.hash, b.token_ids) for b in bm.blocks], ran_ahead=ran_ahead,
                    ended_on_eos=[s.seq_id for s in seqs if not s.ignore_eos and s.num_completion_tokens < s.max_tokens])
    finally:
        Sequence.block_size, Sequence._ids = old_bs, old_ids


@pytest.mark.parametrize("nblk", [40, 14, 9])
@pytest.mark.parametrize("depth", [1, 2, 4])
def test_run_ahead_bookkeeping_equals_the_step_by_step_loop(nblk, depth):
    """Token values that arrive ``depth`` steps late (stand-ins appended, values patched in, full blocks sealed when
    their tokens are known) leave every step's sequences and block tables, the token lists, the prefix-cache hashes,
    the free list and the blocks exactly as the step-by-step loop does: with room to spare (40 blocks of 16 tokens),
    with preemption (14) and with most sequences waiting most of the time (9)."""
    for seed in range(4):
        a = _simulate(False, depth, nblk, seed)
        b = _simulate(True, depth, nblk, seed)
        for key in ("trace", "tokens", "hashes", "free", "blocks"):
            assert a[key] == b[key], (key, seed)
        decode_steps = sum(1 for t in a["trace"] if t[0] == "d")
        assert a["ran_ahead"] == 0 and b["ran_ahead"] == decode_steps > 50
    if nblk < 40:
        assert sum(1 for t in a["trace"] if t[0] == "p") > 3      # preempted sequences were prefilled again


@pytest.mark.parametrize("nblk", [40, 12])
def test_run_ahead_with_requests_that_arrive_while_steps_are_in_flight(nblk):
    """Requests added between steps (a serving loop) while decode steps are in flight: the loop drains and takes the
    newcomer's prefill exactly where the step-by-step loop does; while a sequence that may end on EOS is running no
    step runs ahead, and after it has ended (one does end on EOS, at its fifth token) the steps run ahead again."""
    for seed in range(4):
        a = _simulate(False, 2, nblk, seed, arrivals=True)
        b = _simulate(True, 2, nblk, seed, arrivals=True)
        for key in ("trace", "tokens", "hashes", "free", "blocks"):
            assert a[key] == b[key], (key, seed)
        decode_steps = sum(1 for t in a["trace"] if t[0] == "d")
        assert a["ran_ahead"] == 0 and 10 < b["ran_ahead"] < decode_steps
        assert len(a["ended_on_eos"]) >= 1 and a["ended_on_eos"] == b["ended_on_eos"]


def test_run_ahead_is_refused_when_a_sequence_may_end_on_a_token_value():
    from tinyllmforge_amd.config import Config
    from tinyllmforge_amd.engine.scheduler import Scheduler
    from tinyllmforge_amd.engine.sequence import Sequence
    from tinyllmforge_amd.sampling_params import SamplingParams
    sch = Scheduler(Config("qwen3-0.6b", num_kvcache_blocks=8, max_num_seqs=4, max_model_len=1024))
    a = Sequence([1, 2, 3], SamplingParams(temperature=0.0, max_tokens=4, ignore_eos=True))
    b = Sequence([4, 5, 6], SamplingParams(temperature=0.0, max_tokens=4, ignore_eos=False))
    sch.add(a)
    assert not sch.can_run_ahead()                 # a prefill comes first
    batch, prefill = sch.schedule()
    sch.postprocess(batch, [7])
    assert prefill and sch.can_run_ahead()
    sch.add(b)
    assert not sch.can_run_ahead()                 # the newcomer fits: the next step is its prefill
    batch, prefill = sch.schedule()
    sch.postprocess(batch, [8])
    assert prefill and not sch.can_run_ahead()     # b may end on EOS
