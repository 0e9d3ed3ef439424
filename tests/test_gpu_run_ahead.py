"""Decode steps that run ahead of the read-back of their token ids (Config.run_ahead) against the step-by-step
loop of the reference (tinyvllm/engine/llm_engine.py:53-59): same tokens, same step counts, same block ids and
prefix-cache state, with sequences ending at different lengths, preemption out of a small KV pool, a
temperature > 0, and a sequence that may end on EOS (which takes the step-by-step loop)."""
import os
import sys

import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

pytestmark = pytest.mark.gpu


def small_config():
    from tinyllmforge_amd.config import QWEN3_SHAPES
    return dict(QWEN3_SHAPES["qwen3-0.6b"], num_hidden_layers=3, max_position_embeddings=4096)


def prompts_and_params(n, temperature, seed, eos_free=True, eos_index=3):
    from random import Random
    from tinyllmforge_amd import SamplingParams
    r = Random(seed)
    prompts = [[r.randint(0, 9999) for _ in range(r.randint(20, 700))] for _ in range(n)]
    sps = [SamplingParams(temperature=temperature, ignore_eos=eos_free or i != eos_index, max_tokens=r.randint(3, 300)) for i in range(n)]
    return prompts, sps


def run(run_ahead, blocks, temperature, eos_free=True, quantization="w8a16", arrivals=None, eos_index=3):
    """arrivals: [(step, request index), ...] - requests added after that many engine steps (or when the engine falls
    idle before); every other request is there from the start."""
    from tinyllmforge_amd import LLM
    llm = LLM(small_config(), max_model_len=2048, max_num_batched_tokens=4096, max_num_seqs=16, num_kvcache_blocks=blocks,
              enforce_eager=False, seed=3, quantization=quantization, run_ahead=run_ahead)
    try:
        llm.config.eos = 17      # only matters for the sequence that does not ignore it
        llm.scheduler.eos = 17
        prompts, sps = prompts_and_params(14, temperature, seed=5, eos_free=eos_free, eos_index=eos_index)
        trace = []
        pending = sorted(arrivals or [])
        late = {i for _, i in pending}
        for i, (p, sp) in enumerate(zip(prompts, sps)):
            if i not in late:
                llm.add_request(p, sp)
        done = {}
        while pending or not llm.is_finished():
            while pending and (pending[0][0] <= len(trace) or llm.is_finished()):
                i = pending.pop(0)[1]
                llm.add_request(prompts[i], sps[i])
            finished, n = llm.step()
            trace.append(n)
            for sid, toks in finished:
                assert sid not in done
                done[sid] = list(toks)
        bm = llm.scheduler.block_manager
        first = min(done)
        state = dict(tokens=[done[k] for k in sorted(done)], trace=trace, free=list(bm.free_block_ids), ahead=llm.steps_ahead,
                     hashes={h: b for h, b in bm.hash_to_block_id.items()}, blocks=[(b.hash, b.ref_count) for b in bm.blocks])
        assert not bm.used_block_ids and not bm.unsealed and not llm._ahead
        return state
    finally:
        llm.exit()
        del llm
        import gc
        gc.collect()
        torch.cuda.empty_cache()


@pytest.mark.parametrize("blocks,temperature", [(64, 0.0), (9, 0.0), (64, 0.7), (9, 0.7)])
def test_run_ahead_equals_the_step_by_step_loop(blocks, temperature):
    """64 blocks: no pressure; 9 blocks of 256 tokens for 14 sequences of up to 1000 tokens: sequences are
    preempted and re-prefilled, which the run-ahead loop has to notice (it drains before every prefill)."""
    a = run(False, blocks, temperature)
    b = run(True, blocks, temperature)
    assert len(a["tokens"]) == 14 and all(len(t) >= 3 for t in a["tokens"])
    assert a["trace"] == b["trace"], "step kinds and sizes differ"
    assert a["tokens"] == b["tokens"]
    assert a["free"] == b["free"] and a["hashes"] == b["hashes"] and a["blocks"] == b["blocks"]
    decode_steps = sum(1 for n in a["trace"] if n < 0)
    assert decode_steps > 100 and a["ahead"] == 0
    # every decode step ran ahead, whether or not preempted sequences were waiting for blocks
    assert b["ahead"] == decode_steps, (b["ahead"], decode_steps)


def test_a_sequence_that_may_end_on_eos_keeps_the_step_by_step_loop():
    a = run(False, 64, 0.0, eos_free=False)
    b = run(True, 64, 0.0, eos_free=False)
    assert a["tokens"] == b["tokens"] and a["trace"] == b["trace"] and a["hashes"] == b["hashes"]
    assert 0 < b["ahead"] < sum(1 for n in b["trace"] if n < 0)     # only after that sequence has ended


def test_requests_that_arrive_while_steps_are_in_flight():
    """A serving loop: five requests are added between steps while decode steps are in flight, one of them may end on
    EOS.  The loop drains and takes each newcomer's prefill where the step-by-step loop does."""
    arrivals = [(5, 9), (20, 10), (20, 11), (60, 12), (120, 13)]
    a = run(False, 64, 0.0, eos_free=False, arrivals=arrivals, eos_index=11)
    b = run(True, 64, 0.0, eos_free=False, arrivals=arrivals, eos_index=11)
    assert len(a["tokens"]) == 14
    assert a["tokens"] == b["tokens"] and a["trace"] == b["trace"]
    assert a["free"] == b["free"] and a["hashes"] == b["hashes"] and a["blocks"] == b["blocks"]
    assert sum(1 for n in a["trace"] if n > 0) >= 5            # the first batch and at least four later prefills
    assert 20 < b["ahead"] < sum(1 for n in b["trace"] if n < 0)


def test_run_ahead_with_bf16_linears_and_logits():
    """bf16 linears, temperature 0: the LM head + argmax epilogue; the ids never touch the host between steps."""
    a = run(False, 64, 0.0, quantization=None)
    b = run(True, 64, 0.0, quantization=None)
    assert a["tokens"] == b["tokens"] and a["trace"] == b["trace"]
