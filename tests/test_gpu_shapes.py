"""GPU parity at the benchmark configurations' own shapes.

* BASELINE config 2 (paged decode attention, B = 64, 2048-block pool: cache offsets pass 2^31 bytes) against
  the oracle on sampled rows, bf16 and e4m3 rows.
* The Qwen3-8B-shaped engine (config 4: 36 layers, hidden 4096, 32 / 8 heads, intermediate 12288), W8A16 and
  bf16 linears, on sequences of the benchmark's recipe: graph decode == eager decode, fused == unfused layer
  path, step statistics, block manager clean at the end; its KV pool is larger than 2 GiB per layer side and
  the blocks in use are taken from its far end.
* The Qwen3-32B-shaped engine at its own depth (config 5: 64 layers, hidden 5120, 64 / 8 heads, intermediate
  25600), W8A16 linears, e4m3 KV cache, prompts of 2048 ... 8192 tokens of which two share a 1024-token prefix held
  in cached blocks: graph decode == eager decode, fused == unfused layer path, prefix hits counted, block
  manager clean.
* Two-layer decoders at the 8B and 32B WIDTHS against the CPU oracle, teacher-forced: final hidden state and
  whole logit rows at every step.  The 32B-width run uses W8A16 linears, an e4m3 KV cache with a different
  scale per KV head and layer, and a 1024-token prefix held in cached blocks (config 5).
"""
import os
import sys

import pytest
import torch

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


# ----------------------------------------------------------------------------- config 2 at full size
@pytest.mark.parametrize("fp8,hq", [(False, 32), (True, 64)])
def test_config2_full_size_sampled_rows_against_the_oracle(fp8, hq):
    """B = 64, ctx ~ U[512, 4096], 2048-block pool (1 GiB per cache side in bf16: byte offsets beyond 2^31 are
    reached through the random block permutation), K/V written through the store kernel.  Rows of 10 sampled
    sequences (the longest, the shortest and the ones owning the highest block ids among them) are compared
    with ``oracle.ops.paged_decode_attention`` on a copy of just their blocks."""
    from bench import make_decode_case
    from oracle import ops as O
    from tinyllmforge_amd import ops as P
    case = make_decode_case(batch=64, hq=hq, fp8=fp8)
    out = P.paged_decode_attention(case["q"], case["k_cache"], case["v_cache"], case["ctx"], case["bt"], case["scale"],
                                   **case["scales"]).cpu()
    ctx, bt = case["ctx_cpu"], case["bt_cpu"]
    assert int(bt.max()) >= 2000 and case["k_cache"].numel() * case["k_cache"].element_size() == (1 << (29 if fp8 else 30))
    by_len = torch.argsort(ctx)
    by_blk = torch.argsort(bt.max(dim=1).values)
    rows = sorted(set(by_len[:2].tolist() + by_len[-2:].tolist() + by_blk[-3:].tolist() + [0, 31, 63]))
    scales = {k: v.cpu() for k, v in case["scales"].items()}
    worst_abs, worst_l2 = 0.0, 0.0
    for b in rows:
        nb = (int(ctx[b]) + 255) // 256
        ids = bt[b, :nb].long().to(case["k_cache"].device)
        kc, vc = case["k_cache"][ids].cpu(), case["v_cache"][ids].cpu()
        local = torch.arange(nb, dtype=torch.int32).view(1, -1)
        want = O.paged_decode_attention(case["q"][b:b + 1].cpu(), kc, vc, ctx[b:b + 1].to(torch.int32), local,
                                        case["scale"], **scales)
        d = (out[b:b + 1].float() - want.float())
        worst_abs = max(worst_abs, d.abs().max().item())
        worst_l2 = max(worst_l2, (d.norm() / want.float().norm()).item())
    print(f"config 2 (fp8={fp8}, Hq={hq}): {len(rows)} rows, max abs {worst_abs:.2e}, rel L2 {worst_l2:.2e}")
    assert worst_abs <= 2e-2 and worst_l2 <= 1e-3


# ----------------------------------------------------------------------------- config 4: the 8B engine
def bench_sequences(n, max_tokens):
    from bench import e2e_workload
    prompts, _ = e2e_workload(256)
    return prompts[:n], max_tokens


def close(llm):
    """Tear an engine down and hand its memory back before the next one is built."""
    import gc
    llm.exit()
    gc.collect()
    torch.cuda.empty_cache()


def forget_prefix_cache(llm):
    """Drop every prefix-cache entry (no request is live): the next run prefills every token again."""
    bm = llm.scheduler.block_manager
    assert not bm.used_block_ids
    bm.hash_to_block_id.clear()
    for blk in bm.blocks:
        blk.hash, blk.token_ids = -1, []


@pytest.mark.parametrize("quantization", ["w8a16", None])
def test_8b_engine_graph_equals_eager_and_fused_equals_unfused(quantization):
    from tinyllmforge_amd import LLM, SamplingParams
    nblk = 4400                                   # 4400 x 512 KiB = 2.15 GiB per layer and cache side
    llm = LLM("qwen3-8b", enforce_eager=False, max_model_len=4096, quantization=quantization,
              num_kvcache_blocks=nblk, seed=0)
    try:
        runner, bm = llm.model_runner, llm.scheduler.block_manager
        hf = llm.config.hf_config
        assert (hf.num_hidden_layers, hf.hidden_size, hf.num_attention_heads, hf.intermediate_size) == (36, 4096, 32, 12288)
        assert runner.kv_cache.shape == (2, 36, nblk, 256, 8, 128)
        assert runner.graph_bs[-1] == 512 and 48 in runner.graph_bs
        bm.free_block_ids.rotate(-(nblk - 300))    # hand out the pool's last 300 blocks first: offsets > 2^31 bytes
        prompts, max_tokens = bench_sequences(48, 16)
        sp = SamplingParams(temperature=0.0, ignore_eos=True, max_tokens=max_tokens)
        a = [o["token_ids"] for o in llm.generate(prompts, sp)]
        st = dict(llm.last_stats)
        total = sum(len(p) for p in prompts)
        assert st["prefill_steps"] == -(-total // 16384) or st["prefill_steps"] == -(-total // 16384) + 1
        assert st["decode_steps"] == max_tokens - 1 and st["cached_prompt_tokens"] == 0
        assert st["prefill_tokens"] == total + 48      # counted after the sampled token is appended
        assert all(len(x) == max_tokens for x in a)
        assert not bm.used_block_ids and len(bm.free_block_ids) == nblk
        vocab = hf.vocab_size
        assert all(0 <= t < vocab for x in a for t in x)
        assert len({tuple(x) for x in a}) > 1              # different prompts, different continuations

        forget_prefix_cache(llm)
        runner.enforce_eager = True
        try:
            b = [o["token_ids"] for o in llm.generate(prompts, sp)]
        finally:
            runner.enforce_eager = False
        assert llm.last_stats["cached_prompt_tokens"] == 0
        assert a == b, "graph decode and eager decode differ"

        forget_prefix_cache(llm)
        runner.enforce_eager = True
        runner.model.model.fused = False               # the reference's op order: projection, then add-norm
        for layer in runner.model.model.layers:
            layer.self_attn.fused = False              # q/k-norm, RoPE and KV store as separate kernels
        try:
            # same 48 prompts: the same batches, so every GEMM runs the same plan (summation order) in both paths
            c = [o["token_ids"] for o in llm.generate(prompts, SamplingParams(temperature=0.0, ignore_eos=True, max_tokens=6))]
        finally:
            runner.enforce_eager = False
            runner.model.model.fused = True
            for layer in runner.model.model.layers:
                layer.self_attn.fused = True
        assert c == [x[:6] for x in a], "fused and unfused layer paths differ"
        assert not bm.used_block_ids and len(bm.free_block_ids) == nblk
    finally:
        close(llm)


# ----------------------------------------------------------------------------- config 5: the 32B engine
def test_32b_engine_64_layers_cached_prefix_graph_equals_eager_and_fused_equals_unfused():
    """configs[4] at its own depth and width: 64 layers, hidden 5120, 64 query / 8 KV heads, intermediate 25600,
    W8A16 linears, e4m3 KV cache with a different scale per KV head.  Four prompts of 2048 ... 8192 tokens, two of
    them behind a 1024-token prefix that a first request left in cached blocks, 8 greedy tokens each: the prefill
    steps run the paged kernel over e4m3 rows (a prefix hit sends every sequence of the step there), the decode
    steps replay the hipGraph.  The same requests decoded eagerly, and again through the unfused layer path
    (projection, then norm / RoPE / store as separate kernels), must give the same tokens."""
    from tinyllmforge_amd import LLM, SamplingParams
    nblk = 160
    hkv = 8
    k_scale = [(1.0 + 0.1 * h) / 16 for h in range(hkv)]
    v_scale = [(1.4 - 0.05 * h) / 16 for h in range(hkv)]
    llm = LLM("qwen3-32b", enforce_eager=False, max_model_len=8704, max_num_batched_tokens=16384, max_num_seqs=8,
              quantization="w8a16", kv_cache_dtype="fp8_e4m3", kv_k_scale=k_scale, kv_v_scale=v_scale,
              num_kvcache_blocks=nblk, seed=0)
    try:
        runner, bm = llm.model_runner, llm.scheduler.block_manager
        hf = llm.config.hf_config
        assert (hf.num_hidden_layers, hf.hidden_size, hf.num_attention_heads, hf.num_key_value_heads,
                hf.intermediate_size) == (64, 5120, 64, 8, 25600)
        assert runner.kv_cache.shape == (2, 64, nblk, 256, 8, 128) and runner.kv_cache.dtype == torch.float8_e4m3fn
        assert len(runner.model.model.layers) == 64
        shared = random_prompts((1024,), seed=31, vocab=10000)[0]
        bodies = random_prompts((3000 - 1024, 2048, 8192 - 1024, 5000), seed=32, vocab=10000)
        prompts = [shared + bodies[0], bodies[1], shared + bodies[2], bodies[3]]
        assert [len(p) for p in prompts] == [3000, 2048, 8192, 5000]
        sp = SamplingParams(temperature=0.0, ignore_eos=True, max_tokens=8)
        one = SamplingParams(temperature=0.0, ignore_eos=True, max_tokens=1)

        def run(n_tokens=8):
            forget_prefix_cache(llm)
            llm.generate([shared + [1, 2, 3]], one)            # leaves the prefix in four hashed blocks
            out = llm.generate(prompts, SamplingParams(temperature=0.0, ignore_eos=True, max_tokens=n_tokens))
            st = dict(llm.last_stats)
            assert st["cached_prompt_tokens"] == 2048, st      # 1024 tokens for each of the two sequences behind the prefix
            assert not bm.used_block_ids and len(bm.free_block_ids) == nblk
            return [o["token_ids"] for o in out], st

        a, st = run()
        # 18,240 prompt tokens of which 2,048 are cached: the budget (16,384) is charged the uncached ones (scheduler.py:33)
        assert st["decode_steps"] == 7 and st["prefill_steps"] == 1 and st["prefill_tokens"] == 18240 + 4
        assert all(len(x) == 8 for x in a) and all(0 <= t < hf.vocab_size for x in a for t in x)
        assert len({tuple(x) for x in a}) == 4
        runner.enforce_eager = True
        try:
            b, _ = run()
        finally:
            runner.enforce_eager = False
        assert a == b, "graph decode and eager decode differ"
        runner.enforce_eager = True
        runner.model.model.fused = False
        for layer in runner.model.model.layers:
            layer.self_attn.fused = False
        try:
            c, _ = run(4)
        finally:
            runner.enforce_eager = False
            runner.model.model.fused = True
            for layer in runner.model.model.layers:
                layer.self_attn.fused = True
        assert c == [x[:4] for x in a], "fused and unfused layer paths differ"
    finally:
        close(llm)


# ----------------------------------------------------------------------------- widths against the oracle
# Two bf16 pipelines that differ only in fp32 summation order part by accumulated rounding noise: about 16
# bf16 rounding stages over two layers, each worth 2^-9 / sqrt(3) relative, give a relative L2 distance of
# 6e-3 ... 8e-3 between the final hidden states (measured 7.5e-3 at hidden 4096; config 1's 28 layers reach
# 1.5e-2).  A wiring error (wrong head, slot, position, scale or residual) moves it to O(1).
WIDTH_TOL = 1.5e-2


def width_config(name):
    from tinyllmforge_amd.config import QWEN3_SHAPES
    return dict(QWEN3_SHAPES[name], num_hidden_layers=2, max_position_embeddings=4096)


def compare_step(tag, hidden, logits, want_hidden, model, m):
    """Final hidden state and whole logit rows of one step against the oracle's."""
    from oracle import ops as O
    want_rows = model.logits(want_hidden).float()
    h_l2 = ((hidden.float() - want_hidden.float()).norm(dim=-1) / want_hidden.float().norm(dim=-1)).max().item()
    row_l2 = ((logits - want_rows).norm(dim=-1) / want_rows.norm(dim=-1)).max().item()
    ulps = ((logits - want_rows).abs().amax(dim=-1) / O.bf16_ulp(want_rows.abs().amax(dim=-1))).max().item()
    same = (hidden.view(torch.int16) == want_hidden.view(torch.int16)).float().mean().item()
    print(f"{tag}: hidden rel L2 {h_l2:.2e} ({same:.3f} of bits identical), logit rows rel L2 {row_l2:.2e}, "
          f"max |diff| {ulps:.2f} ulp of the row max")
    m["hidden_l2"] = max(m.get("hidden_l2", 0.0), h_l2)
    m["row_l2"] = max(m.get("row_l2", 0.0), row_l2)
    m["ulps"] = max(m.get("ulps", 0.0), ulps)
    return want_rows


def run_width_check(llm, oracle, session, prompts, steps, cached=None):
    """Teacher-forced: the engine's runner and the oracle session see the same sequences, block tables and
    step inputs; after every step both are fed the ORACLE's greedy token."""
    from oracle import ops as O
    from tinyllmforge_amd.engine.sequence import Sequence
    from tinyllmforge_amd.sampling_params import SamplingParams
    from tinyllmforge_amd.utils.context import get_context, reset_context
    runner, sch = llm.model_runner, llm.scheduler
    sp = SamplingParams(temperature=0.0, max_tokens=steps, ignore_eos=True)
    seqs0 = [Sequence(p, sp) for p in prompts]
    for s in seqs0:
        sch.add(s)
    m = {}
    for step in range(steps):
        seqs, is_prefill = sch.schedule()
        assert seqs == seqs0 and is_prefill == (step == 0)
        tables = [list(s.block_table) for s in seqs]
        toks = [list(s.token_ids) for s in seqs]
        if is_prefill:
            ncached = [s.num_cached_tokens for s in seqs]
            if cached is not None:
                assert ncached == cached, (ncached, cached)
            ids, pos = runner.prepare_prefill(seqs)
            assert (get_context().block_tables is not None) == (sum(ncached) > 0)
            want_hidden = session.prefill(toks, tables, ncached)
        else:
            ids, pos = runner.prepare_decode(seqs)
            want_hidden = session.decode(toks, tables)
        hidden = runner.run_hidden(ids, pos, is_prefill)            # graph replay for the decode steps
        logits = runner.model.compute_logits(hidden).float().cpu()
        if is_prefill:
            hidden = hidden[(get_context().cu_seqlens_q[1:] - 1).long()]
        reset_context()
        want_rows = compare_step(f"step {step} ({'prefill' if is_prefill else 'decode'})", hidden.cpu(), logits,
                                 want_hidden, oracle, m)
        # decisions: identical wherever the oracle's top-2 margin exceeds 2 bf16 ulp
        top = want_rows.topk(2, dim=-1)
        margin = (top.values[:, 0] - top.values[:, 1]) / O.bf16_ulp(top.values[:, 0])
        choice = logits.argmax(-1)
        clear = margin > 2
        assert torch.equal(choice[clear], top.indices[clear, 0]), (step, choice, top.indices[:, 0], margin)
        sch.postprocess(seqs, top.indices[:, 0].tolist())
    assert sch.is_finished()
    return m


def cpu_params(llm):
    return {k: v.cpu() for k, v in llm.model_runner.model.checkpoint_parameters().items()}


def random_prompts(lens, seed, vocab=151936):
    g = torch.Generator().manual_seed(seed)
    return [torch.randint(0, vocab, (n,), generator=g).tolist() for n in lens]


def test_8b_width_two_layers_against_the_oracle_bf16_and_w8a16():
    """hidden 4096, 32 / 8 heads, intermediate 12288, vocab 151936, 2 layers; prompts of 33 ... 515 tokens (block
    boundaries 256 and 512 crossed), 1 prefill + 3 graph decode steps.  bf16 linears against the exactly
    rounded oracle, then the same weights quantised (int8 GEMMs, fused gate_up + SiLU-and-mul) against the
    oracle's quantised projections."""
    from oracle.model import OracleQwen3, OracleSession
    from tinyllmforge_amd import LLM
    cfg = width_config("qwen3-8b")
    prompts = random_prompts((100, 260, 515, 33, 256), seed=11)
    llm = LLM(cfg, max_model_len=2048, max_num_batched_tokens=4096, max_num_seqs=8, num_kvcache_blocks=24,
              enforce_eager=False, seed=3)
    params = cpu_params(llm)
    try:
        oracle = OracleQwen3(cfg, params)
        m = run_width_check(llm, oracle, OracleSession(oracle, 24), prompts, 4)
    finally:
        close(llm)
    assert m["hidden_l2"] <= WIDTH_TOL and m["row_l2"] <= WIDTH_TOL and m["ulps"] <= 4.0, m   # measured: 2.0 ... 3.0
    del oracle
    llm = LLM(cfg, max_model_len=2048, max_num_batched_tokens=4096, max_num_seqs=8, num_kvcache_blocks=24,
              enforce_eager=False, seed=3, quantization="w8a16", state_dict=params)
    try:
        oracle = OracleQwen3(cfg, params, w8a16=True)
        m = run_width_check(llm, oracle, OracleSession(oracle, 24), prompts, 4)
    finally:
        close(llm)
    assert m["hidden_l2"] <= WIDTH_TOL and m["row_l2"] <= WIDTH_TOL and m["ulps"] <= 4.0, m   # measured: 2.0 ... 3.0


def test_32b_width_two_layers_fp8_kv_with_cached_prefix_against_the_oracle():
    """hidden 5120, 64 / 8 heads, intermediate 25600, 2 layers, W8A16 linears, e4m3 KV cache whose scale differs
    per KV head and layer, a 1024-token prefix held in cached blocks: a first request fills the prefix blocks,
    then two of three prompts hit them, so the prefill step runs the paged kernel over e4m3 rows for every
    sequence (the fresh tokens are read back quantised) and the decode steps read the same cache."""
    from oracle.model import OracleQwen3, OracleSession
    from tinyllmforge_amd import LLM, SamplingParams
    cfg = width_config("qwen3-32b")
    hkv = cfg["num_key_value_heads"]
    k_scale = [[(1.0 + 0.15 * h + 0.4 * l) / 16 for h in range(hkv)] for l in range(2)]
    v_scale = [[(1.5 - 0.1 * h + 0.3 * l) / 16 for h in range(hkv)] for l in range(2)]
    shared = random_prompts((1024,), seed=21, vocab=10000)[0]
    tails = random_prompts((150, 300, 1200), seed=22, vocab=10000)
    prompts = [shared + tails[0], shared + tails[1], tails[2]]
    llm = LLM(cfg, max_model_len=4096, max_num_batched_tokens=8192, max_num_seqs=8, num_kvcache_blocks=40,
              enforce_eager=False, seed=5, quantization=None)
    params = cpu_params(llm)
    close(llm)
    llm = LLM(cfg, max_model_len=4096, max_num_batched_tokens=8192, max_num_seqs=8, num_kvcache_blocks=40,
              enforce_eager=False, seed=5, quantization="w8a16", state_dict=params, kv_cache_dtype="fp8_e4m3",
              kv_k_scale=k_scale, kv_v_scale=v_scale)
    try:
        attn1 = llm.model_runner.model.model.layers[1].self_attn.attn
        assert torch.allclose(attn1.k_scale.cpu(), torch.tensor(k_scale[1])) and attn1.k_cache.dtype == torch.float8_e4m3fn
        oracle = OracleQwen3(cfg, params, w8a16=True)
        scales = [(torch.tensor(k_scale[l]), torch.tensor(v_scale[l])) for l in range(2)]
        session = OracleSession(oracle, 40, kv_dtype=torch.float8_e4m3fn, kv_scales=scales)
        # the request that leaves the prefix in cached blocks 0 .. 3 (engine and oracle alike)
        first = shared + [1, 2, 3]
        llm.generate([first], SamplingParams(temperature=0.0, max_tokens=1, ignore_eos=True))
        session.prefill([first], [[0, 1, 2, 3, 4]], [0])
        m = run_width_check(llm, oracle, session, prompts, 3, cached=[1024, 1024, 0])
    finally:
        close(llm)
    assert m["hidden_l2"] <= 2 * WIDTH_TOL and m["row_l2"] <= 2 * WIDTH_TOL and m["ulps"] <= 4.0, m   # measured: 2.0 ... 3.0


def test_e4m3_cache_saturation_is_counted_per_layer_and_head():
    """An e4m3 cache clamps at +-448 x scale without an error; `ModelRunner.kv_saturation` counts the clamped
    entries.  Planted codes are found where they were put; a run with an absurdly small K scale saturates K and
    leaves V alone; a bf16 cache reports nothing."""
    from tinyllmforge_amd import LLM, SamplingParams
    cfg = width_config("qwen3-0.6b")
    llm = LLM(cfg, max_model_len=1024, max_num_batched_tokens=2048, max_num_seqs=4, num_kvcache_blocks=6,
              enforce_eager=True, seed=1, kv_cache_dtype="fp8_e4m3", kv_k_scale=1e-4, kv_v_scale=4.0)
    try:
        mr = llm.model_runner
        assert mr.kv_saturation() == dict(entries=mr.kv_cache[0].numel(), k_saturated=0, v_saturated=0,
                                          k_worst=None, v_worst=None)
        with torch.inference_mode():           # the cache was allocated under inference mode
            kv = mr.kv_cache.view(torch.uint8)
            kv[0, 1, 2, 5:9, 3, :] = 0x7e      # K, layer 1, block 2, four rows of KV head 3: +448 x scale
            kv[0, 0, 4, 0, 1, :7] = 0xfe       # K, layer 0: seven entries at -448 x scale
            kv[1, 1, 0, 0, 0, 0] = 0x7d        # V: the largest code below saturation
        got = mr.kv_saturation()
        assert got["k_saturated"] == 4 * 128 + 7 and got["v_saturated"] == 0
        assert got["k_worst"] == dict(layer=1, kv_head=3, saturated=4 * 128) and got["v_worst"] is None
        assert mr.kv_saturation(block_ids=[4])["k_saturated"] == 7
        with torch.inference_mode():
            mr.kv_cache.zero_()
        llm.generate(random_prompts((300,), seed=3, vocab=10000), SamplingParams(temperature=0.0, max_tokens=4, ignore_eos=True))
        got = mr.kv_saturation()
        # k after q/k-norm is of order 1: with a scale of 1e-4 almost every written K entry clamps; |v| << 448 x 4
        assert got["k_saturated"] > 0.9 * 2 * 303 * cfg["num_key_value_heads"] * 128 and got["v_saturated"] == 0, got
    finally:
        close(llm)
    llm = LLM(cfg, max_model_len=1024, max_num_batched_tokens=2048, max_num_seqs=4, num_kvcache_blocks=6,
              enforce_eager=True, seed=1)
    try:
        assert llm.model_runner.kv_saturation()["entries"] == 0
    finally:
        close(llm)
