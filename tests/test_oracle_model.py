"""Pins for the oracle's model-level restatement (CPU).

* incremental decode over the paged cache equals a fresh prefill of the longer prompt
  (a dropped cache row, a wrong slot or a wrong causal offset breaks this);
* the decode-position quirk of the reference really shifts RoPE by one (results change);
* the committed config-1 fixture is what the oracle produces (first steps recomputed here).
"""
import json
import os

import pytest
import torch

from oracle import ops as O
from oracle.model import OracleQwen3, OracleSession, greedy_generate

TINY = dict(hidden_size=256, num_hidden_layers=2, num_attention_heads=2, num_key_value_heads=1, head_dim=128,
            intermediate_size=512, vocab_size=512, max_position_embeddings=1024, rope_theta=1e6, rms_norm_eps=1e-6)


def tiny_params(seed=0):
    g = torch.Generator().manual_seed(seed)
    c = TINY
    H, I, V = c["hidden_size"], c["intermediate_size"], c["vocab_size"]
    qkv = (c["num_attention_heads"] + 2 * c["num_key_value_heads"]) * c["head_dim"]
    n = lambda *s: (torch.randn(*s, generator=g) * 0.05).to(torch.bfloat16)
    p = {"model.embed_tokens.weight": n(V, H), "model.norm.weight": torch.ones(H, dtype=torch.bfloat16)}
    for l in range(c["num_hidden_layers"]):
        pre = f"model.layers.{l}."
        p[pre + "self_attn.qkv_proj.weight"] = n(qkv, H)
        p[pre + "self_attn.o_proj.weight"] = n(H, c["num_attention_heads"] * c["head_dim"])
        p[pre + "self_attn.q_norm.weight"] = torch.ones(128, dtype=torch.bfloat16)
        p[pre + "self_attn.k_norm.weight"] = torch.ones(128, dtype=torch.bfloat16)
        p[pre + "mlp.gate_up_proj.weight"] = n(2 * I, H)
        p[pre + "mlp.down_proj.weight"] = n(H, I)
        p[pre + "input_layernorm.weight"] = torch.ones(H, dtype=torch.bfloat16)
        p[pre + "post_attention_layernorm.weight"] = torch.ones(H, dtype=torch.bfloat16)
    return p


def test_incremental_decode_equals_fresh_prefill():
    model = OracleQwen3(TINY, tiny_params())
    g = torch.Generator().manual_seed(1)
    prompts = [torch.randint(0, 512, (n,), generator=g).tolist() for n in (5, 17)]
    ids, margins, _ = greedy_generate(model, prompts, max_tokens=6, block_size=8, position_quirk=False)
    for b, p in enumerate(prompts):
        for t in range(6):
            if margins[t][b] < 0.05:          # skip decisions too close to call between two code paths
                continue
            ctx = p + ids[b][:t]
            one, _, _ = greedy_generate(model, [ctx], max_tokens=1, block_size=8, position_quirk=False)
            assert one[0][0] == ids[b][t], (b, t)


def test_decode_position_quirk_changes_the_rotation():
    model = OracleQwen3(TINY, tiny_params())
    prompts = [[3, 9, 27, 81, 243]]
    n = 5
    cache = lambda: [(torch.zeros(2, 8, 1, 128, dtype=torch.bfloat16), torch.zeros(2, 8, 1, 128, dtype=torch.bfloat16)) for _ in range(2)]
    bt = torch.tensor([[0, 1]], dtype=torch.int32)
    outs = []
    for pos in (n, n - 1):
        c = cache()
        cu = torch.tensor([0, n], dtype=torch.int32)
        model.forward(torch.tensor(prompts[0]), torch.arange(n), c, torch.arange(n, dtype=torch.int32),
                      lambda q, k, v, kc, vc, ks, vs: O.varlen_prefill_attention(q, k, v, cu, cu, 128 ** -0.5))
        h = model.forward(torch.tensor([7]), torch.tensor([pos]), c, torch.tensor([n], dtype=torch.int32),
                          lambda q, k, v, kc, vc, ks, vs: O.paged_decode_attention(q, kc, vc, torch.tensor([n + 1], dtype=torch.int32), bt, 128 ** -0.5))
        outs.append(h)
        # the new K row went to slot n
        assert c[0][0].view(-1, 128)[n].abs().sum() > 0 and c[0][0].view(-1, 128)[n + 1].abs().sum() == 0
    assert not torch.equal(outs[0], outs[1])


@pytest.mark.parametrize("fixture,w8a16,steps", [("c1_greedy.json", False, 3), ("c1_w8a16_greedy.json", True, 2)])
def test_c1_fixture_first_steps_reproduce(fixture, w8a16, steps):
    """Recompute prefill + the first decode steps of config 1 with the oracle (about 20 s per fixture) and
    compare with the committed fixture: bf16 projections, and the weight-only int8 model."""
    import sys
    sys.path.insert(0, os.path.join(os.path.dirname(__file__), "golden"))
    import make_c1_golden as M
    with open(os.path.join(os.path.dirname(__file__), "golden", fixture)) as f:
        gold = json.load(f)
    cfg = M.c1_config()
    oracle = OracleQwen3(vars(cfg), M.c1_params(cfg), w8a16=w8a16)
    ids, margins, topk = greedy_generate(oracle, M.c1_prompts(), max_tokens=steps, block_size=256)
    assert [r[:steps] for r in gold["token_ids"]] == ids
    for t in range(steps):
        assert gold["top4_ids"][t] == topk[t][0]
        assert gold["top4_logits"][t] == topk[t][1]


def test_w8a16_oracle_routes_the_projections_through_the_int8_linear():
    """``w8a16=True``: every projection equals ``ops.w8a16_linear`` on ``ops.quantize_w8`` of its weight
    (and differs from the bf16 product), embedding and LM head stay bf16; the quantised model is close
    to the bf16 one (int8 per-channel error), not identical."""
    params = tiny_params()
    m8, m16 = OracleQwen3(TINY, params, w8a16=True), OracleQwen3(TINY, params)
    name = "model.layers.1.mlp.down_proj.weight"
    x = (torch.randn(5, params[name].shape[1], generator=torch.Generator().manual_seed(3))).to(torch.bfloat16)
    wq, sc = O.quantize_w8(params[name])
    assert torch.equal(m8.lin(x, name), O.w8a16_linear(x, wq, sc))
    assert not torch.equal(m8.lin(x, name), m16.lin(x, name))
    assert torch.equal(m8.lin(x[:, :TINY["hidden_size"]], "lm_head.weight"), m16.lin(x[:, :TINY["hidden_size"]], "lm_head.weight"))
    assert set(m8.q8) == {k for k in params if k.endswith("proj.weight")}
    prompts = [[3, 9, 27, 81, 243, 5, 6]]
    _, _, t8 = greedy_generate(m8, prompts, max_tokens=1, block_size=8)
    _, _, t16 = greedy_generate(m16, prompts, max_tokens=1, block_size=8)
    a, b = torch.tensor(t8[0][1][0]), torch.tensor(t16[0][1][0])
    assert (a - b).abs().max() < 0.25 * b.abs().max() and not torch.equal(a, b)


def test_session_steps_equal_the_generate_loop_and_a_cached_prefix_changes_nothing():
    """``OracleSession`` against ``greedy_generate`` (same hidden states -> same ids), and the paged prefill with
    a cached prefix against a dense prefill of the same prompts: with bf16 caches the prefix rows read back
    from the cache are the bits the dense path computes, so the last-token hidden states must be equal."""
    model = OracleQwen3(TINY, tiny_params())
    g = torch.Generator().manual_seed(5)
    shared = torch.randint(0, 512, (16,), generator=g).tolist()          # two full blocks of 8
    prompts = [shared + torch.randint(0, 512, (n,), generator=g).tolist() for n in (5, 11)]
    ids, _, _ = greedy_generate(model, prompts, max_tokens=3, block_size=8)
    # dense: each sequence owns its blocks
    ses = OracleSession(model, num_blocks=16, block_size=8)
    tables = [[0, 1, 2, 3], [4, 5, 6, 7]]
    h0 = ses.prefill(prompts, tables, [0, 0])
    seqs = [list(p) for p in prompts]
    got = [[] for _ in prompts]
    h = h0
    for step in range(3):
        toks = O.greedy_sample(model.logits(h)).tolist()
        for b, t in enumerate(toks):
            seqs[b].append(t); got[b].append(t)
        if step < 2:
            h = ses.decode(seqs, tables)
    assert got == ids
    # paged: a first request fills the shared blocks 0, 1; the batch then shares them
    ses2 = OracleSession(model, num_blocks=16, block_size=8)
    ses2.prefill([shared + [1]], [[0, 1, 2]], [0])
    h1 = ses2.prefill(prompts, [[0, 1, 3, 4], [0, 1, 5, 6]], [16, 16])
    assert torch.equal(h0, h1)
    # fp8 caches (build-defined): same driver, e4m3 rows with per-head scales; close to bf16, not equal
    scales = [(torch.tensor([0.05]), torch.tensor([0.03]))] * TINY["num_hidden_layers"]
    ses3 = OracleSession(model, num_blocks=16, block_size=8, kv_dtype=torch.float8_e4m3fn, kv_scales=scales)
    ses3.prefill([shared + [1]], [[0, 1, 2]], [0])
    h2 = ses3.prefill(prompts, [[0, 1, 3, 4], [0, 1, 5, 6]], [16, 16])
    rel = (h2.float() - h0.float()).norm() / h0.float().norm()
    assert 0 < rel < 0.1
    assert ses3.caches[0][0].dtype == torch.float8_e4m3fn and ses3.caches[0][0].view(-1, 128)[0].float().abs().sum() > 0
