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
from oracle.model import OracleQwen3, greedy_generate

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
                      lambda q, k, v, kc, vc: O.varlen_prefill_attention(q, k, v, cu, cu, 128 ** -0.5))
        h = model.forward(torch.tensor([7]), torch.tensor([pos]), c, torch.tensor([n], dtype=torch.int32),
                          lambda q, k, v, kc, vc: O.paged_decode_attention(q, kc, vc, torch.tensor([n + 1], dtype=torch.int32), bt, 128 ** -0.5))
        outs.append(h)
        # the new K row went to slot n
        assert c[0][0].view(-1, 128)[n].abs().sum() > 0 and c[0][0].view(-1, 128)[n + 1].abs().sum() == 0
    assert not torch.equal(outs[0], outs[1])


@pytest.mark.skipif(not os.path.exists(os.path.join(os.path.dirname(__file__), "golden", "c1_greedy.json")), reason="no fixture")
def test_c1_fixture_first_steps_reproduce():
    """Recompute prefill + 2 decode steps of config 1 with the oracle (about 20 s) and compare with the fixture."""
    import sys
    sys.path.insert(0, os.path.join(os.path.dirname(__file__), "golden"))
    import make_c1_golden as M
    with open(os.path.join(os.path.dirname(__file__), "golden", "c1_greedy.json")) as f:
        gold = json.load(f)
    cfg = M.c1_config()
    oracle = OracleQwen3(vars(cfg), M.c1_params(cfg))
    ids, margins, topk = greedy_generate(oracle, M.c1_prompts(), max_tokens=3, block_size=256)
    assert [r[:3] for r in gold["token_ids"]] == ids
    for t in range(3):
        assert gold["top4_ids"][t] == topk[t][0]
        assert gold["top4_logits"][t] == topk[t][1]
