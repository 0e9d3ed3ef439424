"""Writes tests/golden/c1_greedy.json: greedy token ids of the CPU oracle on BASELINE config 1.

    python tests/golden/make_c1_golden.py            # bf16 linears, 32 tokens -> c1_greedy.json
    python tests/golden/make_c1_golden.py --w8a16    # int8 projections, 8 tokens -> c1_w8a16_greedy.json
Beside each .json: *_hidden_bf16_bits.npy, the final hidden states (bf16 bits) behind every step's logits.

Config 1: Qwen3-0.6B-shaped decoder (28 layers, hidden 1024, 16 query / 8 KV heads, head_dim 128,
intermediate 3072, vocab 151936, RMSNorm eps 1e-6 + q/k-norm, RoPE theta 1e6, tied embeddings),
random-init bf16 weights N(0, 0.02) drawn on the CPU from torch.Generator().manual_seed(0) in
named_parameters() order, norm weights 1; 4 prompts of 128 token ids from
torch.randint(0, 151936, (4, 128), generator=manual_seed(0)); 32 greedy tokens each; KV block 256.

The reference cannot run here (it imports flash_attn and needs CUDA), so the expected ids come
from oracle/model.py, whose ops are pinned in tests/test_oracle_ops.py.  Takes about a minute.
"""
import json
import os
import sys
import time

import torch

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)

from oracle.model import OracleQwen3, greedy_generate  # noqa: E402


def c1_config():
    from tinyllmforge_amd.config import QWEN3_SHAPES, ModelConfig
    return ModelConfig.from_any(dict(QWEN3_SHAPES["qwen3-0.6b"], max_position_embeddings=4096))


def c1_params(cfg):
    """The weights are an INPUT shared by both sides: built once with the package's seeded initialiser."""
    from tinyllmforge_amd.models.qwen3 import Qwen3ForCausalLM
    from tinyllmforge_amd.utils.loader import random_init_
    torch.set_default_dtype(torch.bfloat16)
    try:
        model = Qwen3ForCausalLM(cfg)
        random_init_(model, seed=0)
    finally:
        torch.set_default_dtype(torch.float32)
    return {k: v.data for k, v in model.named_parameters()}


def c1_prompts():
    g = torch.Generator().manual_seed(0)
    return torch.randint(0, 151936, (4, 128), generator=g).tolist()


def main():
    w8 = "--w8a16" in sys.argv
    cfg = c1_config()
    t0 = time.time()
    params = c1_params(cfg)
    oracle = OracleQwen3(vars(cfg), params, w8a16=w8)
    prompts = c1_prompts()
    hidden = []
    ids, margins, topk = greedy_generate(oracle, prompts, max_tokens=8 if w8 else 32, block_size=256, trace=hidden)
    out = dict(config="BASELINE.json configs[0]" + (" with int8 per-channel projection weights" if w8 else ""),
               seed=0, prompt_first_tokens=[p[:4] for p in prompts],
               token_ids=ids, top2_margin=[[round(m, 6) for m in row] for row in margins],
               top4_ids=[t[0] for t in topk], top4_logits=[t[1] for t in topk],
               bf16_ulp_note="margins are differences of bf16 logits; 0.0 is an exact tie (first index wins)")
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "c1_w8a16_greedy.json" if w8 else "c1_greedy.json")
    with open(path, "w") as f:
        json.dump(out, f)
    # the final hidden states behind every step's logits, bf16 bit patterns [steps, 4, hidden]: with the LM head
    # weight (an input both sides share) they determine the oracle's whole logit rows
    import numpy as np
    bits = torch.stack(hidden).view(torch.int16).numpy()
    np.save(path.replace("_greedy.json", "_hidden_bf16_bits.npy"), bits)
    print("wrote", path, "in %.1f s" % (time.time() - t0))
    print("min margin", min(min(r) for r in margins))


if __name__ == "__main__":
    main()
