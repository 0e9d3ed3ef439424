"""CPU restatement of one Qwen3 decoder forward and of a greedy generate loop
(test infrastructure: see ``oracle/__init__.py``).

Follows the reference's op order (tinyvllm/models/qwen3.py:74-96, 123-130, 158-172, 185-195,
229-234; layers/embed_head.py:58-63; layers/sampler.py:13-14) and its step inputs
(engine/model_runner.py:164-228), including ``positions = len(seq)`` for decode steps
(model_runner.py:219).

Every linear is the exactly rounded one (``ops.linear_exact``: fp64 accumulation, one rounding
to bf16) so that the token ids do not depend on the accumulation order of the host's BLAS;
the reference's ``F.linear`` is the same contraction with an unspecified fp32 order.
"""
from __future__ import annotations

import torch

from . import ops as O


class OracleQwen3:
    def __init__(self, cfg: dict, params: dict, exact: bool = True, w8a16: bool = False):
        """``params``: ``{name: tensor}`` with the reference's packed parameter names
        (``model.layers.N.self_attn.qkv_proj.weight`` ...).  ``exact=False`` runs the linears as the
        reference does on a CPU (``F.linear`` in bf16, no fp64 copies): used for timing only.
        ``w8a16=True`` (build-defined, not in the reference): the four projections of every layer are
        quantised with ``ops.quantize_w8`` and run through ``ops.w8a16_linear``; embedding and LM head
        stay bf16."""
        self.cfg = dict(cfg)
        self.exact = exact
        self.p = {k: v.detach().cpu() for k, v in params.items()}
        self.q8 = {}
        if w8a16:
            for k in list(self.p):
                if k.endswith("proj.weight"):
                    self.q8[k] = O.quantize_w8(self.p[k])
        self.q8d = {k: wq.double() for k, (wq, _) in self.q8.items()}    # fp64 copies, made once
        self.p64 = {}
        if exact:
            tied = "lm_head.weight" not in self.p
            self.p64 = {k: v.double() for k, v in self.p.items()
                        if (k.endswith("proj.weight") and k not in self.q8) or k.startswith("lm_head")
                        or (tied and "embed_tokens" in k)}
        c = self.cfg
        self.Hq, self.Hkv, self.Dh = c["num_attention_heads"], c["num_key_value_heads"], c["head_dim"]
        self.eps = c.get("rms_norm_eps", 1e-6)
        self.table = O.rope_table(self.Dh, c.get("max_position_embeddings", 40960), c.get("rope_theta", 1e6))
        self.L = c["num_hidden_layers"]
        if "lm_head.weight" not in self.p:
            self.p["lm_head.weight"] = self.p["model.embed_tokens.weight"]
        if exact and "lm_head.weight" not in self.p64:
            self.p64["lm_head.weight"] = self.p64["model.embed_tokens.weight"]

    def lin(self, x, name):
        if name in self.q8:        # ops.w8a16_linear with the weight's fp64 copy kept between calls
            return ((x.double() @ self.q8d[name].t()).float() * self.q8[name][1].float()[None, :]).to(x.dtype)
        if not self.exact:
            return O.linear(x, self.p[name])
        return (x.double() @ self.p64[name].t()).to(x.dtype)

    def forward(self, input_ids, positions, caches, slot_mapping, attend, kv_scales=None):
        """``caches[l] = (k_cache, v_cache)``; ``attend(q, k, v, k_cache, v_cache, k_scale, v_scale)`` does the
        step's attention.  ``kv_scales[l] = (k_scale, v_scale)`` (fp32 ``[Hkv]``) for e4m3 caches (build-defined,
        ``ops.store_kvcache_fp8``); None for caches in the model dtype."""
        p = self.p
        x = O.embedding(input_ids, p["model.embed_tokens.weight"])
        residual = None
        q_size, kv_size = self.Hq * self.Dh, self.Hkv * self.Dh
        for l in range(self.L):
            pre = f"model.layers.{l}."
            if residual is None:
                residual = x
                x = O.rms_norm(x, p[pre + "input_layernorm.weight"], self.eps)
            else:
                x, residual = O.add_rms_norm(x, residual, p[pre + "input_layernorm.weight"], self.eps)
            qkv = self.lin(x, pre + "self_attn.qkv_proj.weight")
            q, k, v = qkv.split([q_size, kv_size, kv_size], dim=-1)
            n = q.shape[0]
            q = O.rms_norm(q.reshape(n, self.Hq, self.Dh), p[pre + "self_attn.q_norm.weight"], self.eps).reshape(n, -1)
            k = O.rms_norm(k.reshape(n, self.Hkv, self.Dh), p[pre + "self_attn.k_norm.weight"], self.eps).reshape(n, -1)
            q, k = O.rope(positions, q, k, self.table, self.Dh)
            kc, vc = caches[l]
            ks, vs = kv_scales[l] if kv_scales is not None else (None, None)
            k3, v3 = k.view(n, self.Hkv, self.Dh), v.reshape(n, self.Hkv, self.Dh)
            if ks is None:
                O.store_kvcache(k3, v3, kc, vc, slot_mapping)
            else:
                O.store_kvcache_fp8(k3, v3, kc, vc, slot_mapping, ks, vs)
            o = attend(q.view(n, self.Hq, self.Dh), k3, v3, kc, vc, ks, vs)
            x = self.lin(o, pre + "self_attn.o_proj.weight")
            x, residual = O.add_rms_norm(x, residual, p[pre + "post_attention_layernorm.weight"], self.eps)
            x = self.lin(x, pre + "mlp.gate_up_proj.weight")
            x = O.silu_and_mul(x)
            x = self.lin(x, pre + "mlp.down_proj.weight")
        x, _ = O.add_rms_norm(x, residual, p["model.norm.weight"], self.eps)
        return x

    def logits(self, hidden):
        return self.lin(hidden, "lm_head.weight")


def greedy_generate(model: OracleQwen3, prompts: list[list[int]], max_tokens: int, block_size: int = 256,
                    position_quirk: bool = True, trace: list | None = None):
    """All prompts prefilled in one step, then ``max_tokens - 1`` decode steps of the whole batch.

    Returns ``(token_ids, margins, topk)``: the generated ids per sequence; per step and sequence the
    gap between the two largest logits (fp32 of the bf16 logits), to judge near-ties; and per step
    and sequence the four largest logits as ``(ids, values)``.  ``trace`` (a list) receives the final hidden
    states ``[B, hidden]`` that each step's logits were computed from.
    """
    B = len(prompts)
    Hkv, Dh = model.Hkv, model.Dh
    max_len = max(len(p) for p in prompts) + max_tokens + 1
    nblk_seq = -(-max_len // block_size)
    caches = [(torch.zeros(B * nblk_seq, block_size, Hkv, Dh, dtype=torch.bfloat16),
               torch.zeros(B * nblk_seq, block_size, Hkv, Dh, dtype=torch.bfloat16)) for _ in range(model.L)]
    bt = torch.arange(B * nblk_seq, dtype=torch.int32).view(B, nblk_seq)     # sequence b owns blocks b*n .. b*n+n-1
    scale = O.softmax_scale(Dh)
    seqs = [list(p) for p in prompts]
    out = [[] for _ in range(B)]
    margins, topk = [], []

    def slot(b, t):
        return int(bt[b, t // block_size]) * block_size + t % block_size

    def sample(hidden_rows):
        if trace is not None:
            trace.append(hidden_rows.clone())
        lg = model.logits(hidden_rows)
        top = lg.float().topk(4, dim=-1)
        margins.append((top.values[:, 0] - top.values[:, 1]).tolist())
        topk.append((top.indices.tolist(), top.values.tolist()))
        return O.greedy_sample(lg).tolist()

    # prefill
    lens = [len(s) for s in seqs]
    ids = torch.tensor([t for s in seqs for t in s], dtype=torch.int64)
    pos = torch.tensor([t for s in seqs for t in range(len(s))], dtype=torch.int64)
    slots = torch.tensor([slot(b, t) for b, s in enumerate(seqs) for t in range(len(s))], dtype=torch.int32)
    cu = torch.tensor([0] + list(torch.tensor(lens).cumsum(0)), dtype=torch.int32)
    h = model.forward(ids, pos, caches, slots,
                      lambda q, k, v, kc, vc, ks, vs: O.varlen_prefill_attention(q, k, v, cu, cu, scale))
    toks = sample(h[(cu[1:] - 1).long()])
    for b in range(B):
        seqs[b].append(toks[b]); out[b].append(toks[b])
    # decode
    for _ in range(max_tokens - 1):
        n = [len(s) for s in seqs]
        ids = torch.tensor([s[-1] for s in seqs], dtype=torch.int64)
        pos = torch.tensor([(x if position_quirk else x - 1) for x in n], dtype=torch.int64)
        slots = torch.tensor([slot(b, n[b] - 1) for b in range(B)], dtype=torch.int32)
        cl = torch.tensor(n, dtype=torch.int32)
        h = model.forward(ids, pos, caches, slots,
                          lambda q, k, v, kc, vc, ks, vs: O.paged_decode_attention(q, kc, vc, cl, bt, scale))
        toks = sample(h)
        for b in range(B):
            seqs[b].append(toks[b]); out[b].append(toks[b])
    return out, margins, topk


class OracleSession:
    """Step-by-step driver with the engine's step inputs (tinyvllm/engine/model_runner.py:164-228): a prefill
    step over the uncached tail of every prompt - reading K/V of EVERY sequence from the paged cache as soon as
    one of them has a cached prefix (layers/attention.py:99-100) - and decode steps of the whole batch.
    The caller owns the block tables, so cached prefixes are expressed by sharing block ids between
    sequences.  Optional e4m3 caches with per-layer ``(k_scale, v_scale)`` (build-defined)."""

    def __init__(self, model: OracleQwen3, num_blocks: int, block_size: int = 256, kv_dtype=torch.bfloat16,
                 kv_scales=None, position_quirk: bool = True):
        self.m, self.bs, self.quirk = model, block_size, position_quirk
        self.kv_scales = kv_scales
        self.caches = [(torch.zeros(num_blocks, block_size, model.Hkv, model.Dh, dtype=kv_dtype),
                        torch.zeros(num_blocks, block_size, model.Hkv, model.Dh, dtype=kv_dtype))
                       for _ in range(model.L)]
        self.scale = O.softmax_scale(model.Dh)

    def _slots(self, table, ts):
        return [int(table[t // self.bs]) * self.bs + t % self.bs for t in ts]

    def prefill(self, seqs, tables, num_cached):
        """``seqs[b]``: token ids; ``tables[b]``: block ids; ``num_cached[b]``: leading tokens already in the cache
        (a multiple of the block size).  Returns the final hidden state of each sequence's last token."""
        ids, pos, slots, cu_q, cu_k = [], [], [], [0], [0]
        for s, tb, c in zip(seqs, tables, num_cached):
            n = len(s)
            ids += s[c:n]
            pos += list(range(c, n))
            slots += self._slots(tb, range(c, n))
            cu_q.append(cu_q[-1] + n - c)
            cu_k.append(cu_k[-1] + n)
        cu_q, cu_k = torch.tensor(cu_q, dtype=torch.int32), torch.tensor(cu_k, dtype=torch.int32)
        paged = int(cu_k[-1]) > int(cu_q[-1])
        width = max(len(t) for t in tables)
        bt = torch.tensor([list(t) + [-1] * (width - len(t)) for t in tables], dtype=torch.int32)

        def attend(q, k, v, kc, vc, ks, vs):
            if paged:
                return O.varlen_prefill_attention(q, kc, vc, cu_q, cu_k, self.scale, block_tables=bt,
                                                  k_scale=ks, v_scale=vs)
            return O.varlen_prefill_attention(q, k, v, cu_q, cu_k, self.scale)

        h = self.m.forward(torch.tensor(ids, dtype=torch.int64), torch.tensor(pos, dtype=torch.int64), self.caches,
                           torch.tensor(slots, dtype=torch.int32), attend, self.kv_scales)
        return h[(cu_q[1:] - 1).long()]

    def decode(self, seqs, tables):
        """One decode step: the last token of every sequence is fed (its K/V stored at index ``len - 1``),
        position ``len`` with the reference's quirk (model_runner.py:219).  Returns the hidden states."""
        n = [len(s) for s in seqs]
        width = max(len(t) for t in tables)
        bt = torch.tensor([list(t) + [-1] * (width - len(t)) for t in tables], dtype=torch.int32)
        cl = torch.tensor(n, dtype=torch.int32)
        slots = torch.tensor([self._slots(tb, [x - 1])[0] for tb, x in zip(tables, n)], dtype=torch.int32)
        pos = torch.tensor([(x if self.quirk else x - 1) for x in n], dtype=torch.int64)
        return self.m.forward(torch.tensor([s[-1] for s in seqs], dtype=torch.int64), pos, self.caches, slots,
                              lambda q, k, v, kc, vc, ks, vs: O.paged_decode_attention(q, kc, vc, cl, bt, self.scale,
                                                                                       ks, vs),
                              self.kv_scales)
