"""Per-op CPU oracle (test infrastructure: see ``oracle/__init__.py``).

All functions take and return CPU torch tensors.  "bf16(x)" below means one
round-to-nearest-even conversion to bfloat16; the reference's rounding points
are kept exactly where its eager text puts them.
"""
from __future__ import annotations

import math

import torch
import torch.nn.functional as F

FP8_MAX = 448.0  # largest finite OCP e4m3fn value


# --------------------------------------------------------------------------- a1
def store_kvcache(key, value, k_cache, v_cache, slot_mapping):
    """tinyvllm/layers/attention.py:33-48 (kernel 9-30; spec twin 52-67).

    ``cache.view(-1, D)[slot[i]] = x[i].view(D)`` for K and V, a bit copy.
    ``key``/``value`` are ``[N, Hkv, Dh]`` (any row stride), caches are
    ``[nblk, block, Hkv, Dh]`` contiguous, ``slot_mapping`` int32 ``[N]``.
    Negative slots are skipped (graph padding rows must not touch the cache;
    the reference zero-pads and overwrites slot 0, model_runner.py:252-259,
    which this build deliberately does not reproduce).
    """
    n, h, d = key.shape
    D = h * d
    kc = k_cache.view(-1, D)
    vc = v_cache.view(-1, D)
    for i in range(n):
        s = int(slot_mapping[i])
        if s < 0:
            continue
        kc[s] = key[i].reshape(D)
        vc[s] = value[i].reshape(D)


def store_kvcache_fp8(key, value, k_cache, v_cache, slot_mapping, k_scale, v_scale):
    """Build-defined (no reference counterpart): ``c = e4m3(sat(x / s[kvh]))``.

    Caches are ``torch.float8_e4m3fn`` ``[nblk, block, Hkv, Dh]``; ``k_scale`` /
    ``v_scale`` are fp32 ``[Hkv]``.  The division is carried out in fp32.
    """
    n, h, d = key.shape
    kq = quantize_fp8(key, k_scale)
    vq = quantize_fp8(value, v_scale)
    kc = k_cache.view(-1, h, d)
    vc = v_cache.view(-1, h, d)
    for i in range(n):
        s = int(slot_mapping[i])
        if s < 0:
            continue
        kc[s] = kq[i]
        vc[s] = vq[i]


def quantize_fp8(x, scale):
    """``e4m3fn(clamp(float(x) / scale[h], -448, 448))`` for ``x [N, H, D]``."""
    y = x.float() / scale.float().view(1, -1, 1)
    return y.clamp(-FP8_MAX, FP8_MAX).to(torch.float8_e4m3fn)


def dequantize_fp8(c, scale):
    """``float(c) * scale[h]`` for ``c [..., H, D]`` -> fp32."""
    return c.float() * scale.float().view(*([1] * (c.dim() - 2)), -1, 1)


# --------------------------------------------------------------------------- a5 / a6
def rms_norm(x, weight, eps):
    """tinyvllm/layers/layernorm.py:21-31: two bf16 roundings, weight multiply in bf16."""
    dt = x.dtype
    x32 = x.to(torch.float32)
    var = x32.pow(2).mean(dim=-1, keepdim=True)
    x32 = x32 * torch.rsqrt(var + eps)
    return x32.to(dt) * weight.to(dt)


def add_rms_norm(x, residual, weight, eps):
    """tinyvllm/layers/layernorm.py:33-45: variance from the unrounded fp32 sum."""
    dt = x.dtype
    s = x.to(torch.float32) + residual.to(torch.float32)
    residual_out = s.to(dt)
    var = s.pow(2).mean(dim=-1, keepdim=True)
    y = (s * torch.rsqrt(var + eps)).to(dt) * weight.to(dt)
    return y, residual_out


# --------------------------------------------------------------------------- a7
def rope_table(head_size, max_position, base):
    """tinyvllm/layers/rotary_embedding.py:31-36: fp32 ``[max_pos, head_size]`` = cos || sin."""
    inv_freq = 1.0 / (base ** (torch.arange(0, head_size, 2, dtype=torch.float32) / head_size))
    t = torch.arange(max_position, dtype=torch.float32)
    freqs = torch.einsum("i,j -> ij", t, inv_freq)
    return torch.cat((freqs.cos(), freqs.sin()), dim=-1)


def _apply_rotary(x, cos, sin):
    """tinyvllm/layers/rotary_embedding.py:5-15 (neox half split, one rounding)."""
    cos = cos.unsqueeze(-2)
    sin = sin.unsqueeze(-2)
    x1, x2 = torch.chunk(x.to(torch.float32), 2, dim=-1)
    y1 = cos * x1 - sin * x2
    y2 = cos * x2 + sin * x1
    return torch.cat((y1, y2), dim=-1).to(x.dtype)


def rope(positions, query, key, cos_sin_cache, head_size):
    """tinyvllm/layers/rotary_embedding.py:41-57."""
    n = positions.size(0)
    cs = cos_sin_cache[positions]
    cos, sin = cs.chunk(2, -1)
    q = _apply_rotary(query.reshape(n, -1, head_size), cos, sin).reshape(n, -1)
    k = _apply_rotary(key.reshape(n, -1, head_size), cos, sin).reshape(n, -1)
    return q, k


# --------------------------------------------------------------------------- a8
def silu_and_mul(x):
    """tinyvllm/layers/activation.py:11-14 in eager form: bf16(bf16(silu(g)) * u)."""
    g, u = x.chunk(2, -1)
    return F.silu(g) * u


# --------------------------------------------------------------------------- a9
def greedy_sample(logits):
    """tinyvllm/layers/sampler.py:13-14,21 with every temperature 0: first max index."""
    return logits.to(torch.float32).argmax(dim=-1)


def philox4x32_10(counter, key):
    """Philox4x32-10 (Salmon, Moraes, Dror, Shaw: "Parallel random numbers: as easy as 1, 2, 3", SC'11;
    the Random123 library).  ``counter`` uint32 ``[..., 4]``, ``key`` two uint32 -> uint32 ``[..., 4]``."""
    import numpy as np
    c = [np.asarray(counter[..., i], dtype=np.uint64) for i in range(4)]
    k0, k1 = int(key[0]), int(key[1])
    mask = np.uint64(0xFFFFFFFF)
    for _ in range(10):
        p0 = np.uint64(0xD2511F53) * c[0]
        p1 = np.uint64(0xCD9E8D57) * c[2]
        c = [(p1 >> np.uint64(32)) ^ c[1] ^ np.uint64(k0), p1 & mask,
             (p0 >> np.uint64(32)) ^ c[3] ^ np.uint64(k1), p0 & mask]
        k0, k1 = (k0 + 0x9E3779B9) & 0xFFFFFFFF, (k1 + 0xBB67AE85) & 0xFFFFFFFF
    return np.stack(c, -1).astype(np.uint32)


def sample_scores(logits, temperatures, seed, offset):
    """Build-defined noise for tinyvllm/layers/sampler.py:15-20.  The reference's
    ``argmax(softmax(l / T) / (e + 1e-10))`` with ``e ~ Exp(1)`` equals ``argmax(l / T - log(e + 1e-10))``
    (common normaliser, monotone log); ``e = -log(u)``, ``u = (x >> 8) 2^-24 + 2^-25`` with ``x`` the
    Philox word of (key = seed, counter = (i // 4, row, offset), word i % 4).  Rows with T == 0 keep their
    logits.  Returns the fp32 scores ``[rows, vocab]``; the sample is their first argmax."""
    import numpy as np
    l = logits.to(torch.float32).numpy()
    t = np.asarray(temperatures, dtype=np.float32)
    rows, vocab = l.shape
    nq = (vocab + 3) // 4
    ctr = np.zeros((rows, nq, 4), dtype=np.uint32)
    ctr[..., 0] = np.arange(nq, dtype=np.uint32)[None, :]
    ctr[..., 1] = np.arange(rows, dtype=np.uint32)[:, None]
    ctr[..., 2] = offset & 0xFFFFFFFF
    ctr[..., 3] = (offset >> 32) & 0xFFFFFFFF
    x = philox4x32_10(ctr, (seed & 0xFFFFFFFF, (seed >> 32) & 0xFFFFFFFF)).reshape(rows, nq * 4)[:, :vocab]
    u = (x >> np.uint32(8)).astype(np.float32) * np.float32(2.0 ** -24) + np.float32(2.0 ** -25)
    e = -np.log(u, dtype=np.float32)
    safe_t = np.where(t == 0, np.float32(1), t)[:, None]
    noisy = l / safe_t - np.log(e + np.float32(1e-10), dtype=np.float32)
    return torch.from_numpy(np.where((t == 0)[:, None], l, noisy).astype(np.float32))


def sample(logits, temperatures, seed, offset):
    return sample_scores(logits, temperatures, seed, offset).argmax(dim=-1)


# --------------------------------------------------------------------------- a10
def linear(x, weight, bias=None):
    """tinyvllm/layers/linear.py:48-49, 82-83, 180-181: ``bf16(sum_k x[m,k] W[n,k])``."""
    return F.linear(x, weight, bias)


def linear_exact(x, weight):
    """Same contraction with an fp64 accumulator and one rounding to ``x.dtype``."""
    return (x.double() @ weight.double().t()).to(x.dtype)


def quantize_w8(weight):
    """Build-defined symmetric per-output-channel int8 quantiser for ``W [N, K]``.

    ``scale[n] = max_k |W[n,k]| / 127`` (fp32; 1.0 for an all-zero row),
    ``Wq = clamp(round_half_even(W / scale), -127, 127)``.
    """
    w = weight.float()
    amax = w.abs().amax(dim=1)
    scale = torch.where(amax > 0, amax / 127.0, torch.ones_like(amax))
    wq = torch.round(w / scale[:, None]).clamp(-127, 127).to(torch.int8)
    return wq, scale


def w8a16_linear(x, wq, scale):
    """Build-defined: ``y = bf16( (sum_k x[m,k] * float(Wq[n,k])) * scale[n] )``.

    The contraction is done in fp64 here (the int8 -> float conversion is exact,
    products of a bf16 and an int8 value are exact in fp32) and the scale is
    applied in fp32 to the fp32-rounded sum.
    """
    acc = (x.double() @ wq.double().t()).float()
    return (acc * scale.float()[None, :]).to(x.dtype)


# --------------------------------------------------------------------------- a3
def _gather_paged(cache, block_table, ctx):
    """Rows ``0..ctx-1`` of one sequence from ``cache [nblk, bs, Hkv, Dh]``."""
    bs = cache.shape[1]
    nb = (ctx + bs - 1) // bs
    rows = cache[block_table[:nb].long()].reshape(nb * bs, *cache.shape[2:])
    return rows[:ctx]


def paged_decode_attention(q, k_cache, v_cache, context_lens, block_tables, scale,
                           k_scale=None, v_scale=None):
    """tinyvllm/layers/attention.py:106-109 (``flash_attn_with_kvcache``, one query per seq).

    ``q [B, Hq, Dh]``; K/V row ``t`` of sequence ``b`` is
    ``cache[block_tables[b, t // bs], t % bs, h // (Hq/Hkv), :]``; returns
    ``[B, Hq*Dh]`` = ``bf16(softmax(scale * q K^T) V)`` computed in fp32.  With
    ``k_scale``/``v_scale`` the caches are e4m3 and are dequantised first.
    """
    B, Hq, Dh = q.shape
    Hkv = k_cache.shape[2]
    rep = Hq // Hkv
    out = torch.empty(B, Hq * Dh, dtype=q.dtype)
    for b in range(B):
        ctx = int(context_lens[b])
        k = _gather_paged(k_cache, block_tables[b], ctx)
        v = _gather_paged(v_cache, block_tables[b], ctx)
        if k_scale is not None:
            k = dequantize_fp8(k, k_scale)
            v = dequantize_fp8(v, v_scale)
        k = k.float().repeat_interleave(rep, dim=1)  # [ctx, Hq, Dh]
        v = v.float().repeat_interleave(rep, dim=1)
        s = torch.einsum("hd,thd->ht", q[b].float(), k) * scale
        p = torch.softmax(s, dim=-1)
        out[b] = torch.einsum("ht,thd->hd", p, v).reshape(-1).to(q.dtype)
    return out


# --------------------------------------------------------------------------- a4
def varlen_prefill_attention(q, k, v, cu_seqlens_q, cu_seqlens_k, scale,
                             block_tables=None, k_scale=None, v_scale=None):
    """tinyvllm/layers/attention.py:96-105 (``flash_attn_varlen_func``, causal).

    ``q [Sq, Hq, Dh]``.  Without ``block_tables``: ``k``/``v`` are ``[Sk, Hkv, Dh]``
    packed by ``cu_seqlens_k``.  With ``block_tables``: ``k``/``v`` are the paged
    caches ``[nblk, bs, Hkv, Dh]`` and every sequence reads its K/V rows from
    them (attention.py:99-100).  The causal mask is bottom-right aligned: query
    ``i`` of a sequence with ``c = len_k - len_q`` cached tokens sees keys
    ``0..c+i``.  Returns ``[Sq, Hq*Dh]``.
    """
    Sq, Hq, Dh = q.shape
    Hkv = k.shape[-2]
    rep = Hq // Hkv
    nseq = cu_seqlens_q.numel() - 1
    out = torch.empty(Sq, Hq * Dh, dtype=q.dtype)
    for b in range(nseq):
        q0, q1 = int(cu_seqlens_q[b]), int(cu_seqlens_q[b + 1])
        k0, k1 = int(cu_seqlens_k[b]), int(cu_seqlens_k[b + 1])
        lq, lk = q1 - q0, k1 - k0
        if lq == 0:
            continue
        if block_tables is None:
            kb, vb = k[k0:k1], v[k0:k1]
        else:
            kb = _gather_paged(k, block_tables[b], lk)
            vb = _gather_paged(v, block_tables[b], lk)
            if k_scale is not None:
                kb = dequantize_fp8(kb, k_scale)
                vb = dequantize_fp8(vb, v_scale)
        kb = kb.float().repeat_interleave(rep, dim=1)
        vb = vb.float().repeat_interleave(rep, dim=1)
        s = torch.einsum("qhd,khd->hqk", q[q0:q1].float(), kb) * scale
        qi = torch.arange(lq).view(-1, 1)
        ki = torch.arange(lk).view(1, -1)
        s = s.masked_fill(ki > qi + (lk - lq), float("-inf"))
        p = torch.softmax(s, dim=-1)
        out[q0:q1] = torch.einsum("hqk,khd->qhd", p, vb).reshape(lq, -1).to(q.dtype)
    return out


# --------------------------------------------------------------------------- K9 / K10
def embedding(ids, weight):
    """tinyvllm/layers/embed_head.py:38."""
    return F.embedding(ids, weight)


def lm_head(hidden, weight, cu_seqlens_q=None):
    """tinyvllm/layers/embed_head.py:58-63: last token of each sequence in prefill, then logits."""
    if cu_seqlens_q is not None:
        hidden = hidden[(cu_seqlens_q[1:] - 1).long()].contiguous()
    return F.linear(hidden, weight)


def softmax_scale(head_dim):
    """tinyvllm/models/qwen3.py:41."""
    return head_dim ** (-0.5)


def bf16_ulp(x):
    """Spacing of bfloat16 at ``|x|`` (fp32 tensor), for tolerance statements in tests."""
    e = torch.floor(torch.log2(x.abs().float().clamp_min(2.0 ** -126)))
    return torch.exp2(e - 7)


__all__ = [n for n in dir() if not n.startswith("_") and n not in ("math", "torch", "F", "annotations")]
