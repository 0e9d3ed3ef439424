"""Pins for the CPU oracle: closed forms, invariants, library routines and brute force.

The reference ships no tests or golden vectors, so each oracle function is pinned
by something independent of its own formula.
"""
import math

import numpy as np
import pytest
import torch
import torch.nn.functional as F

from oracle import ops as O

BF = torch.bfloat16


def g(seed):
    return torch.Generator().manual_seed(seed)


# ---------------------------------------------------------------- store_kvcache
def test_store_kvcache_bruteforce_and_untouched_slots():
    N, H, D, nblk, bs = 37, 2, 8, 5, 16
    qkv = torch.randn(N, 6 * H * D, generator=g(0)).to(BF)
    key = qkv[:, :H * D].contiguous().view(N, H, D)
    value = qkv[:, 4 * H * D:5 * H * D].view(N, H, D)        # strided view, like the qkv split
    assert value.stride(0) != H * D
    slots = torch.randperm(nblk * bs, generator=g(1))[:N].to(torch.int32)
    kc = torch.full((nblk, bs, H, D), 7.0, dtype=BF)
    vc = torch.full((nblk, bs, H, D), 9.0, dtype=BF)
    O.store_kvcache(key, value, kc, vc, slots)
    kf, vf = kc.view(-1, H * D), vc.view(-1, H * D)
    written = set(slots.tolist())
    for s in range(nblk * bs):
        if s in written:
            i = slots.tolist().index(s)
            assert torch.equal(kf[s], key[i].reshape(-1)) and torch.equal(vf[s], value[i].reshape(-1))
        else:
            assert (kf[s] == 7.0).all() and (vf[s] == 9.0).all()


def test_store_kvcache_negative_slot_skipped():
    key = torch.ones(3, 1, 4, dtype=BF)
    kc = torch.zeros(2, 2, 1, 4, dtype=BF)
    vc = torch.zeros(2, 2, 1, 4, dtype=BF)
    O.store_kvcache(key, key * 2, kc, vc, torch.tensor([1, -1, 3], dtype=torch.int32))
    assert kc.view(4, 4).sum(1).tolist() == [0, 4, 0, 4]
    assert vc.view(4, 4).sum(1).tolist() == [0, 8, 0, 8]


# ---------------------------------------------------------------- rmsnorm
def test_rms_norm_closed_form_and_unit_rms():
    x = (torch.randn(9, 256, generator=g(2)) * 3).to(BF)
    w = (1 + 0.1 * torch.randn(256, generator=g(3))).to(BF)
    y = O.rms_norm(x, w, 1e-6)
    xd = x.double()
    ref = xd / torch.sqrt((xd * xd).mean(-1, keepdim=True) + 1e-6) * w.double()
    assert y.dtype == BF
    # two bf16 roundings: within 2 ulp of the unrounded closed form
    assert ((y.double() - ref).abs() <= 2 * O.bf16_ulp(ref.float()).double()).all()
    y1 = O.rms_norm(x, torch.ones(256, dtype=BF), 0.0).double()
    assert torch.allclose((y1 * y1).mean(-1), torch.ones(9, dtype=torch.float64), atol=5e-3)


def test_rms_norm_rounds_before_weight_multiply():
    # a value where rounding the normalised x first changes the product
    x = torch.tensor([[1.0, 1.0078125, 0.0, 0.0]]).to(BF)
    w = torch.tensor([1.0, 3.0, 1.0, 1.0]).to(BF)
    y = O.rms_norm(x, w, 0.0)
    n = (x.float() * torch.rsqrt(x.float().pow(2).mean(-1, keepdim=True))).to(BF)
    assert torch.equal(y, (n.float() * w.float()).to(BF))


def test_add_rms_norm_reduces_to_rms_norm_and_residual_is_rounded_sum():
    x = torch.randn(5, 128, generator=g(4)).to(BF)
    r = torch.randn(5, 128, generator=g(5)).to(BF)
    w = torch.randn(128, generator=g(6)).to(BF)
    y0, r0 = O.add_rms_norm(x, torch.zeros_like(x), w, 1e-6)
    assert torch.equal(y0, O.rms_norm(x, w, 1e-6)) and torch.equal(r0, x)
    y, ro = O.add_rms_norm(x, r, w, 1e-6)
    assert torch.equal(ro, (x.float() + r.float()).to(BF))
    s = x.double() + r.double()
    ref = s / torch.sqrt((s * s).mean(-1, keepdim=True) + 1e-6) * w.double()
    assert ((y.double() - ref).abs() <= 2 * O.bf16_ulp(ref.float()).double() + 1e-12).all()
    # variance comes from the unrounded sum, not from residual_out: differs from the
    # "round first" variant somewhere on a large enough sample
    xs = torch.randn(400, 128, generator=g(7)).to(BF)
    rs = torch.randn(400, 128, generator=g(8)).to(BF)
    ya, rb = O.add_rms_norm(xs, rs, w, 1e-6)
    yb = O.rms_norm(rb, w, 1e-6)
    assert not torch.equal(ya, yb)


# ---------------------------------------------------------------- rope
def test_rope_table_closed_form():
    t = O.rope_table(128, 64, 1e6)
    assert t.shape == (64, 128) and t.dtype == torch.float32
    p, j = 37, 5
    ang = p * (1e6 ** (-(2 * j) / 128))
    assert abs(t[p, j].item() - math.cos(ang)) < 1e-5 and abs(t[p, 64 + j].item() - math.sin(ang)) < 1e-5
    assert torch.equal(t[0, :64], torch.ones(64)) and torch.equal(t[0, 64:], torch.zeros(64))


def test_rope_identity_norm_and_composition():
    tab = O.rope_table(128, 512, 1e4)
    q = torch.randn(6, 4 * 128, generator=g(9)).to(BF)
    k = torch.randn(6, 2 * 128, generator=g(10)).to(BF)
    q0, k0 = O.rope(torch.zeros(6, dtype=torch.int64), q, k, tab, 128)
    assert torch.equal(q0, q) and torch.equal(k0, k)            # pos 0 is the identity
    pos = torch.tensor([1, 7, 100, 255, 300, 511])
    # fp32 inputs isolate the rotation from bf16 rounding
    qf, kf = q.float(), k.float()
    q1, k1 = O.rope(pos, qf, kf, tab, 128)
    a = qf.view(6, 4, 2, 64)
    b = q1.view(6, 4, 2, 64)
    assert torch.allclose((a ** 2).sum(2), (b ** 2).sum(2), rtol=1e-5, atol=1e-6)  # pairs (i, i+64) keep their norm
    # neox pairing, not interleaved: pair (i, i+64) rotated by angle pos * inv_freq[i]
    i, n, h = 3, 2, 1
    ang = pos[n].item() * (1e4 ** (-(2 * i) / 128))
    x1, x2 = a[n, h, 0, i].item(), a[n, h, 1, i].item()
    assert abs(b[n, h, 0, i].item() - (math.cos(ang) * x1 - math.sin(ang) * x2)) < 1e-4
    assert abs(b[n, h, 1, i].item() - (math.cos(ang) * x2 + math.sin(ang) * x1)) < 1e-4
    # R(p1) R(p2) = R(p1 + p2)
    p1, p2 = torch.tensor([3] * 6), torch.tensor([10] * 6)
    qa, _ = O.rope(p1, qf, kf, tab, 128)
    qb, _ = O.rope(p2, qa, kf, tab, 128)
    qc, _ = O.rope(p1 + p2, qf, kf, tab, 128)
    assert torch.allclose(qb, qc, atol=1e-4)
    # bf16 path is one rounding of the fp32 result
    qh, _ = O.rope(pos, q, k, tab, 128)
    assert torch.equal(qh, q1.to(BF))


# ---------------------------------------------------------------- silu_and_mul
def test_silu_and_mul_library_and_closed_form():
    x = (torch.randn(7, 2 * 96, generator=g(11)) * 4).to(BF)
    y = O.silu_and_mul(x)
    gt, up = x[:, :96], x[:, 96:]
    assert torch.equal(y, F.silu(gt) * up)
    sd = gt.double() / (1 + torch.exp(-gt.double()))
    assert torch.equal(y, (sd.to(BF).float() * up.float()).to(BF))   # two roundings
    assert y.shape == (7, 96)


# ---------------------------------------------------------------- sampler
def test_greedy_sample_ties_take_first_index():
    l = torch.tensor([[0.0, 2.0, 2.0, -1.0], [5.0, 5.0, 5.0, 5.0], [-3.0, -2.0, -2.5, -2.0]]).to(BF)
    assert O.greedy_sample(l).tolist() == [1, 0, 1]
    big = torch.randn(3, 5000, generator=g(12)).to(BF)
    assert torch.equal(O.greedy_sample(big), torch.argmax(big.float(), -1))
    assert O.greedy_sample(big).dtype == torch.int64


# ---------------------------------------------------------------- linear / w8a16
def test_philox4x32_10_known_answers():
    """The three known-answer vectors of the Random123 distribution (kat_vectors, philox4x32 10)."""
    kats = [((0, 0, 0, 0), (0, 0), (0x6627e8d5, 0xe169c58d, 0xbc57ac4c, 0x9b00dbd8)),
            ((0xffffffff,) * 4, (0xffffffff,) * 2, (0x408f276d, 0x41c83b0e, 0xa20bc7c6, 0x6d5451fd)),
            ((0x243f6a88, 0x85a308d3, 0x13198a2e, 0x03707344), (0xa4093822, 0x299f31d0),
             (0xd16cfe09, 0x94fdcceb, 0x5001e420, 0x24126ea1))]
    for ctr, key, want in kats:
        got = O.philox4x32_10(np.array(ctr, dtype=np.uint32), key)
        assert tuple(int(v) for v in got) == want
    both = O.philox4x32_10(np.array([kats[0][0], kats[2][0]], dtype=np.uint32)[:, None, :].repeat(3, 1), (0, 0))
    assert both.shape == (2, 3, 4) and tuple(int(v) for v in both[0, 2]) == kats[0][2]      # batched counters


def test_sample_is_the_reference_formula_on_the_same_noise_and_follows_softmax():
    """(1) T == 0 rows keep their logits (greedy, first index).  (2) On the noise the oracle draws, its choice
    maximises the reference's own expression softmax(l/T) / (e + 1e-10) (sampler.py:15-20) evaluated in fp64.
    (3) 40000 independent draws from one row follow softmax(l/T): chi-square over 8 tokens, 7 degrees of
    freedom, bound 30 (p ~ 1e-4).  (4) other offsets and seeds give other draws."""
    l = (torch.randn(64, 1003, generator=g(5)) * 2).to(BF)
    t = torch.tensor([0.0, 0.5, 1.0, 2.0] * 16)
    sc = O.sample_scores(l, t, seed=7, offset=3)
    assert torch.equal(sc[0::4], l[0::4].float())
    ids = O.sample(l, t, 7, 3)
    assert torch.equal(ids[0::4], O.greedy_sample(l[0::4]))
    # recover e from the scores' definition independently: same Philox words, fp64 arithmetic
    rows, vocab = l.shape
    ctr = np.zeros((rows, (vocab + 3) // 4, 4), dtype=np.uint32)
    ctr[..., 0] = np.arange(ctr.shape[1])[None, :]; ctr[..., 1] = np.arange(rows)[:, None]; ctr[..., 2] = 3
    x = O.philox4x32_10(ctr, (7, 0)).reshape(rows, -1)[:, :vocab]
    e = -np.log((x >> 8).astype(np.float64) * 2.0 ** -24 + 2.0 ** -25)
    for r in range(rows):
        if t[r] == 0:
            continue
        p = torch.softmax(l[r].double() / float(t[r]), -1).numpy() / (e[r] + 1e-10)
        assert p[ids[r]] >= p.max() * (1 - 1e-5), r
    logits = torch.tensor([[2.0, 1.0, 0.5, 0.0, -0.5, -1.0, 1.5, -3.0]]).to(BF).repeat(40000, 1)
    draws = O.sample(logits, torch.full((40000,), 0.7), seed=1, offset=0)
    want = torch.softmax(logits[0].double() / 0.7, -1) * 40000
    got = torch.bincount(draws, minlength=8).double()
    assert (((got - want) ** 2) / want).sum().item() < 30
    assert not torch.equal(draws, O.sample(logits, torch.full((40000,), 0.7), seed=1, offset=1))
    assert not torch.equal(draws, O.sample(logits, torch.full((40000,), 0.7), seed=2, offset=0))


def test_linear_matches_fp64():
    x = torch.randn(5, 64, generator=g(13)).to(BF)
    w = (torch.randn(24, 64, generator=g(14)) * 0.1).to(BF)
    ref = x.double() @ w.double().t()
    assert (O.linear(x, w).double() - ref).abs().max() < 2e-2
    assert (O.linear_exact(x, w).double() - ref).abs().max() <= O.bf16_ulp(ref.float()).max().item()


def test_w8a16_exact_on_integer_inputs():
    x = torch.randint(-8, 9, (6, 128), generator=g(15)).to(BF)          # integers: exact in bf16
    wq = torch.randint(-127, 128, (10, 128), generator=g(16)).to(torch.int8)
    scale = torch.full((10,), 0.5)
    y = O.w8a16_linear(x, wq, scale)
    exact = (x.long() @ wq.long().t())                                    # integer arithmetic
    assert torch.equal(y, (exact.float() * 0.5).to(BF))
    # per-output-channel: scale[n] multiplies column n only
    scale2 = scale.clone(); scale2[3] = 2.0
    y2 = O.w8a16_linear(x, wq, scale2)
    assert torch.equal(y2[:, 3], (exact[:, 3].float() * 2.0).to(BF))
    assert torch.equal(torch.cat([y2[:, :3], y2[:, 4:]], 1), torch.cat([y[:, :3], y[:, 4:]], 1))


def test_quantize_w8_roundtrip():
    w = torch.randn(12, 40, generator=g(17))
    wq, s = O.quantize_w8(w)
    assert wq.dtype == torch.int8 and s.shape == (12,) and wq.abs().max() <= 127
    assert (wq.float() * s[:, None] - w).abs().max() <= s.max() * 0.5 + 1e-7
    assert (wq.abs().amax(1) == 127).all()
    z, sz = O.quantize_w8(torch.zeros(2, 4))
    assert (z == 0).all() and (sz == 1).all()


# ---------------------------------------------------------------- paged decode attention
def _paged_setup(seed, B, Hq, Hkv, Dh, bs, ctxs, nblk):
    ge = g(seed)
    q = torch.randn(B, Hq, Dh, generator=ge).to(BF)
    kc = torch.randn(nblk, bs, Hkv, Dh, generator=ge).to(BF)
    vc = torch.randn(nblk, bs, Hkv, Dh, generator=ge).to(BF)
    maxb = max((c + bs - 1) // bs for c in ctxs)
    perm = torch.randperm(nblk, generator=ge).tolist()
    bt = torch.full((B, maxb), -1, dtype=torch.int32)
    for b, c in enumerate(ctxs):
        for j in range((c + bs - 1) // bs):
            bt[b, j] = perm.pop()
    return q, kc, vc, torch.tensor(ctxs, dtype=torch.int32), bt


def test_paged_decode_matches_sdpa_and_loops():
    B, Hq, Hkv, Dh, bs = 3, 4, 2, 16, 8
    ctxs = [1, 8, 21]
    q, kc, vc, cl, bt = _paged_setup(20, B, Hq, Hkv, Dh, bs, ctxs, 12)
    scale = Dh ** -0.5
    out = O.paged_decode_attention(q, kc, vc, cl, bt, scale).view(B, Hq, Dh)
    for b, c in enumerate(ctxs):
        rows_k = torch.stack([kc[bt[b, t // bs], t % bs] for t in range(c)])     # [c, Hkv, Dh]
        rows_v = torch.stack([vc[bt[b, t // bs], t % bs] for t in range(c)])
        for h in range(Hq):
            kh, vh = rows_k[:, h // 2].float(), rows_v[:, h // 2].float()
            ref = F.scaled_dot_product_attention(q[b, h].float()[None, None], kh[None], vh[None], scale=scale)[0, 0]
            assert (out[b, h].float() - ref).abs().max() < 1e-2
            # brute force
            s = [sum(q[b, h, d].item() * kh[t, d].item() for d in range(Dh)) * scale for t in range(c)]
            m = max(s); e = [math.exp(v - m) for v in s]; z = sum(e)
            o0 = sum(e[t] / z * vh[t, 0].item() for t in range(c))
            assert abs(out[b, h, 0].item() - o0) < 1e-2
    # ctx = 1 returns the V row itself
    assert torch.equal(out[0].reshape(Hq, Dh), vc[bt[0, 0], 0].repeat_interleave(2, 0))


def test_paged_decode_pool_permutation_invariance():
    B, Hq, Hkv, Dh, bs = 2, 4, 4, 8, 4
    q, kc, vc, cl, bt = _paged_setup(21, B, Hq, Hkv, Dh, bs, [6, 11], 9)
    o1 = O.paged_decode_attention(q, kc, vc, cl, bt, 0.3)
    perm = torch.randperm(9, generator=g(22))
    inv = torch.empty_like(perm); inv[perm] = torch.arange(9)
    kc2, vc2 = kc[perm], vc[perm]                       # new block j holds old block perm[j]
    bt2 = torch.where(bt >= 0, inv[bt.clamp_min(0).long()].to(torch.int32), bt)
    assert torch.equal(o1, O.paged_decode_attention(q, kc2, vc2, cl, bt2, 0.3))


# ---------------------------------------------------------------- varlen prefill attention
def test_prefill_matches_sdpa_causal_and_bottom_right():
    Hq, Hkv, Dh = 4, 2, 16
    lens_q, lens_k = [5, 9, 1], [5, 12, 7]             # seq 1 has 3 cached tokens, seq 2 has 6
    cq = torch.tensor([0] + list(np.cumsum(lens_q)), dtype=torch.int32)
    ck = torch.tensor([0] + list(np.cumsum(lens_k)), dtype=torch.int32)
    ge = g(23)
    q = torch.randn(sum(lens_q), Hq, Dh, generator=ge).to(BF)
    k = torch.randn(sum(lens_k), Hkv, Dh, generator=ge).to(BF)
    v = torch.randn(sum(lens_k), Hkv, Dh, generator=ge).to(BF)
    out = O.varlen_prefill_attention(q, k, v, cq, ck, 0.25).view(-1, Hq, Dh)
    for b in range(3):
        qs = q[cq[b]:cq[b + 1]].float().transpose(0, 1)                   # [Hq, lq, Dh]
        ks = k[ck[b]:ck[b + 1]].float().repeat_interleave(2, 1).transpose(0, 1)
        vs = v[ck[b]:ck[b + 1]].float().repeat_interleave(2, 1).transpose(0, 1)
        lq, lk = lens_q[b], lens_k[b]
        mask = torch.ones(lq, lk, dtype=torch.bool).tril(diagonal=lk - lq)
        ref = F.scaled_dot_product_attention(qs, ks, vs, attn_mask=mask, scale=0.25).transpose(0, 1)
        assert (out[cq[b]:cq[b + 1]].float() - ref).abs().max() < 1e-2
        if lq == lk:
            ref2 = F.scaled_dot_product_attention(qs, ks, vs, is_causal=True, scale=0.25).transpose(0, 1)
            assert (out[cq[b]:cq[b + 1]].float() - ref2).abs().max() < 1e-2


def test_prefill_paged_equals_dense_after_gather():
    Hq, Hkv, Dh, bs = 2, 1, 8, 4
    lens_q, lens_k = [3, 6], [7, 6]
    cq = torch.tensor([0, 3, 9], dtype=torch.int32)
    ck = torch.tensor([0, 7, 13], dtype=torch.int32)
    ge = g(24)
    q = torch.randn(9, Hq, Dh, generator=ge).to(BF)
    kc = torch.randn(6, bs, Hkv, Dh, generator=ge).to(BF)
    vc = torch.randn(6, bs, Hkv, Dh, generator=ge).to(BF)
    bt = torch.tensor([[4, 1], [0, 5]], dtype=torch.int32)
    kd = torch.cat([kc[bt[b].long()].reshape(-1, Hkv, Dh)[:lens_k[b]] for b in range(2)])
    vd = torch.cat([vc[bt[b].long()].reshape(-1, Hkv, Dh)[:lens_k[b]] for b in range(2)])
    a = O.varlen_prefill_attention(q, kc, vc, cq, ck, 0.35, block_tables=bt)
    b_ = O.varlen_prefill_attention(q, kd, vd, cq, ck, 0.35)
    assert torch.equal(a, b_)
    # last query of a prefill sequence == decode attention over the same cache
    d = O.paged_decode_attention(q[[2, 8]], kc, vc, torch.tensor(lens_k, dtype=torch.int32), bt, 0.35)
    assert (a[[2, 8]].float() - d.float()).abs().max() < 1e-2


# ---------------------------------------------------------------- fp8 KV (build-defined)
def test_fp8_quantise_roundtrip_saturation_and_scale():
    vals = torch.tensor([0.0, 1.0, -1.5, 448.0, 0.015625, 240.0]).view(1, 1, -1)
    s = torch.tensor([1.0])
    c = O.quantize_fp8(vals.to(BF), s)
    assert c.dtype == torch.float8_e4m3fn
    assert torch.equal(O.dequantize_fp8(c, s), vals)                        # representable values survive
    assert O.dequantize_fp8(O.quantize_fp8(torch.tensor([[[1e4, -1e4]]]).to(BF), s), s).tolist() == [[[448.0, -448.0]]]
    s2 = torch.tensor([0.25, 4.0])
    x = torch.tensor([[[1.0, 2.0], [8.0, 16.0]]]).to(BF)                     # [1, 2 heads, 2]
    c2 = O.quantize_fp8(x, s2)
    assert torch.equal(c2.float(), torch.tensor([[[4.0, 8.0], [2.0, 4.0]]]))
    assert torch.equal(O.dequantize_fp8(c2, s2), x.float())


def test_fp8_paged_decode_close_to_bf16():
    B, Hq, Hkv, Dh, bs = 2, 4, 2, 16, 8
    q, kc, vc, cl, bt = _paged_setup(25, B, Hq, Hkv, Dh, bs, [9, 17], 8)
    ks = torch.tensor([0.02, 0.03]); vs = torch.tensor([0.025, 0.02])
    k8 = torch.zeros(8, bs, Hkv, Dh, dtype=torch.float8_e4m3fn)
    v8 = torch.zeros(8, bs, Hkv, Dh, dtype=torch.float8_e4m3fn)
    slots = torch.arange(8 * bs, dtype=torch.int32)
    O.store_kvcache_fp8(kc.view(-1, Hkv, Dh), vc.view(-1, Hkv, Dh), k8, v8, slots, ks, vs)
    assert torch.equal(k8.view(-1, Hkv, Dh).float(), O.quantize_fp8(kc.view(-1, Hkv, Dh), ks).float())
    o8 = O.paged_decode_attention(q, k8, v8, cl, bt, 0.25, ks, vs)
    o16 = O.paged_decode_attention(q, kc, vc, cl, bt, 0.25)
    assert (o8.float() - o16.float()).abs().max() < 0.15
    # equals attention over the dequantised rows exactly
    kd = O.dequantize_fp8(k8, ks).to(torch.float32); vd = O.dequantize_fp8(v8, vs).to(torch.float32)
    od = O.paged_decode_attention(q.float(), kd, vd, cl, bt, 0.25).to(BF)
    assert torch.equal(o8, od)
