"""GPU checks over randomly drawn shapes (seeded): the hand-picked shapes of the other GPU tests name the plans and
boundaries they cover; these walk the planner and the attention kernels' share / segment / tile logic through
shapes nobody picked.

* GEMM entry points: integer-valued activations and small integer weights make every product and every fp32
  partial sum exact, so the result must be bit-identical to an fp64 product rounded once to bf16 -- whatever
  tile, split of K or kernel the plan takes.  The fused forms must equal the calls they replace bit for bit.
* Attention: floating-point kernels, compared with a plain fp32 softmax(QK^T)V evaluated with torch on the same
  device (the CPU oracle would take minutes at these counts): 2e-2 max-abs against the exact result and 1e-3
  relative L2 against the exact result rounded to bf16 (the rounding of the output alone is 1-2e-3 of the
  norm, so it is taken out of the comparison).
"""
import math
import random

import pytest
import torch

pytestmark = pytest.mark.gpu
BF = torch.bfloat16
DEV = "cuda"


def _bits(t):
    return t.contiguous().view(torch.int16)


@pytest.mark.parametrize("seed", [11, 12])
def test_gemm_entry_points_bit_exact_on_integer_data_over_random_shapes(seed):
    import ctypes
    from oracle import ops as O
    from tinyllmforge_amd import _lib, ops as P
    lib = _lib.load()
    rnd = random.Random(seed)
    torch.manual_seed(seed)
    plans = set()
    tab = O.rope_table(128, 512, 1e6).to(DEV)
    for case in range(70):
        M = rnd.choice([rnd.randint(1, 16), rnd.randint(13, 40), rnd.randint(33, 130), rnd.randint(120, 260),
                        rnd.randint(250, 700)])
        N = 16 * rnd.choice([rnd.randint(1, 40), rnd.randint(200, 420), rnd.randint(1500, 1600), 256, 384, 1536, 257])
        K = 64 * rnd.choice([1, 2, 3, 5, 8, 16, 32, 64, 64, 80, 192, rnd.randint(1, 200)])
        what = f"case {case}: M={M} N={N} K={K}"
        x = torch.randint(-4, 5, (M, K), device=DEV).to(BF)
        wq = torch.randint(-3, 4, (N, K), device=DEV, dtype=torch.int8)
        scale = 2.0 ** -9 * torch.randint(1, 4, (N,), device=DEV).float()
        plan = (ctypes.c_int32 * 8)()
        assert lib.tlf_gemm_plan(M, N, K, 1, plan) == 0, what
        plans.add(tuple(plan)[:6])
        ref = ((x.double() @ wq.double().t()) * scale.double()[None, :]).to(BF)
        got = P.w8a16_linear(x, wq, scale)
        assert torch.equal(_bits(got), _bits(ref)), what
        wb = wq.to(BF)
        gotb = P.bf16_linear(x, wb)
        assert torch.equal(_bits(gotb), _bits((x.double() @ wb.double().t()).to(BF))), what
        # LM head + greedy sample: torch.argmax returns the first maximal index, as the reference's sampler does
        assert torch.equal(P.bf16_linear_argmax(x, wb), torch.argmax(gotb.float(), dim=-1)), what
        # projection + add-RMSNorm
        if N <= 16384:
            res = torch.randn(M, N, device=DEV).to(BF)
            nw = (1 + 0.1 * torch.randn(N, device=DEV)).to(BF)
            y2, r2 = P.add_rms_norm(got, res, nw, 1e-6)
            y1, r1 = P.linear_add_rms_norm(x, wq, scale, res, nw, 1e-6)
            assert torch.equal(_bits(y1), _bits(y2)) and torch.equal(_bits(r1), _bits(r2)), what
        # gate_up projection + SiLU-and-mul
        idx = P.gate_up_interleave_index(N, device=DEV)
        fused = P.w8a16_linear_silu_mul(x, wq[idx].contiguous(), scale[idx].contiguous())
        assert torch.equal(_bits(fused), _bits(P.silu_and_mul(got))), what
        # qkv projection + q/k norm + RoPE + cache store
        if M <= 1024:
            hk = rnd.choice([1, 2, 4, 8])
            hq = hk * rnd.choice([1, 2, 4])
            nq = (hq + 2 * hk) * 128
            w2 = P.pack_w8(torch.randint(-3, 4, (nq, K), device=DEV, dtype=torch.int8))
            s2 = torch.rand(nq, device=DEV) * 2e-3 + 1e-4
            x2 = torch.randn(M, K, device=DEV).to(BF)
            pos = torch.randint(0, 512, (M,), device=DEV)
            qw = (1 + 0.2 * torch.randn(128, device=DEV)).to(BF)
            kw = (1 + 0.2 * torch.randn(128, device=DEV)).to(BF)
            slots = torch.randperm(4 * 256, device=DEV)[:M].to(torch.int32)
            kc1 = torch.zeros(4, 256, hk, 128, device=DEV, dtype=BF)
            vc1, kc2, vc2 = kc1.clone(), kc1.clone(), kc1.clone()
            q1, _, _ = P.linear_qknorm_rope_store(x2, w2, s2, qw, kw, 1e-6, pos, tab, hq, hk, 128, kc1, vc1, slots)
            q2, _, _ = P.qknorm_rope_store(P.w8a16_linear(x2, w2, s2), qw, kw, 1e-6, pos, tab, hq, hk, 128, kc2, vc2,
                                           slots)
            assert torch.equal(q1, q2) and torch.equal(kc1, kc2) and torch.equal(vc1, vc2), what
    assert len(plans) >= 15, plans     # the draw reaches many tiles, splits and all three kernels


def _quantise(cache, scales):
    hkv = scales.numel()
    c8 = (cache.float() / scales.view(1, 1, hkv, 1)).clamp(-448, 448).to(torch.float8_e4m3fn)
    return c8, c8.float() * scales.view(1, 1, hkv, 1)


def _assert_attention_close(out, ref, what):
    assert torch.isfinite(out).all(), what
    err = (out - ref).abs().max().item()
    rel = ((out - ref.to(BF).float()).norm() / ref.norm().clamp_min(1e-6)).item()
    assert err <= 2e-2 and rel <= 1e-3, f"{what}: max-abs {err:.3e}, relative L2 {rel:.3e}"


@pytest.mark.parametrize("seed", [21, 22])
def test_paged_decode_attention_over_random_shapes(seed):
    from tinyllmforge_amd import ops as P
    rnd = random.Random(seed)
    torch.manual_seed(seed)
    scale = 1.0 / math.sqrt(128)
    for case in range(60):
        hkv = rnd.choice([1, 2, 4, 8, 16])
        group = rnd.choice([1, 2, 4, 8])
        hq = hkv * group
        bs = rnd.choice([16, 32, 64, 128, 256])
        B = rnd.choice([1, 2, 3, rnd.randint(4, 40), rnd.randint(40, 300)])
        maxctx = rnd.choice([16, 100, 700, 3000]) if B < 64 else rnd.choice([16, 100, 700])
        ctx = torch.tensor([rnd.choice([0, 1, rnd.randint(1, maxctx), rnd.randint(1, maxctx), maxctx])
                            for _ in range(B)], dtype=torch.int32)
        nb = (ctx + bs - 1) // bs
        maxb = max(1, int(nb.max())) + rnd.randint(0, 2)
        nblk = int(nb.sum()) + 3
        fp8 = rnd.random() < 0.4
        what = f"case {case}: B={B} Hkv={hkv} group={group} block={bs} e4m3={fp8} max ctx={maxctx}"
        kc = torch.randn(nblk, bs, hkv, 128, device=DEV).to(BF)
        vc = torch.randn(nblk, bs, hkv, 128, device=DEV).to(BF)
        ks = vs = None
        kref, vref = kc.float(), vc.float()
        if fp8:
            ks = torch.rand(hkv, device=DEV) * 0.02 + 0.01
            vs = torch.rand(hkv, device=DEV) * 0.02 + 0.01
            kc, kref = _quantise(kc, ks)
            vc, vref = _quantise(vc, vs)
        perm = torch.randperm(nblk)
        bt = torch.full((B, maxb), -1, dtype=torch.int32)      # unused entries stay unmapped
        nxt = 0
        for b in range(B):
            bt[b, :int(nb[b])] = perm[nxt:nxt + int(nb[b])].to(torch.int32)
            nxt += int(nb[b])
        q = torch.randn(B, hq, 128, device=DEV).to(BF)
        out = P.paged_decode_attention(q, kc, vc, ctx.to(DEV), bt.to(DEV), scale, k_scale=ks, v_scale=vs)
        out = out.float().view(B, hq, 128)
        ref = torch.zeros(B, hq, 128, device=DEV)              # an empty sequence attends to nothing: zeros
        for b in range(B):
            c = int(ctx[b])
            if c == 0:
                continue
            ids = bt[b, :int(nb[b])].long().to(DEV)
            K = kref[ids].reshape(-1, hkv, 128)[:c].repeat_interleave(group, dim=1)
            V = vref[ids].reshape(-1, hkv, 128)[:c].repeat_interleave(group, dim=1)
            p = torch.softmax(torch.einsum("hd,chd->hc", q[b].float(), K) * scale, dim=-1)
            ref[b] = torch.einsum("hc,chd->hd", p, V)
        _assert_attention_close(out, ref, what)


@pytest.mark.parametrize("seed", [31, 32])
def test_varlen_prefill_attention_over_random_shapes(seed):
    from tinyllmforge_amd import ops as P
    rnd = random.Random(seed)
    torch.manual_seed(seed)
    scale = 1.0 / math.sqrt(128)
    for case in range(40):
        hkv = rnd.choice([1, 2, 4, 8])
        group = rnd.choice([1, 2, 4, 8])
        hq = hkv * group
        nseq = rnd.choice([1, 2, 3, rnd.randint(4, 24)])
        top = 2500 if rnd.random() < 0.2 else 600
        lens = [rnd.choice([1, 2, rnd.randint(1, 70), rnd.randint(1, 300), rnd.randint(300, top)]) for _ in range(nseq)]
        paged = rnd.random() < 0.5
        fp8 = paged and rnd.random() < 0.5
        bs = rnd.choice([16, 64, 256])
        cached = [rnd.choice([0, 0, bs * rnd.randint(1, 3)]) if paged else 0 for _ in range(nseq)]   # prefix hits
        lk = [n + c for n, c in zip(lens, cached)]
        what = (f"case {case}: {nseq} sequences, Hkv={hkv} group={group} paged={paged} e4m3={fp8} block={bs} "
                f"lens={lens[:6]} cached={cached[:6]}")
        cu_q = torch.tensor([0] + torch.tensor(lens).cumsum(0).tolist(), dtype=torch.int32, device=DEV)
        cu_k = torch.tensor([0] + torch.tensor(lk).cumsum(0).tolist(), dtype=torch.int32, device=DEV)
        q = torch.randn(sum(lens), hq, 128, device=DEV).to(BF)
        kfull = torch.randn(sum(lk), hkv, 128, device=DEV).to(BF)
        vfull = torch.randn(sum(lk), hkv, 128, device=DEV).to(BF)
        if paged:
            nb = [(n + bs - 1) // bs for n in lk]
            nblk = sum(nb) + 2
            perm = torch.randperm(nblk)
            bt = torch.full((nseq, max(nb) + rnd.randint(0, 1)), -1, dtype=torch.int32)
            kc = torch.zeros(nblk, bs, hkv, 128, device=DEV, dtype=BF)
            vc = kc.clone()
            nxt = off = 0
            for s in range(nseq):
                ids = perm[nxt:nxt + nb[s]]
                nxt += nb[s]
                bt[s, :nb[s]] = ids.to(torch.int32)
                pad = torch.zeros(nb[s] * bs - lk[s], hkv, 128, device=DEV, dtype=BF)
                kc[ids.to(DEV)] = torch.cat([kfull[off:off + lk[s]], pad]).view(nb[s], bs, hkv, 128)
                vc[ids.to(DEV)] = torch.cat([vfull[off:off + lk[s]], pad]).view(nb[s], bs, hkv, 128)
                off += lk[s]
            ks = vs = None
            kref, vref = kc.float(), vc.float()
            if fp8:
                ks = torch.rand(hkv, device=DEV) * 0.02 + 0.01
                vs = torch.rand(hkv, device=DEV) * 0.02 + 0.01
                kc, kref = _quantise(kc, ks)
                vc, vref = _quantise(vc, vs)
            out = P.varlen_prefill_attention(q, kc, vc, cu_q, cu_k, max(lens), scale, block_tables=bt.to(DEV),
                                             k_scale=ks, v_scale=vs)
        else:
            out = P.varlen_prefill_attention(q, kfull, vfull, cu_q, cu_k, max(lens), scale)
        out = out.float().view(-1, hq, 128)
        ref = torch.zeros_like(out)
        offq = offk = 0
        for s in range(nseq):
            if paged:
                ids = bt[s, :(lk[s] + bs - 1) // bs].long().to(DEV)
                K = kref[ids].reshape(-1, hkv, 128)[:lk[s]]
                V = vref[ids].reshape(-1, hkv, 128)[:lk[s]]
            else:
                K = kfull[offk:offk + lk[s]].float()
                V = vfull[offk:offk + lk[s]].float()
            K = K.repeat_interleave(group, dim=1)
            V = V.repeat_interleave(group, dim=1)
            sc = torch.einsum("qhd,khd->hqk", q[offq:offq + lens[s]].float(), K) * scale
            # query i of a sequence behind `cached` cached tokens sees keys 0 .. cached + i
            seen = torch.arange(lk[s], device=DEV)[None, :] <= torch.arange(lens[s], device=DEV)[:, None] + cached[s]
            sc = sc.masked_fill(~seen[None], float("-inf"))
            ref[offq:offq + lens[s]] = torch.einsum("hqk,khd->qhd", torch.softmax(sc, dim=-1), V)
            offq += lens[s]
            offk += lk[s]
        _assert_attention_close(out, ref, what)
