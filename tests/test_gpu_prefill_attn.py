"""GPU parity: varlen causal prefill attention (dense and paged K/V) against the CPU oracle.

Tolerance (north star): 2e-2 max-abs, 1e-3 relative L2 on bf16 outputs.
"""
import numpy as np
import pytest
import torch

from oracle import ops as O

pytestmark = pytest.mark.gpu
BF = torch.bfloat16
DEV = "cuda"


def g(seed):
    return torch.Generator().manual_seed(seed)


def check(got, ref):
    got, ref = got.float().cpu(), ref.float()
    err = (got - ref).abs().max().item()
    rel = ((got - ref).norm() / ref.norm().clamp_min(1e-9)).item()
    assert err <= 2e-2, f"max abs {err}"
    assert rel <= 1e-3, f"rel l2 {rel}"


def cu(lens):
    return torch.tensor([0] + list(np.cumsum(lens)), dtype=torch.int32)


@pytest.mark.parametrize("Hq,Hkv,lens", [
    (16, 8, [128, 128, 128, 128]),            # config 1 prefill
    (32, 8, [1, 2, 63, 64, 65, 200, 333]),
    (64, 8, [100, 31]),
    (8, 8, [257, 5]),
    (4, 1, [90]),
    (32, 2, [40, 70]),
])
def test_prefill_dense_causal(Hq, Hkv, lens):
    from tinyllmforge_amd import ops as P
    Dh = 128
    S = sum(lens)
    ge = g(S + Hq)
    q = torch.randn(S, Hq, Dh, generator=ge).to(BF)
    # k contiguous, v a strided view into a wider buffer (as the qkv split gives it)
    kv = torch.randn(S, 3 * Hkv * Dh, generator=ge).to(BF)
    k = kv[:, :Hkv * Dh].contiguous().view(S, Hkv, Dh)
    v = kv[:, 2 * Hkv * Dh:].view(S, Hkv, Dh)
    c = cu(lens)
    scale = Dh ** -0.5
    ref = O.varlen_prefill_attention(q, k, v, c, c, scale)
    kvd = kv.to(DEV)
    got = P.varlen_prefill_attention(q.to(DEV), kvd[:, :Hkv * Dh].contiguous().view(S, Hkv, Dh),
                                     kvd[:, 2 * Hkv * Dh:].view(S, Hkv, Dh), c.to(DEV), c.to(DEV), max(lens), scale)
    check(got, ref)


def paged_case(seed, Hq, Hkv, bs, lens_q, lens_k, nblk):
    ge = g(seed)
    Dh = 128
    q = torch.randn(sum(lens_q), Hq, Dh, generator=ge).to(BF)
    kc = torch.randn(nblk, bs, Hkv, Dh, generator=ge).to(BF)
    vc = torch.randn(nblk, bs, Hkv, Dh, generator=ge).to(BF)
    need = [(l + bs - 1) // bs for l in lens_k]
    perm = torch.randperm(nblk, generator=ge).tolist()
    bt = torch.full((len(lens_k), max(need)), -1, dtype=torch.int32)
    for b, n in enumerate(need):
        for j in range(n):
            bt[b, j] = perm.pop()
    return q, kc, vc, cu(lens_q), cu(lens_k), bt


@pytest.mark.parametrize("Hq,Hkv,bs,lens_q,lens_k", [
    (16, 8, 256, [44, 300, 1], [300, 300, 257]),          # prefix hits: 256 cached, none, 256 cached
    (32, 8, 256, [100, 64], [1124, 64]),                  # 1024-token cached prefix
    (64, 8, 16, [7, 33], [39, 33]),
])
def test_prefill_paged_with_prefix(Hq, Hkv, bs, lens_q, lens_k):
    from tinyllmforge_amd import ops as P
    q, kc, vc, cq, ck, bt = paged_case(Hq + bs, Hq, Hkv, bs, lens_q, lens_k, 24 if bs == 256 else 40)
    scale = 128 ** -0.5
    ref = O.varlen_prefill_attention(q, kc, vc, cq, ck, scale, block_tables=bt)
    got = P.varlen_prefill_attention(q.to(DEV), kc.to(DEV), vc.to(DEV), cq.to(DEV), ck.to(DEV), max(lens_q), scale,
                                     block_tables=bt.to(DEV))
    check(got, ref)


def test_prefill_last_row_equals_decode_attention():
    from tinyllmforge_amd import ops as P
    q, kc, vc, cq, ck, bt = paged_case(5, 32, 8, 256, [50, 10], [562, 10], 8)
    scale = 128 ** -0.5
    pre = P.varlen_prefill_attention(q.to(DEV), kc.to(DEV), vc.to(DEV), cq.to(DEV), ck.to(DEV), 50, scale,
                                     block_tables=bt.to(DEV))
    last = torch.tensor([49, 59])
    dec = P.paged_decode_attention(q[last].to(DEV), kc.to(DEV), vc.to(DEV),
                                   torch.tensor([562, 10], dtype=torch.int32, device=DEV), bt.to(DEV), scale)
    assert (pre[last.to(DEV)].float() - dec.float()).abs().max().item() <= 1e-2


def test_prefill_empty_sequence_in_batch_and_fp8_cache():
    from tinyllmforge_amd import ops as P
    Hq, Hkv, bs, Dh = 16, 8, 256, 128
    q, kc, vc, cq, ck, bt = paged_case(6, Hq, Hkv, bs, [20, 0, 9], [276, 0, 9], 8)
    scale = Dh ** -0.5
    ref = O.varlen_prefill_attention(q, kc, vc, cq, ck, scale, block_tables=bt)
    got = P.varlen_prefill_attention(q.to(DEV), kc.to(DEV), vc.to(DEV), cq.to(DEV), ck.to(DEV), 20, scale,
                                     block_tables=bt.to(DEV))
    check(got, ref)
    # e4m3 cache: compare with the oracle on the same quantised rows
    ks = torch.rand(Hkv, generator=g(1)) * 0.02 + 0.01
    vs = torch.rand(Hkv, generator=g(2)) * 0.02 + 0.01
    k8 = O.quantize_fp8(kc.view(-1, Hkv, Dh), ks).view(kc.shape)
    v8 = O.quantize_fp8(vc.view(-1, Hkv, Dh), vs).view(vc.shape)
    ref8 = O.varlen_prefill_attention(q, k8, v8, cq, ck, scale, block_tables=bt, k_scale=ks, v_scale=vs)
    got8 = P.varlen_prefill_attention(q.to(DEV), k8.to(DEV), v8.to(DEV), cq.to(DEV), ck.to(DEV), 20, scale,
                                      block_tables=bt.to(DEV), k_scale=ks.to(DEV), v_scale=vs.to(DEV))
    check(got8, ref8)


def _sampled_rows_check(q, kc, vc, cq, ck, bt, scale, got, rows, k_scale=None, v_scale=None):
    """Oracle on sampled query rows only: a single query at the end of its visible key range is the same
    bottom-right aligned causal problem (CPU time stays in seconds for 8192-token sequences)."""
    got = got.float().cpu()
    num = den = 0.0
    for seq, i in rows:
        lq = int(cq[seq + 1] - cq[seq])
        lk = int(ck[seq + 1] - ck[seq])
        vis = lk - lq + i + 1
        qi = q[int(cq[seq]) + i:int(cq[seq]) + i + 1]
        ref = O.varlen_prefill_attention(qi, kc, vc, cu([1]), cu([vis]), scale, block_tables=bt[seq:seq + 1],
                                         **({} if k_scale is None else dict(k_scale=k_scale, v_scale=v_scale))).float()
        g_ = got[int(cq[seq]) + i:int(cq[seq]) + i + 1]
        assert (g_ - ref).abs().max().item() <= 2e-2, (seq, i)
        num += float((g_ - ref).pow(2).sum())
        den += float(ref.pow(2).sum())
    rel = (num / den) ** 0.5
    assert rel <= 1e-3, f"rel l2 {rel}"
    return rel


@pytest.mark.parametrize("fp8", [False, True])
def test_prefill_long_sequences_behind_cached_prefix(fp8):
    """BASELINE configs[4] shape (64 query heads, 8 KV heads): an 8192-token prompt, and a 4096-token prompt
    behind a 1024-token cached prefix, bf16 and e4m3 cache rows; sampled rows against the oracle.  The second
    product runs in fp16 (P and V): this is the test of its tolerance at full length."""
    from tinyllmforge_amd import ops as P
    Hq, Hkv, bs, Dh = 64, 8, 256, 128
    lens_q, lens_k = [8192, 4096, 300], [8192, 5120, 300]
    nblk = sum((l + bs - 1) // bs for l in lens_k) + 2
    q, kc, vc, cq, ck, bt = paged_case(41, Hq, Hkv, bs, lens_q, lens_k, nblk)
    scale = Dh ** -0.5
    kw, okw = {}, {}
    if fp8:
        ks = torch.rand(Hkv, generator=g(1)) * 0.02 + 0.01
        vs = torch.rand(Hkv, generator=g(2)) * 0.02 + 0.01
        kc = O.quantize_fp8(kc.view(-1, Hkv, Dh), ks).view(kc.shape)
        vc = O.quantize_fp8(vc.view(-1, Hkv, Dh), vs).view(vc.shape)
        kw = dict(k_scale=ks.to(DEV), v_scale=vs.to(DEV))
        okw = dict(k_scale=ks, v_scale=vs)
    got = P.varlen_prefill_attention(q.to(DEV), kc.to(DEV), vc.to(DEV), cq.to(DEV), ck.to(DEV), max(lens_q), scale,
                                     block_tables=bt.to(DEV), **kw)
    rows = [(0, 0), (0, 1), (0, 63), (0, 64), (0, 4095), (0, 8000), (0, 8191), (1, 0), (1, 17), (1, 2048), (1, 4095),
            (2, 0), (2, 299)]
    rel = _sampled_rows_check(q, kc, vc, cq, ck, bt, scale, got, rows, **okw)
    print(f"PREFILL_ERR long fp8={fp8}: rel l2 {rel:.2e}")


@pytest.mark.parametrize("vmag", [1e-6, 1e-3, 1.0, 3e3, 1e5, "mixed"])
def test_prefill_second_product_over_the_range_of_v(vmag):
    """The second product runs in fp16 on tiles fp16 can hold and in bf16 (P as a hi + lo pair) on the others:
    magnitudes of real activations, a million times smaller (fp16 subnormals) and a hundred thousand times larger
    (beyond the largest fp16) meet the same tolerance, and so does a batch whose tiles differ - N(0,1) rows with
    a run of 1e-6 rows that fills whole tiles, single rows of 1e5 and 3e38, and an all-zero run (relative L2; the
    absolute bound scales with the outputs)."""
    from tinyllmforge_amd import ops as P
    Hq, Hkv, Dh = 32, 8, 128
    lens = [700, 130]
    S = sum(lens)
    ge = g(51)
    q = torch.randn(S, Hq, Dh, generator=ge).to(BF)
    k = torch.randn(S, Hkv, Dh, generator=ge).to(BF)
    v = torch.randn(S, Hkv, Dh, generator=ge)
    if vmag == "mixed":
        v[100:300] *= 1e-6            # tiles 2 and 3 of the first sequence hold nothing above 2^-9
        v[300:370] = 0.0              # an all-zero tile (320 .. 383) and zeros beside small values
        v[400, 3] *= 1e5              # one head of one row beyond fp16
        v[690] *= 1e-6
        v[710:730] *= 1e5             # second sequence: a run of large rows
        v[800, 0, 5] = 3.0e38         # near the largest bf16
        out_scale = 1.0
    else:
        v = v * vmag
        out_scale = vmag
    v = v.to(BF)
    c = cu(lens)
    scale = Dh ** -0.5
    ref = O.varlen_prefill_attention(q, k, v, c, c, scale).float()
    got = P.varlen_prefill_attention(q.to(DEV), k.to(DEV), v.to(DEV), c.to(DEV), c.to(DEV), max(lens), scale).float().cpu()
    assert torch.isfinite(got).all()
    if vmag == "mixed":
        # per KV-head group and sequence: the outliers set the scale of the rows that see them, so compare row by row
        num = (got - ref).reshape(S, -1).norm(dim=-1)
        den = ref.reshape(S, -1).norm(dim=-1).clamp_min(1e-30)
        rel_rows = (num / den)
        assert rel_rows.max().item() <= 4e-3, f"worst row rel l2 {rel_rows.max().item()}"
        # rows 100 .. 299 of the first sequence before any large row: outputs of ordinary size, ordinary bound
        assert (got[:400] - ref[:400]).abs().max().item() <= 2e-2
    rel = ((got - ref).norm() / ref.norm()).item()
    assert rel <= 1e-3, f"rel l2 {rel}"
    if vmag != "mixed":
        assert (got - ref).abs().max().item() <= 2e-2 * max(1.0, out_scale)


@pytest.mark.parametrize("fp8", [False, True])
def test_prefill_one_dominant_key_and_thousands_of_faint_ones(fp8):
    """An attention sink: key 0 scores about 10 to 11.5 (natural log units) above every other key, so each of
    the other 8191 keys has a weight of 1e-5 ... 5e-5 of the maximum - below 2^-14, where an unscaled fp16 P would
    be subnormal - while together they carry a fifth of the softmax mass and, their V rows sharing an offset, a
    fifth of the output.  Sampled rows against the fp32 softmax of the oracle at the 1e-3 relative-L2 bar, bf16
    and e4m3 rows."""
    from tinyllmforge_amd import ops as P
    Hq, Hkv, bs, Dh = 32, 8, 256, 128
    L = 8192
    ge = g(61)
    scale = Dh ** -0.5
    u = torch.ones(Dh) / Dh ** 0.5
    alpha = 8.0
    q = (alpha * u[None, None, :] + 0.05 * torch.randn(L, Hq, Dh, generator=ge)).to(BF)
    delta = 10.0 + 1.5 * torch.rand(L, Hkv, generator=ge)                # ln(max weight / this weight)
    beta = (6.0 - delta) / (alpha * scale)
    beta[0] = 6.0 / (alpha * scale)
    krows = beta[:, :, None] * u[None, None, :]
    vrows = 1.0 + 0.5 * torch.randn(L, Hkv, Dh, generator=ge)
    vrows[0] = torch.randn(Hkv, Dh, generator=ge)
    nblk = L // bs
    perm = torch.randperm(nblk, generator=ge)
    kc = torch.zeros(nblk, bs, Hkv, Dh)
    vc = torch.zeros(nblk, bs, Hkv, Dh)
    kc[perm] = krows.view(nblk, bs, Hkv, Dh)
    vc[perm] = vrows.view(nblk, bs, Hkv, Dh)
    kc, vc = kc.to(BF), vc.to(BF)
    bt = perm.to(torch.int32).view(1, nblk)
    cq = ck = cu([L])
    kw, okw = {}, {}
    if fp8:
        ks, vs = torch.full((Hkv,), 1.0 / 64), torch.full((Hkv,), 1.0 / 64)
        kc = O.quantize_fp8(kc.view(-1, Hkv, Dh), ks).view(kc.shape)
        vc = O.quantize_fp8(vc.view(-1, Hkv, Dh), vs).view(vc.shape)
        kw, okw = dict(k_scale=ks.to(DEV), v_scale=vs.to(DEV)), dict(k_scale=ks, v_scale=vs)
    got = P.varlen_prefill_attention(q.to(DEV), kc.to(DEV), vc.to(DEV), cq.to(DEV), ck.to(DEV), L, scale,
                                     block_tables=bt.to(DEV), **kw)
    # the faint keys really are faint, and really matter: weights relative to the maximum, and their total
    kf = kc.float() * (1.0 / 64 if fp8 else 1.0)
    s_last = (q[L - 1, 0].float() @ kf[perm].view(L, Hkv, Dh)[:, 0].t()) * scale
    w = torch.exp(s_last - s_last.max())
    assert w[1:].max().item() < 2.0 ** -14 and 0.1 < w[1:].sum().item() < 0.5, (w[1:].max().item(), w[1:].sum().item())
    rows = [(0, 8191), (0, 8000), (0, 6001), (0, 4096), (0, 1500), (0, 300), (0, 0)]
    rel = _sampled_rows_check(q, kc, vc, cq, ck, bt, scale, got, rows, **okw)
    print(f"PREFILL_ERR sink fp8={fp8}: rel l2 {rel:.2e}, faint keys carry {w[1:].sum().item() / w.sum().item():.2f} of the mass")


def test_prefill_two_launches_replay_in_a_hipgraph():
    """A call on bf16 rows is two launches (the fp16-product kernel, then the bf16 pass over the row tiles that left
    a marker).  Captured in a hipGraph and replayed several times, with eager work and synchronisations between the
    replays and a fresh (garbage) output buffer content before each, every replay must equal the eager result bit for
    bit - on inputs where some row tiles take the bf16 pass and some do not."""
    from tinyllmforge_amd import ops as P
    Hq, Hkv, Dh = 32, 8, 128
    lens = [700, 130]
    S = sum(lens)
    ge = g(77)
    q = torch.randn(S, Hq, Dh, generator=ge).to(BF).to(DEV)
    k = torch.randn(S, Hkv, Dh, generator=ge).to(BF).to(DEV)
    v = torch.randn(S, Hkv, Dh, generator=ge)
    v[400, 3] *= 1e5                 # one head of one row beyond fp16: the row tiles that see it are redone in bf16
    v[100:300] *= 1e-6               # whole tiles below 2^-9
    v = v.to(BF).to(DEV)
    c = cu(lens).to(DEV)
    scale = Dh ** -0.5
    eager = P.varlen_prefill_attention(q, k, v, c, c, max(lens), scale).clone()
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        P.varlen_prefill_attention(q, k, v, c, c, max(lens), scale)      # warm-up on the capture stream
        with torch.cuda.graph(graph, stream=side):
            out = P.varlen_prefill_attention(q, k, v, c, c, max(lens), scale)
    torch.cuda.synchronize()
    for i in range(5):
        if i == 4:
            out.view(torch.int16).fill_(-91)             # 0xffa5 everywhere: the kernel's own marker pattern as stale content
        else:
            out.fill_(float("nan") if i % 2 else 7.0)    # stale contents, including NaN patterns, must not matter
        junk = torch.randn(1 << 20, device=DEV).sum()    # eager work between the replays
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out.view(torch.int16), eager.view(torch.int16)), f"replay {i}"
        assert torch.isfinite(junk)
