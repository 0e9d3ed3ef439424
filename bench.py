#!/usr/bin/env python3
"""Benchmark of the per-token hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload decode_attn|gemm|all]

Prints ONE JSON line.  A "step" is one pass of the hot-path kernel over one batch of
synthetic input that is already resident in HBM.  The default workload is the paged
decode attention microbench of BASELINE.json configs[1]:

    B=64, Hq=32, Hkv=8, Dh=128, block_size=256, ctx ~ U[512, 4096], seed 0,
    2048-block pool, block tables = prefix of randperm(2048), K/V rows N(0,1) bf16
    written through the KV-store kernel, softmax scale 1/sqrt(128).

``roofline`` is measured live with HIP events on the launch stream: algorithmic bytes per
launch (sum_b ctx_b * Hkv*Dh*2(K,V)*2 B + q and out + tables) over the mean launch time,
against the 8 TB/s HBM peak.  ``cpu_baseline`` times the CPU oracle (this repo's
restatement of the reference op; the checker, never the product) on a bounded sample of
the same workload on the host cores of the box.
"""
from __future__ import annotations

import argparse
import json
import math
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0
MFMA_BF16_PEAK_TFLOPS = 2500.0


def parse():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=30)
    ap.add_argument("--workload", default="decode_attn", choices=["decode_attn", "gemm", "all"])
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--batch", type=int, default=64)
    return ap.parse_args()


# ----------------------------------------------------------------------------- config 2
def make_decode_case(batch=64, hq=32, hkv=8, dh=128, bs=256, pool=2048, seed=0, device="cuda"):
    import torch
    from tinyllmforge_amd import ops as P
    g = torch.Generator().manual_seed(seed)
    ctx = torch.randint(512, 4097, (batch,), generator=g)
    nblk = ((ctx + bs - 1) // bs)
    perm = torch.randperm(pool, generator=g)
    maxb = 4096 // bs
    bt = torch.full((batch, maxb), -1, dtype=torch.int32)
    off = 0
    for b in range(batch):
        n = int(nblk[b])
        bt[b, :n] = perm[off:off + n].to(torch.int32)
        off += n
    # slot of token t of sequence b = bt[b, t // bs] * bs + t % bs
    slots = torch.cat([bt[b, (torch.arange(int(ctx[b])) // bs)].long() * bs + torch.arange(int(ctx[b])) % bs
                       for b in range(batch)]).to(torch.int32)
    total = int(ctx.sum())
    dev = torch.device(device)
    torch.manual_seed(seed)
    k_cache = torch.zeros(pool, bs, hkv, dh, dtype=torch.bfloat16, device=dev)
    v_cache = torch.zeros(pool, bs, hkv, dh, dtype=torch.bfloat16, device=dev)
    slots_d = slots.to(dev)
    chunk = 32768
    for s in range(0, total, chunk):                       # K/V rows go in through the store kernel
        n = min(chunk, total - s)
        kv = torch.randn(n, 2 * hkv * dh, device=dev, dtype=torch.float32).to(torch.bfloat16)
        P.store_kvcache(kv[:, :hkv * dh].view(n, hkv, dh), kv[:, hkv * dh:].view(n, hkv, dh),
                        k_cache, v_cache, slots_d[s:s + n])
    q = torch.randn(batch, hq, dh, device=dev, dtype=torch.float32).to(torch.bfloat16)
    algo_bytes = total * hkv * dh * 2 * 2 + 2 * batch * hq * dh * 2 + batch * (maxb + 1) * 4
    return dict(q=q, k_cache=k_cache, v_cache=v_cache, ctx=ctx.to(torch.int32).to(dev), bt=bt.to(dev),
                scale=1.0 / math.sqrt(dh), algo_bytes=algo_bytes, total_tokens=total,
                ctx_cpu=ctx, bt_cpu=bt)


def time_launches(fn, steps, warmup):
    """Per-launch GPU time (ms) from HIP events on the current stream, plus wall time of the region."""
    import torch
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    starts = [torch.cuda.Event(enable_timing=True) for _ in range(steps)]
    ends = [torch.cuda.Event(enable_timing=True) for _ in range(steps)]
    t0 = time.perf_counter()
    for i in range(steps):
        starts[i].record()
        fn()
        ends[i].record()
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    per = sorted(s.elapsed_time(e) for s, e in zip(starts, ends))
    span = starts[0].elapsed_time(ends[-1])
    return dict(mean_ms=sum(per) / len(per), median_ms=per[len(per) // 2], min_ms=per[0],
                span_ms=span, wall_s=wall)


def time_graph(fn, launches=20, replays=20):
    """Mean GPU time (ms) of one call of ``fn`` when ``launches`` calls are captured into a hipGraph and
    replayed: short kernels are timed back to back, without the host's per-call launch cost."""
    import torch
    fn()
    torch.cuda.synchronize()
    g = torch.cuda.CUDAGraph()
    s = torch.cuda.Stream()
    s.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(s):
        fn()
        with torch.cuda.graph(g, stream=s):
            for _ in range(launches):
                fn()
    torch.cuda.synchronize()
    g.replay()
    torch.cuda.synchronize()
    a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    a.record()
    for _ in range(replays):
        g.replay()
    b.record()
    torch.cuda.synchronize()
    return a.elapsed_time(b) / (launches * replays)


def bench_probes(args):
    """Rate of a plain read-only and a plain copy kernel over 1 GiB: the practical HBM ceiling of the box."""
    import torch
    from tinyllmforge_amd import _lib
    lib = _lib.load()
    n = 1 << 30
    src = torch.empty(n, dtype=torch.uint8, device="cuda").random_(0, 255)
    dst = torch.empty(n, dtype=torch.uint8, device="cuda")
    sink = torch.zeros(1, dtype=torch.int32, device="cuda")
    st = torch.cuda.current_stream().cuda_stream
    tr = time_launches(lambda: _lib.check(lib.tlf_probe_read(src.data_ptr(), n, sink.data_ptr(), st), "probe"), 30, 5)
    tc = time_launches(lambda: _lib.check(lib.tlf_probe_copy(src.data_ptr(), dst.data_ptr(), n, st), "probe"), 30, 5)
    return dict(read_GBps=round(n / (tr["mean_ms"] * 1e-3) / 1e9, 1),
                copy_GBps=round(2 * n / (tc["mean_ms"] * 1e-3) / 1e9, 1), bytes=n)


def bench_decode_attn(args):
    import torch
    from tinyllmforge_amd import ops as P
    case = make_decode_case(batch=args.batch)

    def step():
        return P.paged_decode_attention(case["q"], case["k_cache"], case["v_cache"], case["ctx"], case["bt"],
                                        case["scale"])

    t = time_launches(step, args.steps, args.warmup)
    # "step" time = back-to-back launches over the timed region (what a decode loop sees)
    ms_per_step = t["span_ms"] / args.steps
    gbps = case["algo_bytes"] / (ms_per_step * 1e-3) / 1e9
    kern_gbps = case["algo_bytes"] / (t["mean_ms"] * 1e-3) / 1e9
    res = dict(ms_per_step=ms_per_step, value=gbps,
               roofline=dict(bound="hbm", achieved=round(kern_gbps, 1), peak=HBM_PEAK_GBPS, unit="GB/s",
                             frac=round(kern_gbps / HBM_PEAK_GBPS, 4), traffic=None,
                             kernel="paged_decode_kernel<8,false> + paged_decode_merge_kernel",
                             launch_ms_mean=round(t["mean_ms"], 5), launch_ms_median=round(t["median_ms"], 5),
                             launch_ms_min=round(t["min_ms"], 5), algorithmic_bytes=case["algo_bytes"]),
               case=case)
    return res


def cpu_baseline_decode(case, budget_s=20.0):
    """CPU oracle on the first sequences of the same batch until ~budget_s of CPU work."""
    import torch
    from oracle import ops as O
    q = case["q"].cpu()
    ctx, bt = case["ctx_cpu"].to(torch.int32), case["bt_cpu"]
    # gather only the blocks the sample needs (the pool is 2 GiB; copy block by block)
    nseq, nbytes, spent = 0, 0, 0.0
    hkv, dh = case["k_cache"].shape[2], case["k_cache"].shape[3]
    while nseq < q.shape[0] and spent < budget_s:
        b = nseq
        nb = (int(ctx[b]) + 255) // 256
        ids = bt[b, :nb].long()
        kc = case["k_cache"][ids.to(case["k_cache"].device)].cpu()
        vc = case["v_cache"][ids.to(case["k_cache"].device)].cpu()
        local_bt = torch.arange(nb, dtype=torch.int32).view(1, -1)
        t0 = time.perf_counter()
        O.paged_decode_attention(q[b:b + 1], kc, vc, ctx[b:b + 1], local_bt, case["scale"])
        spent += time.perf_counter() - t0
        nbytes += int(ctx[b]) * hkv * dh * 2 * 2
        nseq += 1
    return dict(value=round(nbytes / spent / 1e9, 3), unit="GB/s", cores=torch.get_num_threads(), kind="port",
                sample=f"first {nseq} of {q.shape[0]} sequences of the same batch "
                       f"({nbytes / 1e6:.0f} MB of K/V rows), {spent:.1f} s of CPU oracle time")


# ----------------------------------------------------------------------------- config 3
GEMM_SHAPES = {"qkv": (6144, 4096), "o_proj": (4096, 4096), "gate_up": (24576, 4096), "down": (4096, 12288)}


def bench_gemm(args, ms=(1, 16, 64, 256, 2048)):
    import torch
    from tinyllmforge_amd import ops as P
    torch.manual_seed(0)
    rows = []
    for name, (N, K) in GEMM_SHAPES.items():
        wq = torch.randint(-127, 128, (N, K), device="cuda", dtype=torch.int8)
        scale = torch.rand(N, device="cuda") * 9e-3 + 1e-3
        for M in ms:
            x = torch.randn(M, K, device="cuda").to(torch.bfloat16)
            sec = time_graph(lambda: P.w8a16_linear(x, wq, scale)) * 1e-3
            nbytes = N * K + 4 * N + 2 * M * K + 2 * M * N
            flops = 2.0 * M * N * K
            bound = "hbm" if M <= 64 else "mfma"
            rows.append(dict(shape=name, M=M, N=N, K=K, us=round(sec * 1e6, 2), GBps=round(nbytes / sec / 1e9, 1),
                             TFLOPs=round(flops / sec / 1e12, 1), bound=bound,
                             frac=round((nbytes / sec / 1e9 / HBM_PEAK_GBPS) if bound == "hbm"
                                        else (flops / sec / 1e12 / MFMA_BF16_PEAK_TFLOPS), 4)))
    return rows


def main():
    args = parse()
    if args.gpus != 1:
        print("bench.py measures one GPU: this build has no multi-GPU path (run with --gpus 1)", file=sys.stderr)
        sys.exit(2)
    import torch
    if not torch.cuda.is_available():
        print("bench.py needs a GPU (the HIP path has no CPU fallback)", file=sys.stderr)
        sys.exit(1)
    torch.cuda.set_device(0)
    out = {}
    extra = {}
    res = bench_decode_attn(args)
    extra["hbm_probe"] = bench_probes(args)
    if args.workload in ("gemm", "all"):
        extra["w8a16_gemm"] = bench_gemm(args)
    cpu = None
    if not args.no_cpu_baseline:
        cpu = cpu_baseline_decode(res["case"])
    out = {
        "metric": "paged-decode HBM GB/s vs peak",
        "value": round(res["value"], 1),
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(res["ms_per_step"], 5),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16",
        "data": "synthetic",
        "config": {"workload": "BASELINE.json configs[1]: paged decode attention microbench, B=%d Hq=32 Hkv=8 Dh=128 "
                               "block_size=256 ctx~U[512,4096] pool=2048 blocks" % args.batch,
                   "total_context_tokens": res["case"]["total_tokens"]},
        "roofline": res["roofline"],
        "cpu_baseline": cpu,
    }
    if extra:
        out["extra"] = extra
    print(json.dumps(out))


if __name__ == "__main__":
    main()
