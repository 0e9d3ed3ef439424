#!/usr/bin/env python3
"""Benchmark of the per-token hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload e2e|decode_attn|gemm|all]

Prints ONE JSON line.

``value`` (default workload ``e2e``) is BASELINE.json's headline metric: output tokens/s of a
Qwen3-8B-shaped decoder (36 layers, hidden 4096, 32 query / 8 KV heads, head_dim 128,
intermediate 12288, vocab 151936; random-init weights, W8A16 linears; the bf16 run is reported
beside it) on the reference's own bench.py recipe (tinyvllm bench.py:39-59): ``seed(0)``, 256
prompts of ``randint(100, 1024)`` random token ids, ``max_tokens = randint(100, 1024)``,
``ignore_eos``, continuous batching, hipGraph-captured decode, one warm-up ``generate`` first;
tok/s = sum(max_tokens) / wall time of ``generate()``, prefill included.  Greedy sampling
(temperature 0; the reference's script uses 0.6, timed as a second leg) keeps the run
deterministic.  A "step" is one engine step (one prefill or one decode pass over the running
batch).  ``value`` is always the whole job; ``--steps K`` only chooses what ``steps`` and
``ms_per_step`` describe: the first K engine steps of that same timed run (0 = all of them).

``roofline`` is the paged decode attention kernel, the largest single consumer of a decode step,
measured live with HIP events on its launch stream on BASELINE.json configs[1]
(B=64, Hq=32, Hkv=8, Dh=128, block 256, ctx ~ U[512, 4096], 2048-block pool, seed 0):
algorithmic bytes per launch (sum_b ctx_b * Hkv*Dh*2(K,V)*2 B + q and out + tables) over the
mean launch time, against the 8 TB/s HBM peak.

``cpu_baseline`` times the CPU oracle (this repo's restatement of the reference's PyTorch layer
semantics; the checker, never the product) on a bounded sample of the same workload on the box's
host cores.
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
# HBM bytes per decode-attention launch on the default configs[1] workload, from two rocprofv3 --pmc runs
# (FETCH_SIZE x 2.0 and WRITE_SIZE x 1.0 KiB per dispatch, factors taken from the 1 GiB copy probe), main + merge kernel
DECODE_ATTN_TRAFFIC_BYTES = int((313290.1 + 2605.8) * 2.0 * 1024 + (5088.1 + 512.0) * 1024)
MFMA_BF16_PEAK_TFLOPS = 2500.0


def parse():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=0,
                    help="engine steps that steps/ms_per_step describe (0 = all); value is always the whole job")
    ap.add_argument("--warmup", type=int, default=1, help="warm-up generate() calls before the timed run")
    ap.add_argument("--workload", default="e2e",
                    choices=["e2e", "decode_attn", "gemm", "prefill_attn", "elementwise", "clock", "c5", "all"])
    ap.add_argument("--attn-steps", type=int, default=200, help="timed launches of the decode-attention microbench")
    ap.add_argument("--num-seqs", type=int, default=256)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--batch", type=int, default=64)
    ap.add_argument("--fp8", action="store_true", help="decode_attn: e4m3 cache rows (BASELINE.json configs[4]'s attention)")
    ap.add_argument("--hq", type=int, default=32, help="decode_attn: query heads (8 KV heads)")
    ap.add_argument("--gemm-shapes", default="8b", choices=["8b", "32b", "0.6b", "all"],
                    help="gemm: projection shapes of which model (configs[2] is 8b)")
    ap.add_argument("--gemm-m", default="", help="gemm: comma-separated token counts instead of the default list")
    ap.add_argument("--skip-bf16", action="store_true", help="e2e: skip the second run with bf16 linears (profiling)")
    ap.add_argument("--skip-c5", action="store_true", help="e2e: skip the Qwen3-32B-shape run (configs[4])")
    ap.add_argument("--skip-gemm", action="store_true", help="e2e: skip the W8A16 GEMM table (configs[2])")
    return ap.parse_args()


# ----------------------------------------------------------------------------- config 2
def make_decode_case(batch=64, hq=32, hkv=8, dh=128, bs=256, pool=2048, seed=0, device="cuda", fp8=False):
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
    cache_dtype = torch.float8_e4m3fn if fp8 else torch.bfloat16
    k_cache = torch.zeros(pool, bs, hkv, dh, dtype=cache_dtype, device=dev)
    v_cache = torch.zeros(pool, bs, hkv, dh, dtype=cache_dtype, device=dev)
    scales = dict(k_scale=torch.full((hkv,), 0.02, device=dev), v_scale=torch.full((hkv,), 0.02, device=dev)) if fp8 else {}
    slots_d = slots.to(dev)
    chunk = 32768
    for s in range(0, total, chunk):                       # K/V rows go in through the store kernel
        n = min(chunk, total - s)
        kv = torch.randn(n, 2 * hkv * dh, device=dev, dtype=torch.float32).to(torch.bfloat16)
        P.store_kvcache(kv[:, :hkv * dh].view(n, hkv, dh), kv[:, hkv * dh:].view(n, hkv, dh),
                        k_cache, v_cache, slots_d[s:s + n], **scales)
    q = torch.randn(batch, hq, dh, device=dev, dtype=torch.float32).to(torch.bfloat16)
    algo_bytes = total * hkv * dh * 2 * (1 if fp8 else 2) + 2 * batch * hq * dh * 2 + batch * (maxb + 1) * 4
    return dict(q=q, k_cache=k_cache, v_cache=v_cache, ctx=ctx.to(torch.int32).to(dev), bt=bt.to(dev),
                scale=1.0 / math.sqrt(dh), algo_bytes=algo_bytes, total_tokens=total,
                ctx_cpu=ctx, bt_cpu=bt, scales=scales)


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
    res = dict(read_GBps=round(n / (tr["mean_ms"] * 1e-3) / 1e9, 1),
               copy_GBps=round(2 * n / (tc["mean_ms"] * 1e-3) / 1e9, 1), bytes=n)
    # what the matrix cores sustain from registers, on small-integer and on random operands
    out = torch.empty(512 * 256, dtype=torch.float32, device="cuda")
    iters = 4000
    flop = 2.0 * 32 * 32 * 16 * 16 * iters * 2048
    mf = {}
    for mode, name in ((0, "small_int_TFLOPs"), (1, "random_TFLOPs")):
        t = time_launches(lambda: _lib.check(lib.tlf_probe_mfma(out.data_ptr(), iters, mode, st), "probe"), 5, 2)
        mf[name] = round(flop / (t["mean_ms"] * 1e-3) / 1e12, 1)
    mf["note"] = "register-only v_mfma_f32_32x32x16_bf16 stream, two waves per SIMD: the clock drops on random data"
    res["mfma_probe"] = mf
    # an HBM stream and an L2-resident stream through the same CUs at once: the launch takes the sum of the two
    small = src[:1 << 20]
    def mix(big_bytes, eighths):
        t = time_launches(lambda: _lib.check(lib.tlf_probe_mix(src.data_ptr(), big_bytes, small.data_ptr(), 1 << 20, eighths,
                                                               sink.data_ptr(), st), "probe"), 10, 3)
        return t["mean_ms"] * 1e3
    hbm_alone = mix(n, 0)
    both = mix(n, 22)                               # 2.75 KiB out of L2 per KiB from HBM: a GEMM at 128 tokens
    l2_alone = mix(16 << 20, 22 * 64)               # the same L2 bytes beside a negligible HBM part
    res["mixed_traffic_probe"] = dict(hbm_1GiB_alone_us=round(hbm_alone, 1), l2_2p75GiB_alone_us=round(l2_alone, 1),
                                      both_at_once_us=round(both, 1), sum_us=round(hbm_alone + l2_alone, 1),
                                      note="4 waves per CU stream from HBM, 4 re-read 1 MiB out of L2; loads return in "
                                           "order through a CU's L1, so the two do not overlap")
    return res


def bench_clock(args, seconds=2.0):
    """The shader clock the part holds under each load, read from ``rocm-smi --showclocks`` (a child process polled
    from a thread) while the load runs back to back: the register-only MFMA stream on small integers and on random
    operands, the W8A16 GEMM of the gate_up projection at 8192 tokens on random and on small-integer data, and the
    paged decode attention microbench.  The matrix-core peak scales with that clock (2.5 PFLOP/s is at 2.4 GHz)."""
    import re
    import shutil
    import subprocess
    import threading
    import torch
    from tinyllmforge_amd import _lib, ops as P
    smi = shutil.which("rocm-smi") or "/opt/rocm/bin/rocm-smi"
    if not os.path.exists(smi):
        return {"skipped": "rocm-smi not found"}
    lib = _lib.load()
    st = torch.cuda.current_stream().cuda_stream

    def read_sclk():
        try:
            r = subprocess.run([smi, "--showclocks"], capture_output=True, text=True, timeout=10)
        except Exception:
            return None
        for line in r.stdout.splitlines():
            if "sclk" in line:
                m = re.search(r"\((\d+)Mhz\)", line)
                if m:
                    return int(m.group(1))
        return None

    def under_load(fn, work_per_call):
        stop, seen = threading.Event(), []

        def poll():
            while not stop.is_set():
                v = read_sclk()
                if v is not None:
                    seen.append(v)
        fn()
        torch.cuda.synchronize()
        th = threading.Thread(target=poll)
        th.start()
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        t0, calls, gpu_ms = time.perf_counter(), 0, 0.0
        while time.perf_counter() - t0 < seconds:
            a.record()
            for _ in range(10):
                fn()
            b.record()
            torch.cuda.synchronize()
            gpu_ms += a.elapsed_time(b)
            calls += 10
        stop.set()
        th.join()
        body = seen[1:] or seen            # the first reading may predate the load
        mhz = sorted(body)[len(body) // 2] if body else None
        return mhz, work_per_call * calls / (gpu_ms * 1e-3)

    out = {"idle_sclk_MHz": read_sclk(), "loads": []}
    buf = torch.empty(512 * 256, dtype=torch.float32, device="cuda")
    iters = 4000
    flop = 2.0 * 32 * 32 * 16 * 16 * iters * 2048
    for mode, name in ((0, "mfma stream, small integers"), (1, "mfma stream, random operands"),
                       (3, "mfma stream, random operands, idle cycles after every MFMA")):
        mhz, rate = under_load(lambda: _lib.check(lib.tlf_probe_mfma(buf.data_ptr(), iters, mode, st), "probe"), flop)
        out["loads"].append(dict(load=name, sclk_MHz=mhz, TFLOPs=round(rate / 1e12, 1)))
    N, K, M = 24576, 4096, 8192
    g = torch.Generator(device="cuda").manual_seed(0)
    sc = torch.rand(N, device="cuda", generator=g) * 0.01
    for name, lo, hi, xs in (("W8A16 GEMM gate_up 8192 tokens, random data", -127, 128, None),
                             ("W8A16 GEMM gate_up 8192 tokens, small integers", -2, 3, 2)):
        w = P.pack_w8(torch.randint(lo, hi, (N, K), dtype=torch.int8, device="cuda", generator=g))
        x = (torch.randn(M, K, device="cuda", generator=g) if xs is None else
             torch.randint(-xs, xs + 1, (M, K), device="cuda", generator=g).float()).to(torch.bfloat16)
        mhz, rate = under_load(lambda: P.w8a16_linear(x, w, sc), 2.0 * M * N * K)
        out["loads"].append(dict(load=name, sclk_MHz=mhz, TFLOPs=round(rate / 1e12, 1)))
        del w, x
    case = make_decode_case(batch=args.batch)
    mhz, rate = under_load(lambda: P.paged_decode_attention(case["q"], case["k_cache"], case["v_cache"], case["ctx"], case["bt"],
                                                            case["scale"], **case["scales"]), case["algo_bytes"])
    out["loads"].append(dict(load="paged decode attention, configs[1]", sclk_MHz=mhz, GBps=round(rate / 1e9, 1)))
    for r in out["loads"]:
        if r.get("TFLOPs") and r["sclk_MHz"]:
            # share of what the matrix cores could do at the clock the part held
            r["of_peak_at_that_clock"] = round(r["TFLOPs"] / (MFMA_BF16_PEAK_TFLOPS * r["sclk_MHz"] / 2400.0), 3)
    return out


def bench_decode_attn(args, fp8=False, hq=32):
    import torch
    from tinyllmforge_amd import ops as P
    case = make_decode_case(batch=args.batch, fp8=fp8, hq=hq)

    def step():
        return P.paged_decode_attention(case["q"], case["k_cache"], case["v_cache"], case["ctx"], case["bt"],
                                        case["scale"], **case["scales"])

    t = time_launches(step, args.attn_steps, 30)
    # the same call as the engine issues it: the work split made once per decode step for all layers
    plan = P.paged_decode_plan(case["ctx"], case["bt"], case["k_cache"].shape[1])
    tp = time_launches(lambda: P.paged_decode_attention(case["q"], case["k_cache"], case["v_cache"], case["ctx"], case["bt"],
                                                        case["scale"], plan=plan, **case["scales"]), args.attn_steps, 30)
    tk = time_launches(lambda: P.paged_decode_plan(case["ctx"], case["bt"], case["k_cache"].shape[1], out=plan), 50, 10)
    planned = dict(launch_ms_mean=round(tp["mean_ms"], 5), launch_ms_median=round(tp["median_ms"], 5),
                   GBps=round(case["algo_bytes"] / (tp["mean_ms"] * 1e-3) / 1e9, 1),
                   frac=round(case["algo_bytes"] / (tp["mean_ms"] * 1e-3) / 1e9 / HBM_PEAK_GBPS, 4),
                   plan_kernel_us=round(tk["mean_ms"] * 1e3, 2),
                   note="tlf_paged_decode_attn_planned; the plan kernel runs once per decode step (36 layers here share it) "
                        "and is not part of this launch; roofline above is the self-contained call")
    # "step" time = back-to-back launches over the timed region (what a decode loop sees)
    ms_per_step = t["span_ms"] / args.attn_steps
    gbps = case["algo_bytes"] / (ms_per_step * 1e-3) / 1e9
    kern_gbps = case["algo_bytes"] / (t["mean_ms"] * 1e-3) / 1e9
    res = dict(ms_per_step=ms_per_step, value=gbps,
               roofline=dict(bound="hbm", achieved=round(kern_gbps, 1), peak=HBM_PEAK_GBPS, unit="GB/s",
                             frac=round(kern_gbps / HBM_PEAK_GBPS, 4),
                             traffic=DECODE_ATTN_TRAFFIC_BYTES if args.batch == 64 and not fp8 and hq == 32 else None,
                             kernel="paged_decode_kernel<8,%s> + paged_decode_merge_kernel" % ("true" if fp8 else "false"),
                             launch_ms_mean=round(t["mean_ms"], 5), launch_ms_median=round(t["median_ms"], 5),
                             launch_ms_min=round(t["min_ms"], 5), algorithmic_bytes=case["algo_bytes"]),
               planned=planned, case=case)
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
GEMM_SHAPES_32B = {"qkv_32b": (10240, 5120), "o_proj_32b": (5120, 8192), "gate_up_32b": (51200, 5120),
                   "down_32b": (5120, 25600)}
GEMM_SHAPES_06B = {"qkv_0.6b": (4096, 1024), "o_proj_0.6b": (1024, 2048), "gate_up_0.6b": (6144, 1024),
                   "down_0.6b": (1024, 3072)}


def bench_gemm(args, ms=(1, 16, 64, 128, 256, 2048, 8192), shapes=None):
    """W8A16 GEMM table.  Up to M = 256 a decode step finds its weights in HBM (a layer's weights were last
    touched one whole step ago), so those cells cycle through enough copies of the weight to exceed the
    256 MB Infinity Cache several times ("cold"); the same call on one resident copy is reported beside it
    ("warm").  Larger M is compute bound and timed on one copy."""
    import torch
    from tinyllmforge_amd import ops as P
    torch.manual_seed(0)
    import ctypes
    from tinyllmforge_amd import _lib
    lib = _lib.load()
    rows = []
    if getattr(args, "gemm_m", ""):
        ms = tuple(int(a) for a in args.gemm_m.split(","))
    for name, (N, K) in (shapes or GEMM_SHAPES).items():
        copies = max(2, -(-(768 << 20) // (N * K)))
        wqs = [P.pack_w8(torch.randint(-127, 128, (N, K), device="cuda", dtype=torch.int8)) for _ in range(copies)]
        scale = torch.rand(N, device="cuda") * 9e-3 + 1e-3
        for M in ms:
            x = torch.randn(M, K, device="cuda").to(torch.bfloat16)
            warm = time_graph(lambda: P.w8a16_linear(x, wqs[0], scale)) * 1e-3
            sec = warm
            if M <= 256:
                def cycle():
                    for w in wqs:
                        P.w8a16_linear(x, w, scale)
                sec = time_graph(cycle, launches=2, replays=10) * 1e-3 / copies
            nbytes = N * K + 4 * N + 2 * M * K + 2 * M * N
            flops = 2.0 * M * N * K
            bound = "hbm" if M <= 128 else "mfma"
            plan = (ctypes.c_int32 * 8)()
            lib.tlf_gemm_plan(M, N, K, 1, plan)
            rows.append(dict(shape=name, M=M, N=N, K=K, plan=list(plan)[:6],
                             us=round(sec * 1e6, 2), weights="cold" if M <= 256 else "warm",
                             us_warm=round(warm * 1e6, 2), GBps=round(nbytes / sec / 1e9, 1),
                             TFLOPs=round(flops / sec / 1e12, 1), bound=bound,
                             frac=round((nbytes / sec / 1e9 / HBM_PEAK_GBPS) if bound == "hbm"
                                        else (flops / sec / 1e12 / MFMA_BF16_PEAK_TFLOPS), 4)))
        del wqs
        torch.cuda.empty_cache()
    return rows


def cpu_baseline_gemm(budget_s=20.0):
    """CPU oracle (``oracle.ops.w8a16_linear``: fp64 contraction of bf16 activations with int8 weights, scale,
    one rounding) on the qkv projection shape at M = 256, then 2048 while the budget lasts."""
    import torch
    from oracle import ops as O
    torch.manual_seed(0)
    N, K = GEMM_SHAPES["qkv"]
    wq = torch.randint(-127, 128, (N, K), dtype=torch.int8)
    scale = torch.rand(N) * 9e-3 + 1e-3
    flops, spent, done = 0.0, 0.0, []
    for M in (256, 2048):
        x = torch.randn(M, K).to(torch.bfloat16)
        O.w8a16_linear(x[:16], wq, scale)                     # warm-up
        for _ in range(3):
            if spent >= budget_s:
                break
            t0 = time.perf_counter()
            O.w8a16_linear(x, wq, scale)
            spent += time.perf_counter() - t0
            flops += 2.0 * M * N * K
            done.append(M)
    return dict(value=round(flops / spent / 1e12, 4), unit="TFLOP/s", cores=torch.get_num_threads(), kind="port",
                sample=f"qkv projection (N={N}, K={K}) at M = {sorted(set(done))}, {len(done)} calls, "
                       f"{spent:.1f} s of CPU oracle time")


# ----------------------------------------------------------------------------- elementwise kernels
def bench_elementwise(args, sizes=(16384, 256)):
    """The single-pass kernels at the 8B widths (hidden 4096, 32 / 8 heads of 128, intermediate 12288, vocabulary
    151,936) at a prefill step's size (16,384 tokens) and a decode step's (256): algorithmic bytes (every input
    element read once, every output element written once) over the hipGraph-timed launch, against 8 TB/s.
    At 16,384 tokens each kernel cycles through enough independent copies of its tensors to exceed the 256 MB
    Infinity Cache ("cold"); at 256 tokens the tensors are a few MB and sit in L2, as they do between two kernels
    of a decode step ("warm": these cells measure launch and latency, not bandwidth)."""
    import torch
    from tinyllmforge_amd import ops as P
    from tinyllmforge_amd.layers.rotary_embedding import build_cos_sin_cache
    torch.manual_seed(0)
    BF, dev = torch.bfloat16, "cuda"
    H, Hq, Hkv, Dh, I, V = 4096, 32, 8, 128, 12288, 151936
    QKV = (Hq + 2 * Hkv) * Dh
    tab = build_cos_sin_cache(Dh, 40960, 1e6).to(dev)
    w_h = torch.ones(H, dtype=BF, device=dev)
    w_d = torch.ones(Dh, dtype=BF, device=dev)
    emb = (torch.randn(V, H, device=dev) * 0.02).to(BF)
    rows = []

    def timed(name, n, nbytes, per_copy_bytes, make, cold=None):
        cold = n > 1024 if cold is None else cold
        copies = max(2, -(-(768 << 20) // max(1, per_copy_bytes))) if cold else 1
        calls = [make() for _ in range(copies)]

        def cycle():
            for c in calls:
                c()
        sec = time_graph(cycle, launches=40 if copies == 1 else 2, replays=10) * 1e-3 / copies
        gbps = nbytes / sec / 1e9
        rows.append(dict(kernel=name, tokens=n, us=round(sec * 1e6, 2), algorithmic_MB=round(nbytes / 1e6, 2),
                         GBps=round(gbps, 1), frac=round(gbps / HBM_PEAK_GBPS, 4), data="cold" if copies > 1 else "warm"))
        del calls
        torch.cuda.empty_cache()

    def slots_of(n, nblk):
        """Cache slots as the engine hands them out: a prefill step's tokens fill whole 256-token blocks in
        order, the blocks lie anywhere in the pool; a decode step's tokens are one per sequence, anywhere."""
        if n <= 1024:
            return torch.randperm(nblk * 256, device=dev)[:n].to(torch.int32)
        blocks = torch.randperm(nblk, device=dev)
        t = torch.arange(n, device=dev)
        return (blocks[t // 256] * 256 + t % 256).to(torch.int32)

    for n in sizes:
        nblk = -(-n // 256) + 1 if n > 1024 else 2048

        def mk_store():
            qkv = torch.randn(n, QKV, device=dev).to(BF)
            key = torch.randn(n, Hkv, Dh, device=dev).to(BF)
            val = qkv[:, (Hq + Hkv) * Dh:].view(n, Hkv, Dh)          # a view into the projection, as the model passes it
            kc = torch.zeros(nblk, 256, Hkv, Dh, dtype=BF, device=dev)
            vc = torch.zeros_like(kc)
            slots = slots_of(n, nblk)
            return lambda: P.store_kvcache(key, val, kc, vc, slots)
        timed("store_kvcache", n, n * (4 * Hkv * Dh * 2 + 4), n * (QKV * 2 + 3 * Hkv * Dh * 2), mk_store)

        def mk_rms():
            x = torch.randn(n, H, device=dev).to(BF)
            return lambda: P.rms_norm(x, w_h, 1e-6)
        timed("rmsnorm", n, n * H * 4, n * H * 4, mk_rms)

        def mk_add_rms():
            x = torch.randn(n, H, device=dev).to(BF)
            r = torch.randn(n, H, device=dev).to(BF)
            return lambda: P.add_rms_norm(x, r, w_h, 1e-6)
        timed("add_rmsnorm", n, n * H * 8, n * H * 8, mk_add_rms)

        def mk_rope():
            q = torch.randn(n, Hq * Dh, device=dev).to(BF)
            k = torch.randn(n, Hkv * Dh, device=dev).to(BF)
            pos = torch.randint(0, 4096, (n,), device=dev)
            return lambda: P.rope(pos, q, k, tab, Dh)
        timed("rope", n, n * ((Hq + Hkv) * Dh * 4 + 8 + Dh * 4), n * (Hq + Hkv) * Dh * 4, mk_rope)

        def mk_fused():
            qkv = torch.randn(n, QKV, device=dev).to(BF)
            pos = torch.randint(0, 4096, (n,), device=dev)
            kc = torch.zeros(nblk, 256, Hkv, Dh, dtype=BF, device=dev)
            vc = torch.zeros_like(kc)
            slots = slots_of(n, nblk)
            return lambda: P.qknorm_rope_store(qkv, w_d, w_d, 1e-6, pos, tab, Hq, Hkv, Dh, kc, vc, slots)
        timed("qknorm_rope_store", n, n * (QKV * 2 + Hq * Dh * 2 + 2 * Hkv * Dh * 2 + 8 + Dh * 4 + 4),
              n * (QKV * 2 + Hq * Dh * 2 + 2 * Hkv * Dh * 2), mk_fused)

        def mk_silu():
            x = torch.randn(n, 2 * I, device=dev).to(BF)
            return lambda: P.silu_and_mul(x)
        timed("silu_and_mul", n, n * I * 6, n * I * 6, mk_silu)

        def mk_emb():
            ids = torch.randint(0, V, (n,), device=dev)
            return lambda: P.embedding(ids, emb)
        timed("embedding", n, n * (H * 4 + 8), n * H * 4, mk_emb)

    def mk_argmax():
        logits = torch.randn(256, V, device=dev).to(BF)
        return lambda: P.argmax(logits)
    # 78 MB of logits a copy: ten copies exceed the Infinity Cache three times
    timed("argmax (256 x 151936)", 256, 256 * V * 2 + 256 * 8, 256 * V * 2, mk_argmax, cold=True)
    return rows


# ----------------------------------------------------------------------------- prefill attention microbench
def bench_prefill_attn(args):
    """Varlen causal prefill attention at the 8B shape (32 / 8 heads, packed bf16 K/V) and the 32B shape
    (64 / 8 heads, paged e4m3 rows, optionally behind a cached prefix).  flops = 4 Hq Dh sum(len^2 / 2 +
    len * cached); frac against the dense bf16 MFMA peak."""
    import torch
    from tinyllmforge_amd import ops as P
    torch.manual_seed(0)
    dev, dh, bs = "cuda", 128, 256
    rows = []

    def run(name, lens, hq, hkv, fp8=False, cached=0):
        S = sum(lens)
        q = torch.randn(S, hq, dh, device=dev).to(torch.bfloat16)
        cu = torch.tensor([0] + list(torch.tensor(lens).cumsum(0)), dtype=torch.int32, device=dev)
        flops = sum(4.0 * hq * dh * (l * l / 2 + l * cached) for l in lens)
        if not fp8:
            k = torch.randn(S, hkv, dh, device=dev).to(torch.bfloat16)
            v = torch.randn(S, hkv, dh, device=dev).to(torch.bfloat16)
            f = lambda: P.varlen_prefill_attention(q, k, v, cu, cu, max(lens), 1 / math.sqrt(dh))
        else:
            klens = [l + cached for l in lens]
            nb = [(l + bs - 1) // bs for l in klens]
            kc = (torch.randn(sum(nb), bs, hkv, dh, device=dev) * 0.5).to(torch.float8_e4m3fn)
            vc = (torch.randn(sum(nb), bs, hkv, dh, device=dev) * 0.5).to(torch.float8_e4m3fn)
            bt = torch.full((len(lens), max(nb)), -1, dtype=torch.int32)
            o = 0
            for i, n in enumerate(nb):
                bt[i, :n] = torch.arange(o, o + n)
                o += n
            bt = bt.to(dev)
            cuk = torch.tensor([0] + list(torch.tensor(klens).cumsum(0)), dtype=torch.int32, device=dev)
            ksc, vsc = torch.full((hkv,), 0.02, device=dev), torch.full((hkv,), 0.02, device=dev)
            f = lambda: P.varlen_prefill_attention(q, kc, vc, cu, cuk, max(lens), 1 / math.sqrt(dh), block_tables=bt,
                                                   k_scale=ksc, v_scale=vsc)
        sec = time_graph(f, 5, 5) * 1e-3
        rows.append(dict(case=name, tokens=S, us=round(sec * 1e6, 1), TFLOPs=round(flops / sec / 1e12, 1),
                         frac=round(flops / sec / 1e12 / MFMA_BF16_PEAK_TFLOPS, 4)))

    run("8B shape, bf16 rows, 16 x 1024 tokens", [1024] * 16, 32, 8)
    run("8B shape, bf16 rows, 28 x 560 tokens", [560] * 28, 32, 8)
    run("8B shape, bf16 rows, 4 x 4096 tokens", [4096] * 4, 32, 8)
    run("32B shape, e4m3 rows (paged), 2 x 8192 tokens", [8192] * 2, 64, 8, fp8=True)
    run("32B shape, e4m3 rows (paged), 3 x 4096 tokens behind 1024 cached", [4096] * 3, 64, 8, fp8=True, cached=1024)
    return rows


# ----------------------------------------------------------------------------- config 5 (32B shape, fp8 KV, shared prefixes)
def bench_c5(args):
    """BASELINE.json configs[4]: Qwen3-32B-shaped decoder, W8A16 linears, e4m3 KV cache with per-head scales,
    32 sequences with prompts ~U[2048, 8192], half of them sharing a 1024-token prefix held in cached blocks
    (a first generate() of one prefix-only request fills those blocks), 256 greedy output tokens each."""
    import torch
    from random import randint, seed
    from tinyllmforge_amd import LLM, SamplingParams
    seed(0)
    shared = [randint(0, 10000) for _ in range(1024)]
    prompts = []
    for i in range(32):
        n = randint(2048, 8192)
        body = [randint(0, 10000) for _ in range(n)]
        prompts.append(shared + body[1024:] if i % 2 == 0 else body)
    llm = LLM("qwen3-32b", enforce_eager=False, max_model_len=8704, max_num_batched_tokens=16384, max_num_seqs=32,
              quantization="w8a16", kv_cache_dtype="fp8_e4m3", gpu_memory_utilization=0.6, seed=0)
    sp = SamplingParams(temperature=0.0, ignore_eos=True, max_tokens=256)
    llm.generate([shared + [1, 2, 3]], SamplingParams(temperature=0.0, max_tokens=2, ignore_eos=True))   # warm-up + prefix fill
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    llm.generate(prompts, sp)
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    st = llm.last_stats
    res = dict(tok_s=round(32 * 256 / wall, 1), wall_s=round(wall, 3), prompt_tokens=sum(len(p) for p in prompts),
               prefill_s=round(st["prefill_time"], 3), decode_s=round(st["decode_time"], 3),
               decode_ms_per_step=round(1e3 * st["decode_time"] / max(1, st["decode_steps"]), 3),
               prefill_steps=st["prefill_steps"], decode_steps=st["decode_steps"],
               cached_prompt_tokens=st["cached_prompt_tokens"],
               decode_byte_floor=decode_byte_floor(llm.config.hf_config, st, "w8a16", kv_itemsize=1),
               kv_blocks=llm.config.num_kvcache_blocks, kv_dtype="fp8_e4m3")
    sat = llm.model_runner.kv_saturation()                      # after the timed region
    res["kv_saturated_fraction"] = dict(k=round(sat["k_saturated"] / max(1, sat["entries"]), 8),
                                        v=round(sat["v_saturated"] / max(1, sat["entries"]), 8),
                                        k_worst=sat["k_worst"], v_worst=sat["v_worst"])
    llm.exit()
    return res


# ----------------------------------------------------------------------------- config 4 (end to end)
def e2e_workload(num_seqs=256):
    """The reference's bench.py recipe (pure-python ``random``: platform independent)."""
    from random import randint, seed
    seed(0)
    prompts = [[randint(0, 10000) for _ in range(randint(100, 1024))] for _ in range(num_seqs)]
    max_tokens = [randint(100, 1024) for _ in range(num_seqs)]
    return prompts, max_tokens


def timed_generate(llm, prompts, sps, mark_steps=0):
    """The engine's generate() loop (tinyvllm llm_engine.py:64-101) with its per-step statistics, plus the
    wall time at which the first ``mark_steps`` engine steps were done.  Returns (stats, wall_s, wall_at_mark)."""
    import torch
    for p, sp in zip(prompts, sps):
        llm.add_request(p, sp)
    st = dict(prefill_steps=0, decode_steps=0, prefill_time=0.0, decode_time=0.0, cached_prompt_tokens=0,
              decode_context_tokens=0)
    steps, at_mark = 0, None
    torch.cuda.synchronize()
    t_begin = time.perf_counter()
    while not llm.is_finished():
        t0 = time.perf_counter()
        _, num_tokens = llm.step()            # ends in the step's device -> host copy of the token ids
        dt = time.perf_counter() - t0
        kind = "prefill" if num_tokens > 0 else "decode"
        st[kind + "_steps"] += 1
        st[kind + "_time"] += dt
        st["cached_prompt_tokens"] += llm._step_info[0]
        st["decode_context_tokens"] += llm._step_info[1]
        steps += 1
        if steps == mark_steps:
            at_mark = time.perf_counter() - t_begin
    torch.cuda.synchronize()
    wall = time.perf_counter() - t_begin
    return st, wall, at_mark


def bench_e2e(args, quantization):
    import torch
    from tinyllmforge_amd import LLM, SamplingParams
    prompts, max_tokens = e2e_workload(args.num_seqs)
    t0 = time.perf_counter()
    llm = LLM("qwen3-8b", enforce_eager=False, max_model_len=4096, quantization=quantization,
              gpu_memory_utilization=0.6, seed=0)
    init_s = time.perf_counter() - t0
    sps = [SamplingParams(temperature=0.0, ignore_eos=True, max_tokens=m) for m in max_tokens]
    for _ in range(max(1, args.warmup)):
        llm.generate([[1, 2, 3, 4, 5, 6, 7, 8]], SamplingParams(temperature=0.0, max_tokens=8, ignore_eos=True))
    ahead0 = llm.steps_ahead
    st, wall, at_mark = timed_generate(llm, prompts, sps, args.steps)
    steps_ahead = llm.steps_ahead - ahead0
    total = sum(max_tokens)                  # every sequence runs to its max_tokens (ignore_eos)
    all_steps = st["prefill_steps"] + st["decode_steps"]
    stats = dict(steps=all_steps, prefill_steps=st["prefill_steps"], decode_steps=st["decode_steps"],
                 prefill_s=round(st["prefill_time"], 3), decode_s=round(st["decode_time"], 3),
                 decode_ms_per_step=round(1e3 * st["decode_time"] / max(1, st["decode_steps"]), 3),
                 decode_steps_run_ahead=steps_ahead,     # launched before the ids of the step before were read back
                 decode_byte_floor=decode_byte_floor(llm.config.hf_config, st, quantization, kv_itemsize=2))
    if args.steps > 0 and at_mark is not None:
        slice_steps, slice_s = args.steps, at_mark
    else:
        slice_steps, slice_s = all_steps, wall
    mr = llm.model_runner
    if getattr(mr, "graph_kernels", None):
        # kernels of one decode step: the captured graph of the largest batch bucket plus the LM head + argmax
        # that follow it (counted by the library around one call)
        from tinyllmforge_amd import _lib
        lib = _lib.load()
        top = max(mr.graph_kernels)
        before = lib.tlf_kernel_launches()
        mr.model.compute_greedy_ids(mr.graph_vars["outputs"][:top])
        torch.cuda.synchronize()
        stats["kernels_per_decode_step"] = dict(batch_bucket=top, in_graph=mr.graph_kernels[top],
                                                lm_head_and_argmax=lib.tlf_kernel_launches() - before,
                                                layers=llm.config.hf_config.num_hidden_layers)
    res = dict(tok_s=total / wall, wall_s=wall, total_output_tokens=total, init_s=round(init_s, 1), stats=stats,
               kv_blocks=llm.config.num_kvcache_blocks, slice_steps=slice_steps, slice_s=slice_s)
    if quantization is not None:
        # the reference's script samples at temperature 0.6 (bench.py:49): same workload through the
        # logits + sampling-kernel path instead of the fused LM head + argmax
        hot = [SamplingParams(temperature=0.6, ignore_eos=True, max_tokens=m) for m in max_tokens]
        shifted = [[(t + 1) % 10001 for t in p] for p in prompts]          # other tokens: no prefix-cache hits
        st6, w, _ = timed_generate(llm, shifted, hot)
        res["temperature_0.6"] = dict(tok_s=round(total / w, 1), wall_s=round(w, 3),
                                      decode_ms_per_step=round(1e3 * st6["decode_time"] / max(1, st6["decode_steps"]), 3))
    cpu = None
    if quantization is None and not args.no_cpu_baseline:
        cpu = cpu_baseline_e2e(llm, prompts)
    llm.exit()
    del llm
    import gc
    gc.collect()
    torch.cuda.empty_cache()
    return res, cpu


def decode_byte_floor(hf, st, quantization, kv_itemsize):
    """Bytes a decode phase cannot avoid: every linear weight (and the bf16 LM head) once per step plus every
    context token's K and V row once per layer; the time they take at the HBM peak, beside the measured time."""
    h, i, L = hf.hidden_size, hf.intermediate_size, hf.num_hidden_layers
    hq, hkv, dh, v = hf.num_attention_heads, hf.num_key_value_heads, hf.head_dim, hf.vocab_size
    lin = L * ((hq + 2 * hkv) * dh * h + hq * dh * h + 2 * i * h + h * i)
    w_step = lin * (1 if quantization == "w8a16" else 2) + v * h * 2
    kv = st["decode_context_tokens"] * hkv * dh * 2 * kv_itemsize * L
    floor_s = (st["decode_steps"] * w_step + kv) / (HBM_PEAK_GBPS * 1e9)
    return dict(weight_GB_per_step=round(w_step / 1e9, 3), kv_GB_total=round(kv / 1e9, 1),
                floor_s_at_hbm_peak=round(floor_s, 3), measured_s=round(st["decode_time"], 3),
                frac=round(floor_s / max(st["decode_time"], 1e-9), 4))


def cpu_baseline_e2e(llm, prompts, nseq=3, out_tokens=6):
    """CPU oracle (bf16 F.linear, the reference's own CPU arithmetic) on the first ``nseq`` sequences of the
    same workload, ``out_tokens`` greedy tokens each, with the same weights copied from the GPU model."""
    import torch
    from oracle.model import OracleQwen3, greedy_generate
    torch.set_num_threads(os.cpu_count() if (os.cpu_count() or 0) <= 64 else 16)
    cfg = vars(llm.config.hf_config)
    params = {k: v.cpu() for k, v in llm.model_runner.model.checkpoint_parameters().items()}
    model = OracleQwen3(cfg, params, exact=False)
    sample = prompts[:nseq]
    t0 = time.perf_counter()
    greedy_generate(model, sample, max_tokens=out_tokens, block_size=256)
    dt = time.perf_counter() - t0
    return dict(value=round(nseq * out_tokens / dt, 4), unit="tok/s", cores=torch.get_num_threads(), kind="port",
                sample=f"first {nseq} of 256 sequences of the same workload (prompts {[len(p) for p in sample]} tokens), "
                       f"{out_tokens} greedy output tokens each, bf16 linears, same weights: {dt:.1f} s of CPU oracle time "
                       f"(prefill included, as in the metric)")


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
    extra = {}
    attn = bench_decode_attn(args, fp8=args.fp8, hq=args.hq) if args.workload == "decode_attn" else bench_decode_attn(args)
    roofline = attn["roofline"]
    extra["paged_decode_GBps_back_to_back"] = round(attn["value"], 1)
    extra["paged_decode_planned"] = attn["planned"]
    extra["hbm_probe"] = bench_probes(args)
    if args.workload in ("gemm", "all"):
        sets = {"8b": GEMM_SHAPES, "32b": GEMM_SHAPES_32B, "0.6b": GEMM_SHAPES_06B,
                "all": {**GEMM_SHAPES, **GEMM_SHAPES_32B, **GEMM_SHAPES_06B}}
        extra["w8a16_gemm"] = bench_gemm(args, shapes=sets[args.gemm_shapes])
    if args.workload == "gemm":   # its own line: the linear-layer microbench (BASELINE.json configs[2])
        best = max(r["TFLOPs"] for r in extra["w8a16_gemm"])
        print(json.dumps({
            "metric": "W8A16 GEMM TFLOP/s vs bf16 MFMA peak", "value": best, "unit": "TFLOP/s", "n_gpus": 1, "steps": 100,
            "warmup": 10, "ms_per_step": None, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
            "dtype": "bf16", "data": "synthetic",
            "config": {"workload": "BASELINE.json configs[2]: y = x W^T, int8 per-channel weights, bf16 activations, the four "
                                   "Qwen3-8B projection shapes, M = 1 ... 8192, random normal x, random int8 W"},
            "roofline": roofline, "cpu_baseline": None if args.no_cpu_baseline else cpu_baseline_gemm(),
            "extra": extra}))
        return
    if args.workload == "clock":   # its own line: the shader clock under each load
        clk = bench_clock(args)
        extra["clock_probe"] = clk
        gemm = next((r for r in clk.get("loads", []) if "random data" in r["load"]), None)
        print(json.dumps({
            "metric": "W8A16 GEMM TFLOP/s vs bf16 MFMA peak", "value": gemm and gemm["TFLOPs"], "unit": "TFLOP/s", "n_gpus": 1,
            "steps": None, "warmup": 1, "ms_per_step": None, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
            "dtype": "bf16", "data": "synthetic",
            "config": {"workload": "shader clock (rocm-smi) under the MFMA stream, the gate_up GEMM at 8192 tokens and decode attention"},
            "roofline": roofline, "cpu_baseline": None, "extra": extra}))
        return
    if args.workload == "elementwise":   # its own line: the single-pass kernels
        rows = bench_elementwise(args)
        extra["elementwise"] = rows
        big = [r for r in rows if r["data"] == "cold"]
        worst = min(big, key=lambda r: r["frac"])
        print(json.dumps({
            "metric": "elementwise kernels: algorithmic GB/s vs HBM peak (worst kernel at 16,384 tokens)", "value": worst["GBps"],
            "unit": "GB/s", "n_gpus": 1, "steps": 20, "warmup": 1, "ms_per_step": round(worst["us"] * 1e-3, 5),
            "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
            "config": {"workload": "single-pass kernels at the Qwen3-8B widths, 16,384 and 256 tokens: " + worst["kernel"]},
            "roofline": {"bound": "hbm", "achieved": worst["GBps"], "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                         "frac": worst["frac"], "traffic": None, "kernel": worst["kernel"]},
            "cpu_baseline": None, "extra": extra}))
        return
    if args.workload == "prefill_attn":   # its own line: the prefill-attention microbench
        rows = bench_prefill_attn(args)
        extra["prefill_attn"] = rows
        best = max(rows, key=lambda r: r["TFLOPs"])
        print(json.dumps({
            "metric": "varlen causal prefill attention TFLOP/s vs bf16 MFMA peak", "value": best["TFLOPs"], "unit": "TFLOP/s",
            "n_gpus": 1, "steps": 25, "warmup": 6, "ms_per_step": round(best["us"] * 1e-3, 4), "higher_is_better": True,
            "scaling": "weak", "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
            "config": {"workload": "prefill attention microbench: " + best["case"]},
            "roofline": {"bound": "mfma", "achieved": best["TFLOPs"], "peak": MFMA_BF16_PEAK_TFLOPS, "unit": "TFLOP/s",
                         "frac": best["frac"], "traffic": None, "kernel": "prefill_attn_kernel"},
            "cpu_baseline": None, "extra": extra}))
        return
    if args.workload == "decode_attn":
        cpu = None if args.no_cpu_baseline else cpu_baseline_decode(attn["case"])
        out = {
            "metric": "paged-decode HBM GB/s vs peak", "value": round(attn["value"], 1), "unit": "GB/s", "n_gpus": 1,
            "steps": args.attn_steps, "warmup": 30, "ms_per_step": round(attn["ms_per_step"], 5),
            "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
            "config": {"workload": "BASELINE.json configs[1]: paged decode attention microbench, B=%d Hq=%d Hkv=8 "
                                   "Dh=128 block_size=256 ctx~U[512,4096] pool=2048 blocks, %s cache rows"
                                   % (args.batch, args.hq, "e4m3" if args.fp8 else "bf16"),
                       "total_context_tokens": attn["case"]["total_tokens"]},
            "roofline": roofline, "cpu_baseline": cpu, "extra": extra}
        print(json.dumps(out))
        return
    del attn
    torch.cuda.empty_cache()
    if args.workload == "e2e" and not args.skip_gemm:
        extra["w8a16_gemm"] = bench_gemm(args)          # BASELINE.json configs[2]
        extra["elementwise"] = bench_elementwise(args)
        extra["clock_probe"] = bench_clock(args)
    # the decode microbench on e4m3 rows with 64 query heads (the 32B shape's attention)
    a8 = bench_decode_attn(args, fp8=True, hq=64)
    a8.pop("case")
    extra["paged_decode_fp8_rows"] = dict(a8["roofline"], planned=a8["planned"])
    del a8
    torch.cuda.empty_cache()
    if args.workload in ("c5", "all") or (args.workload == "e2e" and not args.skip_c5):
        c5 = bench_c5(args)
        extra["config5_qwen3_32b_fp8kv"] = c5
        import gc
        gc.collect()
        torch.cuda.empty_cache()
        if args.workload == "c5":   # its own line: same metric on the 32B-shape configuration
            steps = c5["prefill_steps"] + c5["decode_steps"]
            print(json.dumps({
                "metric": "output tok/s (Qwen3-32B-shape, 1 GPU); paged-decode HBM GB/s vs peak", "value": c5["tok_s"],
                "unit": "tok/s", "n_gpus": 1, "steps": steps, "warmup": 1,
                "ms_per_step": round(1e3 * c5["wall_s"] / max(1, steps), 4), "higher_is_better": True,
                "scaling": "weak", "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
                "config": {"workload": "BASELINE.json configs[4]: Qwen3-32B-shaped decoder, random-init, W8A16 linears, "
                                       "e4m3 KV cache, 32 sequences, prompts ~U[2048,8192] tokens (half share a cached "
                                       "1024-token prefix), 256 greedy output tokens each, hipGraph decode",
                           "roofline_workload": "BASELINE.json configs[1] paged decode attention microbench"},
                "roofline": roofline, "cpu_baseline": None, "extra": extra}))
            return
    w8, _ = bench_e2e(args, "w8a16")
    cpu = None
    if not args.skip_bf16:
        bf, cpu = bench_e2e(args, None)
        extra["bf16_linears"] = {"tok_s": round(bf["tok_s"], 1), "wall_s": round(bf["wall_s"], 3), "stats": bf["stats"]}
    extra["w8a16_linears"] = {"tok_s": round(w8["tok_s"], 1), "wall_s": round(w8["wall_s"], 3), "stats": w8["stats"],
                              "kv_blocks": w8["kv_blocks"]}
    if "temperature_0.6" in w8:
        extra["w8a16_linears"]["temperature_0.6"] = w8["temperature_0.6"]
    whole = w8["slice_steps"] == w8["stats"]["steps"]
    out = {
        "metric": "output tok/s (Qwen3-8B-shape, 1 GPU); paged-decode HBM GB/s vs peak",
        "value": round(w8["tok_s"], 1),
        "unit": "tok/s",
        "n_gpus": 1,
        "steps": w8["slice_steps"],
        "warmup": max(1, args.warmup),
        "ms_per_step": round(1e3 * w8["slice_s"] / max(1, w8["slice_steps"]), 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16",
        "data": "synthetic",
        "config": {"workload": "BASELINE.json configs[3]: end-to-end Qwen3-8B-shaped decoder, random-init, W8A16 linears "
                               "(int8 weights, bf16 activations and MFMA), bf16 KV cache, %d sequences, prompts and outputs "
                               "~U[100,1024] tokens, ignore_eos, greedy, continuous batching, hipGraph decode; value = "
                               "sum(max_tokens) / wall time of the WHOLE job (%d engine steps, %.3f s)"
                               % (args.num_seqs, w8["stats"]["steps"], w8["wall_s"]),
                   "steps_describe": ("all engine steps of the timed job" if whole else
                                      "the first %d engine steps of the same timed job (prefill-heavy: the job starts "
                                      "with its prefill steps); ms_per_step is their mean" % w8["slice_steps"]),
                   "total_output_tokens": w8["total_output_tokens"],
                   "roofline_workload": "BASELINE.json configs[1] paged decode attention microbench"},
        "roofline": roofline,
        "cpu_baseline": cpu,
        "extra": extra,
    }
    print(json.dumps(out))


if __name__ == "__main__":
    main()
