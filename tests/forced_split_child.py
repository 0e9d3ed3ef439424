"""Child process of test_gpu_gemm.py::test_reduce_kernels_under_forced_split_counts: the library reads TLF_GEMM_PLAN
once per process, so every forced plan needs a process of its own.  Exits 0 when, under the plan in the environment,
the fused projection + add-RMSNorm equals projection, then add-RMSNorm, bit for bit, and the projection alone is exact
on integer-valued data (fp64 product, one rounding)."""
import os
import sys

sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.abspath(__file__))))

import torch  # noqa: E402

from tinyllmforge_amd import ops as P  # noqa: E402


def main():
    import ctypes
    from tinyllmforge_amd import _lib
    lib = _lib.load()
    want = int(os.environ["TLF_GEMM_PLAN"].split(",")[2])
    torch.manual_seed(1)
    bad = []
    for (M, N, K) in [(40, 5120, 2048), (40, 4096, 2048), (33, 10240, 2048), (70, 2048, 2048), (17, 8192, 4096)]:
        plan = (ctypes.c_int32 * 8)()
        lib.tlf_gemm_plan(M, N, K, 1, plan)
        if plan[5] != want:        # fields: tile n, tile m, stages, occupancy, K groups, splits, K per split, group
            bad.append(("plan not forced", (M, N, K), list(plan)))
        x = torch.randn(M, K, device="cuda").to(torch.bfloat16)
        wq = torch.randint(-127, 128, (N, K), dtype=torch.int8, device="cuda")
        sc = torch.rand(N, device="cuda") * 0.01 + 0.001
        res = torch.randn(M, N, device="cuda").to(torch.bfloat16)
        nw = torch.randn(N, device="cuda").to(torch.bfloat16)
        y1, r1 = P.linear_add_rms_norm(x, wq, sc, res, nw, 1e-6)
        y2, r2 = P.add_rms_norm(P.w8a16_linear(x, wq, sc), res.clone(), nw, 1e-6)
        xi = torch.randint(-3, 4, (M, K), device="cuda").to(torch.bfloat16)
        wi = torch.randint(-5, 6, (N, K), dtype=torch.int8, device="cuda")
        ref = ((xi.double() @ wi.double().T) * 0.25).to(torch.bfloat16)
        got = P.w8a16_linear(xi, wi, torch.full((N,), 0.25, device="cuda"))
        if not (torch.equal(y1, y2) and torch.equal(r1, r2) and torch.equal(ref, got)):
            bad.append((M, N, K))
    print("plan", os.environ.get("TLF_GEMM_PLAN"), "mismatches", bad, flush=True)
    return 1 if bad else 0


if __name__ == "__main__":
    sys.exit(main())
