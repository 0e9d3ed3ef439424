"""CPU-side checks of the C-ABI library: it loads and exports every declared symbol.

No compute call is made here (there is no GPU in the build container).
"""
import ctypes
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "tlf_hip.h")


def declared_symbols():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(tlf_[a-z0-9_]+)\s*\(", text)))


def test_header_declares_the_expected_entry_points():
    syms = declared_symbols()
    for name in ["tlf_store_kvcache", "tlf_paged_decode_attn", "tlf_varlen_prefill_attn", "tlf_rmsnorm",
                 "tlf_add_rmsnorm", "tlf_rope", "tlf_silu_and_mul", "tlf_argmax", "tlf_w8a16_gemm"]:
        assert name in syms


def test_library_loads_and_exports_every_declared_symbol():
    from tinyllmforge_amd import _lib
    assert os.path.exists(_lib.LIB_PATH), "build the library first: python tinyllmforge_amd/csrc/build.py"
    lib = _lib.load()
    for name in declared_symbols():
        assert hasattr(lib, name), f"{name} declared in tlf_hip.h but not exported"
        assert name in _lib.SIGNATURES, f"{name} has no ctypes signature"
    assert sorted(_lib.SIGNATURES) == declared_symbols()
    assert lib.tlf_version() == _lib.ABI_VERSION
    assert lib.tlf_error_string(0) == b"ok"
    assert b"NULL" in lib.tlf_error_string(-1)


def test_argument_rejection_happens_before_any_launch():
    """NULL pointers / bad shapes are rejected on the host; nothing touches a GPU."""
    from tinyllmforge_amd import _lib
    lib = _lib.load()
    assert lib.tlf_store_kvcache(None, 0, None, 0, None, None, None, 4, 2048, 10, None) == -1
    assert lib.tlf_store_kvcache(None, 0, None, 0, None, None, None, 0, 2048, 10, None) == 0   # empty batch
    assert lib.tlf_silu_and_mul(16, 16, 3, 12, None) == -2        # inter % 8 != 0
    assert lib.tlf_silu_and_mul(8, 16, 3, 16, None) == -3         # misaligned x
    assert lib.tlf_rmsnorm(16, 128, 16, 16, 2, 1, 100, 1e-6, None) == -2
    assert lib.tlf_argmax(16, 64, 16, 2, 64, None, 0, None) == -4
    assert lib.tlf_paged_decode_attn(16, 4096, 16, 16, 0, None, None, 16, 16, 16, 16,
                                     2, 32, 8, 64, 256, 16, 10, 0.1, None, 0, None) == -5  # Dh != 128
    assert lib.tlf_argmax_workspace_bytes(4, 151936) > 0
    # the decode plan: NULL operands, too many sequences, a block size that is no multiple of a tile, a small buffer
    a256 = 4096
    nplan = lib.tlf_paged_decode_plan_bytes()
    assert nplan > 0 and nplan % 16 == 0
    assert lib.tlf_paged_decode_plan(None, a256, 16, 4, 256, 16, a256, nplan, None) == -1
    assert lib.tlf_paged_decode_plan(a256, a256, 16, 1025, 256, 16, a256, nplan, None) == -2
    assert lib.tlf_paged_decode_plan(a256, a256, 16, 4, 250, 16, a256, nplan, None) == -2
    assert lib.tlf_paged_decode_plan(a256, a256, 8, 4, 256, 16, a256, nplan, None) == -2          # table stride < max_blocks
    assert lib.tlf_paged_decode_plan(a256, a256, 16, 4, 256, 16, a256, nplan - 4, None) == -4
    assert lib.tlf_paged_decode_plan(a256, a256, 16, 0, 256, 16, None, 0, None) == 0               # no sequences
    assert lib.tlf_paged_decode_attn_planned(16, 4096, 16, 16, 0, None, None, 16, 16, 16, 16,
                                             2, 32, 8, 128, 256, 16, 10, 0.1, a256, 1 << 30, None, None) == -1   # no plan
    # the fused entry points: NULL operands, a missing or misaligned workspace, bad shapes
    a = 4096                                                          # any 256-byte aligned non-NULL value
    assert lib.tlf_w8a16_gemm_add_rmsnorm(a, 4096, a, a, None, a, a, a, 8, 4096, 4096, 1e-6, a, 1 << 30, None) == -1
    assert lib.tlf_w8a16_gemm_add_rmsnorm(a, 4096, a, a, a, a, a, a, 8, 4096, 4096, 1e-6, None, 0, None) == -4
    assert lib.tlf_w8a16_gemm_add_rmsnorm(a, 4096, a, a, a, a, a, a, 8, 32768, 4096, 1e-6, a, 1 << 30, None) == -2
    assert lib.tlf_bf16_gemm_add_rmsnorm(a, 4096, a, a, a, a, a, 0, 4096, 4096, 1e-6, None, 0, None) == 0   # no tokens
    assert lib.tlf_bf16_gemm_argmax(a, 4096, a, None, 8, 4096, 4096, a, 1 << 30, None) == -1
    assert lib.tlf_bf16_gemm_argmax(a, 4096, a, a, 8, 4096, 4096, a, 16, None) == -4
    assert lib.tlf_bf16_gemm_argmax(a, 4000, a, a, 8, 4096, 4096, a, 1 << 30, None) == -2        # row stride < K
    assert lib.tlf_sample(a, 1024, None, a, 4, 1024, 0, 0, a, 1 << 20, None) == -1
    assert lib.tlf_sample(a, 1000, a, a, 4, 1024, 0, 0, a, 1 << 20, None) == -2
    assert lib.tlf_sample(a, 1024, a, a, 4, 1024, 0, 0, a, 8, None) == -4
    # the entry point without allocation: its limit is enforced on the host, before anything touches a GPU
    assert lib.tlf_argmax_noalloc_max_rows() == 1024
    assert lib.tlf_argmax_noalloc(a, 64, a, 1025, 64, None) == -6 and b"scratch" in lib.tlf_error_string(-6)
    assert lib.tlf_argmax_noalloc(None, 64, a, 4, 64, None) == -1
    assert lib.tlf_argmax_noalloc(a, 60, a, 4, 64, None) == -2
    assert lib.tlf_argmax_noalloc(a, 64, a, 0, 64, None) == 0
    m, n, k = 200, 4096, 12288
    assert lib.tlf_gemm_add_rmsnorm_workspace_bytes(m, n, k) >= lib.tlf_w8a16_gemm_workspace_bytes(m, n, k) + m * n * 2
    assert lib.tlf_gemm_argmax_workspace_bytes(256, 151936, 4096) >= 256 * (151936 // 32) * 8
    assert lib.tlf_gemm_argmax_workspace_bytes(4, 151936, 4096) >= 4 * 151936 * 2 + lib.tlf_argmax_workspace_bytes(4, 151936)


def test_ops_refuse_cpu_tensors():
    import torch
    from tinyllmforge_amd import ops, _lib
    with pytest.raises(_lib.TlfError):
        ops.silu_and_mul(torch.zeros(2, 16, dtype=torch.bfloat16))


def test_gemm_plan_has_a_kernel_for_every_shape_the_models_use():
    """Host-only sweep of the GEMM planner (no GPU call): every token count from 1 to 600 and a few large
    ones, every projection of the three Qwen3 shapes plus the LM head, int8 and bf16 weights, must map to
    an existing kernel instance with a consistent split of K that the workspace query covers."""
    import ctypes
    from tinyllmforge_amd import _lib
    lib = _lib.load()
    shapes = set()
    for h, hq, hkv, inter in [(1024, 16, 8, 3072), (4096, 32, 8, 12288), (5120, 64, 8, 25600)]:
        shapes |= {((hq + 2 * hkv) * 128, h), (h, hq * 128), (2 * inter, h), (h, inter), (151936, h)}
    ms = list(range(1, 601)) + [777, 1024, 2047, 4096, 8192, 16384]
    plan = (ctypes.c_int32 * 8)()
    seen = set()
    for n, k in sorted(shapes):
        for w8 in (0, 1):
            for m in ms:
                rc = lib.tlf_gemm_plan(m, n, k, w8, plan)
                assert rc == 0, f"no kernel for M={m} N={n} K={k} w8={w8}: rc={rc} plan={list(plan)}"
                bn, bm, stages, occ, kgroups, splits, k_per_split, group_n = list(plan)
                seen.add((bn, bm, stages, occ, kgroups))
                assert k_per_split % 64 == 0 and splits >= 1 and splits * k_per_split >= k
                assert (splits - 1) * k_per_split < k, "an empty split"
                if bn:   # tiled kernel
                    assert (k_per_split // 64) % kgroups == 0 and ((k - (splits - 1) * k_per_split) // 64) % kgroups == 0
                    assert 1 <= group_n <= 4
                    if splits > 1:
                        assert lib.tlf_w8a16_gemm_workspace_bytes(m, n, k) >= splits * m * n * 4
    assert len(seen) >= 6, seen          # the sweep reaches the skinny kernel and several tile shapes
    assert lib.tlf_gemm_plan(4, 1024, 100, 1, plan) == -2   # K not a multiple of 64
