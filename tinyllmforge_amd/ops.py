"""Tensor-level wrappers over the C ABI: one function per hot-path op.

Each wrapper validates what only Python can see (device, dtype), allocates the
output through torch (the caller owns every buffer, as in the reference) and
enqueues the kernel on torch's current stream, so calls are capturable by
``torch.cuda.graph``.  A tensor that is not on the GPU is an error.
"""
from __future__ import annotations

import torch

from . import _lib
from ._lib import KV_BF16, KV_FP8_E4M3, check

BF16 = torch.bfloat16


def _stream():
    return torch.cuda.current_stream().cuda_stream


def _need(t: torch.Tensor, dtype, name: str):
    if not t.is_cuda:
        raise _lib.TlfError(f"{name} must be a GPU tensor (the HIP path has no CPU fallback)")
    if dtype is not None and t.dtype != dtype:
        raise _lib.TlfError(f"{name} must be {dtype}, got {t.dtype}")


_workspaces: dict = {}
_retired: list = []   # outgrown buffers stay alive: a captured graph may still point at them


def _workspace(nbytes: int, device, tag: str) -> torch.Tensor:
    """Grow-only scratch buffer per (device, tag).  Never freed, so pointers recorded in a
    captured graph stay valid.  No kernel needs it cleared."""
    key = (device, tag)
    ws = _workspaces.get(key)
    if ws is None or ws.numel() < nbytes:
        if ws is not None:
            _retired.append(ws)
        ws = torch.empty(max(nbytes, 256), dtype=torch.uint8, device=device)
        _workspaces[key] = ws
    return ws


def kv_dtype_code(cache: torch.Tensor) -> int:
    if cache.dtype == BF16:
        return KV_BF16
    if cache.dtype == torch.float8_e4m3fn:
        return KV_FP8_E4M3
    raise _lib.TlfError(f"unsupported KV-cache dtype {cache.dtype}")


# ------------------------------------------------------------------ a1
def store_kvcache(key, value, k_cache, v_cache, slot_mapping, k_scale=None, v_scale=None):
    """``key``/``value`` ``[N, Hkv, Dh]`` (row stride free), caches ``[nblk, bs, Hkv, Dh]``."""
    lib = _lib.load()
    _need(key, BF16, "key"); _need(value, BF16, "value")
    _need(slot_mapping, torch.int32, "slot_mapping")
    n, h, d = key.shape
    assert key.stride(-1) == 1 and value.stride(-1) == 1
    assert key.stride(1) == d and value.stride(1) == d
    assert k_cache.is_contiguous() and v_cache.is_contiguous()
    assert slot_mapping.numel() == n
    num_slots = k_cache.numel() // (h * d)
    if k_cache.dtype == BF16:
        check(lib.tlf_store_kvcache(key.data_ptr(), key.stride(0) * 2, value.data_ptr(), value.stride(0) * 2,
                                    k_cache.data_ptr(), v_cache.data_ptr(), slot_mapping.data_ptr(),
                                    n, h * d * 2, num_slots, _stream()), "tlf_store_kvcache")
    else:
        _need(k_scale, torch.float32, "k_scale"); _need(v_scale, torch.float32, "v_scale")
        check(lib.tlf_store_kvcache_fp8(key.data_ptr(), key.stride(0) * 2, value.data_ptr(), value.stride(0) * 2,
                                        k_cache.data_ptr(), v_cache.data_ptr(), slot_mapping.data_ptr(),
                                        n, h, d, k_scale.data_ptr(), v_scale.data_ptr(), num_slots, _stream()),
              "tlf_store_kvcache_fp8")


# ------------------------------------------------------------------ a5 / a6
def rms_norm(x, weight, eps):
    """``x [..., cols]`` bf16; leading dims may be a strided view ``[outer, inner, cols]``."""
    lib = _lib.load()
    _need(x, BF16, "x"); _need(weight, BF16, "weight")
    cols = x.shape[-1]
    assert x.stride(-1) == 1
    if x.dim() == 3 and not x.is_contiguous():
        outer, inner = x.shape[0], x.shape[1]
        assert x.stride(1) == cols
        ostride = x.stride(0)
    else:
        x = x if x.is_contiguous() else x.contiguous()
        outer, inner, ostride = x.numel() // cols, 1, cols
    y = torch.empty(x.shape, dtype=BF16, device=x.device)
    check(lib.tlf_rmsnorm(x.data_ptr(), ostride, weight.data_ptr(), y.data_ptr(), outer, inner, cols,
                          float(eps), _stream()), "tlf_rmsnorm")
    return y


def add_rms_norm(x, residual, weight, eps):
    lib = _lib.load()
    _need(x, BF16, "x"); _need(residual, BF16, "residual"); _need(weight, BF16, "weight")
    assert x.is_contiguous() and residual.is_contiguous() and x.shape == residual.shape
    cols = x.shape[-1]
    rows = x.numel() // cols
    y = torch.empty_like(x)
    r = torch.empty_like(x)
    check(lib.tlf_add_rmsnorm(x.data_ptr(), residual.data_ptr(), weight.data_ptr(), y.data_ptr(),
                              r.data_ptr(), rows, cols, float(eps), _stream()), "tlf_add_rmsnorm")
    return y, r


# ------------------------------------------------------------------ a7
def rope(positions, q, k, cos_sin, head_dim):
    lib = _lib.load()
    _need(positions, torch.int64, "positions"); _need(q, BF16, "q"); _need(k, BF16, "k")
    _need(cos_sin, torch.float32, "cos_sin_cache")
    n = positions.numel()
    assert q.stride(-1) == 1 and k.stride(-1) == 1 and q.dim() == 2 and k.dim() == 2
    hq, hkv = q.shape[1] // head_dim, k.shape[1] // head_dim
    qo = torch.empty(q.shape, dtype=BF16, device=q.device)
    ko = torch.empty(k.shape, dtype=BF16, device=k.device)
    check(lib.tlf_rope(positions.data_ptr(), q.data_ptr(), q.stride(0), k.data_ptr(), k.stride(0),
                       cos_sin.data_ptr(), qo.data_ptr(), ko.data_ptr(), n, hq, hkv, head_dim,
                       cos_sin.shape[0], _stream()), "tlf_rope")
    return qo, ko


def qknorm_rope_store(qkv, q_weight, k_weight, eps, positions, cos_sin, num_q_heads, num_kv_heads, head_dim,
                      k_cache=None, v_cache=None, slot_mapping=None, k_scale=None, v_scale=None,
                      want_kv=False):
    """Fused q/k-norm + RoPE + KV store.  Returns ``(q, k, v)``; ``k``/``v`` are None unless ``want_kv``."""
    lib = _lib.load()
    _need(qkv, BF16, "qkv"); _need(positions, torch.int64, "positions")
    n = qkv.shape[0]
    assert qkv.stride(-1) == 1
    q = torch.empty(n, num_q_heads * head_dim, dtype=BF16, device=qkv.device)
    k = v = None
    if want_kv:
        k = torch.empty(n, num_kv_heads * head_dim, dtype=BF16, device=qkv.device)
        v = torch.empty(n, num_kv_heads * head_dim, dtype=BF16, device=qkv.device)
    has_cache = k_cache is not None and k_cache.numel() > 0 and slot_mapping is not None
    kvd = kv_dtype_code(k_cache) if has_cache else KV_BF16
    num_slots = (k_cache.numel() // (num_kv_heads * head_dim)) if has_cache else 0
    check(lib.tlf_qknorm_rope_store(
        qkv.data_ptr(), qkv.stride(0), q_weight.data_ptr(), k_weight.data_ptr(), float(eps),
        positions.data_ptr(), cos_sin.data_ptr(), cos_sin.shape[0], q.data_ptr(),
        k.data_ptr() if k is not None else None, v.data_ptr() if v is not None else None,
        k_cache.data_ptr() if has_cache else None, v_cache.data_ptr() if has_cache else None,
        slot_mapping.data_ptr() if has_cache else None, num_slots, kvd,
        k_scale.data_ptr() if k_scale is not None else None,
        v_scale.data_ptr() if v_scale is not None else None,
        n, num_q_heads, num_kv_heads, head_dim, _stream()), "tlf_qknorm_rope_store")
    return q, k, v


# ------------------------------------------------------------------ a8
def silu_and_mul(x):
    lib = _lib.load()
    _need(x, BF16, "x")
    assert x.is_contiguous() and x.shape[-1] % 2 == 0
    inter = x.shape[-1] // 2
    rows = x.numel() // (2 * inter)
    y = torch.empty(*x.shape[:-1], inter, dtype=BF16, device=x.device)
    check(lib.tlf_silu_and_mul(x.data_ptr(), y.data_ptr(), rows, inter, _stream()), "tlf_silu_and_mul")
    return y


# ------------------------------------------------------------------ a9
def argmax(logits):
    lib = _lib.load()
    _need(logits, BF16, "logits")
    assert logits.dim() == 2 and logits.stride(1) == 1
    rows, vocab = logits.shape
    out = torch.empty(rows, dtype=torch.int64, device=logits.device)
    nbytes = lib.tlf_argmax_workspace_bytes(rows, vocab)
    ws = _workspace(nbytes, logits.device, "argmax")
    check(lib.tlf_argmax(logits.data_ptr(), logits.stride(0), out.data_ptr(), rows, vocab,
                         ws.data_ptr(), ws.numel(), _stream()), "tlf_argmax")
    return out


def sample(logits, temperatures, seed: int, offset: int):
    """Sampler with temperatures: greedy where ``temperatures == 0``, else one draw from
    ``softmax(logits / T)`` by the exponential-race formula of the reference, noise from Philox4x32-10
    at (``seed``, ``offset``).  int64 ``[rows]``."""
    lib = _lib.load()
    _need(logits, BF16, "logits"); _need(temperatures, torch.float32, "temperatures")
    assert logits.dim() == 2 and logits.stride(1) == 1 and temperatures.is_contiguous()
    rows, vocab = logits.shape
    assert temperatures.numel() == rows
    out = torch.empty(rows, dtype=torch.int64, device=logits.device)
    ws = _workspace(lib.tlf_argmax_workspace_bytes(rows, vocab), logits.device, "argmax")
    check(lib.tlf_sample(logits.data_ptr(), logits.stride(0), temperatures.data_ptr(), out.data_ptr(), rows,
                         vocab, seed & (2 ** 64 - 1), offset & (2 ** 64 - 1), ws.data_ptr(), ws.numel(),
                         _stream()), "tlf_sample")
    return out


# ------------------------------------------------------------------ K9
def embedding(ids, weight):
    lib = _lib.load()
    _need(ids, torch.int64, "ids"); _need(weight, BF16, "weight")
    assert weight.is_contiguous() and ids.is_contiguous()
    n = ids.numel()
    y = torch.empty(*ids.shape, weight.shape[1], dtype=BF16, device=weight.device)
    check(lib.tlf_embedding(ids.data_ptr(), weight.data_ptr(), y.data_ptr(), n, weight.shape[0],
                            weight.shape[1], _stream()), "tlf_embedding")
    return y


# ------------------------------------------------------------------ a10
class PackedW8:
    """An int8 weight ``[n, k]`` in the tile order the W8A16 kernels read (``tlf_w8a16_pack_weight``):
    same bytes as the row-major tensor, rows padded to a multiple of 32."""
    __slots__ = ("data", "n", "k")

    def __init__(self, data: torch.Tensor, n: int, k: int):
        self.data, self.n, self.k = data, n, k

    @property
    def shape(self):
        return (self.n, self.k)

    @property
    def device(self):
        return self.data.device

    def data_ptr(self):
        return self.data.data_ptr()


def pack_w8(wq: torch.Tensor) -> PackedW8:
    """Row-major int8 ``[N, K]`` -> ``PackedW8`` (one pass on the GPU)."""
    lib = _lib.load()
    _need(wq, torch.int8, "wq")
    assert wq.dim() == 2
    wq = wq.contiguous()
    N, K = wq.shape
    nbytes = lib.tlf_w8a16_packed_bytes(N, K)
    if nbytes == 0:
        raise _lib.TlfError(f"cannot pack an int8 weight of shape {tuple(wq.shape)} (K % 64 != 0)")
    out = torch.empty(nbytes, dtype=torch.int8, device=wq.device)
    check(lib.tlf_w8a16_pack_weight(wq.data_ptr(), out.data_ptr(), N, K, _stream()), "tlf_w8a16_pack_weight")
    return PackedW8(out, N, K)


def _packed(wq) -> PackedW8:
    """Weights may be given row-major (packed on the fly: convenient for one-off calls) or packed."""
    return wq if isinstance(wq, PackedW8) else pack_w8(wq)


def w8a16_linear(x, wq, scale):
    lib = _lib.load()
    w = _packed(wq)
    _need(x, BF16, "x"); _need(scale, torch.float32, "scale")
    assert x.stride(-1) == 1
    x2 = x.reshape(-1, x.shape[-1])
    M, K = x2.shape
    N = w.n
    assert w.k == K and scale.numel() == N
    y = torch.empty(M, N, dtype=BF16, device=x.device)
    nbytes = lib.tlf_w8a16_gemm_workspace_bytes(M, N, K)
    ws = _workspace(nbytes, x.device, "gemm")
    check(lib.tlf_w8a16_gemm(x2.data_ptr(), x2.stride(0), w.data_ptr(), scale.data_ptr(), y.data_ptr(),
                             M, N, K, ws.data_ptr(), ws.numel(), _stream()), "tlf_w8a16_gemm")
    return y.view(*x.shape[:-1], N)


def gate_up_interleave_index(n: int, device=None):
    """Row order of the fused gate_up weight: rows ``16 j .. 16 j + 7`` = gate channels ``8 j ..``, rows
    ``16 j + 8 .. 16 j + 15`` = the matching up channels; ``n`` = 2 x intermediate size.  ``w[idx]``
    interleaves a ``[gate; up]`` stacked weight (or scale)."""
    assert n % 16 == 0
    half = n // 2
    j = torch.arange(n, device=device)
    group, r = j // 16, j % 16
    return torch.where(r < 8, group * 8 + r, half + group * 8 + (r - 8))


def w8a16_linear_silu_mul(x, wq_interleaved, scale_interleaved):
    """``silu(gate) * up`` of the int8 gate_up projection in one kernel; weight rows interleaved as
    ``gate_up_interleave_index`` says.  Returns ``[..., N / 2]``."""
    lib = _lib.load()
    w = _packed(wq_interleaved)
    _need(x, BF16, "x"); _need(scale_interleaved, torch.float32, "scale")
    assert x.stride(-1) == 1
    x2 = x.reshape(-1, x.shape[-1])
    M, K = x2.shape
    N = w.n
    assert w.k == K
    y = torch.empty(M, N // 2, dtype=BF16, device=x.device)
    check(lib.tlf_w8a16_gemm_silu_mul(x2.data_ptr(), x2.stride(0), w.data_ptr(),
                                      scale_interleaved.data_ptr(), y.data_ptr(), M, N, K, _stream()),
          "tlf_w8a16_gemm_silu_mul")
    return y.view(*x.shape[:-1], N // 2)


def bf16_linear_silu_mul(x, w_interleaved):
    """``silu(gate) * up`` of the bf16 gate_up projection in one kernel; weight rows interleaved as
    ``gate_up_interleave_index`` says.  Returns ``[..., N / 2]``; the bits of ``silu_and_mul(bf16_linear(x, w))``."""
    lib = _lib.load()
    _need(x, BF16, "x"); _need(w_interleaved, BF16, "w")
    assert x.stride(-1) == 1 and w_interleaved.is_contiguous()
    x2 = x.reshape(-1, x.shape[-1])
    M, K = x2.shape
    N = w_interleaved.shape[0]
    assert w_interleaved.shape[1] == K and N % 16 == 0
    y = torch.empty(M, N // 2, dtype=BF16, device=x.device)
    check(lib.tlf_bf16_gemm_silu_mul(x2.data_ptr(), x2.stride(0), w_interleaved.data_ptr(), y.data_ptr(), M, N, K,
                                     _stream()), "tlf_bf16_gemm_silu_mul")
    return y.view(*x.shape[:-1], N // 2)


def bf16_linear(x, w):
    lib = _lib.load()
    _need(x, BF16, "x"); _need(w, BF16, "w")
    assert x.stride(-1) == 1 and w.is_contiguous()
    x2 = x.reshape(-1, x.shape[-1])
    M, K = x2.shape
    N = w.shape[0]
    y = torch.empty(M, N, dtype=BF16, device=x.device)
    nbytes = lib.tlf_w8a16_gemm_workspace_bytes(M, N, K)
    ws = _workspace(nbytes, x.device, "gemm")
    check(lib.tlf_bf16_gemm(x2.data_ptr(), x2.stride(0), w.data_ptr(), y.data_ptr(), M, N, K,
                            ws.data_ptr(), ws.numel(), _stream()), "tlf_bf16_gemm")
    return y.view(*x.shape[:-1], N)


def bf16_linear_argmax(x, w):
    """``argmax(bf16_linear(x, w), -1)`` (first index among ties) without the logits: int64 ``[M]``."""
    lib = _lib.load()
    _need(x, BF16, "x"); _need(w, BF16, "w")
    assert x.stride(-1) == 1 and w.is_contiguous() and x.dim() == 2
    M, K = x.shape
    N = w.shape[0]
    out = torch.empty(M, dtype=torch.int64, device=x.device)
    ws = _workspace(lib.tlf_gemm_argmax_workspace_bytes(M, N, K), x.device, "gemm")
    check(lib.tlf_bf16_gemm_argmax(x.data_ptr(), x.stride(0), w.data_ptr(), out.data_ptr(), M, N, K,
                                   ws.data_ptr(), ws.numel(), _stream()), "tlf_bf16_gemm_argmax")
    return out


def linear_add_rms_norm(x, w, scale, residual, norm_weight, eps):
    """``add_rms_norm(linear(x), residual)`` behind one call: ``w`` int8 with ``scale`` (weight-only int8)
    or bf16 with ``scale=None``.  Returns ``(normed, new_residual)``, the bits of the two separate calls."""
    lib = _lib.load()
    w8 = scale is not None
    if w8:
        w = _packed(w)
    else:
        _need(w, BF16, "w")
        assert w.is_contiguous()
    _need(x, BF16, "x"); _need(residual, BF16, "residual"); _need(norm_weight, BF16, "norm_weight")
    assert x.stride(-1) == 1 and residual.is_contiguous()
    x2 = x.reshape(-1, x.shape[-1])
    M, K = x2.shape
    N = w.shape[0]
    assert residual.numel() == M * N
    y = torch.empty(M, N, dtype=BF16, device=x.device)
    r = torch.empty(M, N, dtype=BF16, device=x.device)
    ws = _workspace(lib.tlf_gemm_add_rmsnorm_workspace_bytes(M, N, K), x.device, "gemm")
    if w8:
        _need(scale, torch.float32, "scale")
        check(lib.tlf_w8a16_gemm_add_rmsnorm(
            x2.data_ptr(), x2.stride(0), w.data_ptr(), scale.data_ptr(), residual.data_ptr(),
            norm_weight.data_ptr(), y.data_ptr(), r.data_ptr(), M, N, K, float(eps), ws.data_ptr(),
            ws.numel(), _stream()), "tlf_w8a16_gemm_add_rmsnorm")
    else:
        check(lib.tlf_bf16_gemm_add_rmsnorm(
            x2.data_ptr(), x2.stride(0), w.data_ptr(), residual.data_ptr(), norm_weight.data_ptr(),
            y.data_ptr(), r.data_ptr(), M, N, K, float(eps), ws.data_ptr(), ws.numel(), _stream()),
            "tlf_bf16_gemm_add_rmsnorm")
    shape = (*x.shape[:-1], N)
    return y.view(shape), r.view(shape)


def linear_qknorm_rope_store(x, w, scale, q_weight, k_weight, eps, positions, cos_sin, num_q_heads, num_kv_heads,
                             head_dim, k_cache=None, v_cache=None, slot_mapping=None, k_scale=None, v_scale=None,
                             want_kv=False):
    """``qknorm_rope_store(linear(x), ...)`` behind one call: ``w`` int8 with ``scale`` (weight-only int8) or
    bf16 with ``scale=None``.  Returns ``(q, k, v)`` with the bits of the two separate calls."""
    lib = _lib.load()
    w8 = scale is not None
    if w8:
        w = _packed(w)
        _need(scale, torch.float32, "scale")
    else:
        _need(w, BF16, "w")
        assert w.is_contiguous()
    _need(x, BF16, "x"); _need(positions, torch.int64, "positions")
    assert x.stride(-1) == 1
    x2 = x.reshape(-1, x.shape[-1])
    n, K = x2.shape
    N = (num_q_heads + 2 * num_kv_heads) * head_dim
    assert w.shape[0] == N
    q = torch.empty(n, num_q_heads * head_dim, dtype=BF16, device=x.device)
    k = v = None
    if want_kv:
        k = torch.empty(n, num_kv_heads * head_dim, dtype=BF16, device=x.device)
        v = torch.empty(n, num_kv_heads * head_dim, dtype=BF16, device=x.device)
    has_cache = k_cache is not None and k_cache.numel() > 0 and slot_mapping is not None
    kvd = kv_dtype_code(k_cache) if has_cache else KV_BF16
    num_slots = (k_cache.numel() // (num_kv_heads * head_dim)) if has_cache else 0
    ws = _workspace(lib.tlf_gemm_qknorm_rope_store_workspace_bytes(n, N, K), x.device, "gemm")
    tail = (q_weight.data_ptr(), k_weight.data_ptr(), float(eps), positions.data_ptr(), cos_sin.data_ptr(),
            cos_sin.shape[0], q.data_ptr(), k.data_ptr() if k is not None else None,
            v.data_ptr() if v is not None else None, k_cache.data_ptr() if has_cache else None,
            v_cache.data_ptr() if has_cache else None, slot_mapping.data_ptr() if has_cache else None, num_slots,
            kvd, k_scale.data_ptr() if k_scale is not None else None,
            v_scale.data_ptr() if v_scale is not None else None, n, num_q_heads, num_kv_heads, head_dim, K,
            ws.data_ptr(), ws.numel(), _stream())
    if w8:
        check(lib.tlf_w8a16_gemm_qknorm_rope_store(x2.data_ptr(), x2.stride(0), w.data_ptr(), scale.data_ptr(),
                                                   *tail), "tlf_w8a16_gemm_qknorm_rope_store")
    else:
        check(lib.tlf_bf16_gemm_qknorm_rope_store(x2.data_ptr(), x2.stride(0), w.data_ptr(), *tail),
              "tlf_bf16_gemm_qknorm_rope_store")
    return q, k, v


# ------------------------------------------------------------------ a3
def paged_decode_plan(context_lens, block_tables, block_size, out=None):
    """The work split of ``paged_decode_attention`` for one decode step, made once for all layers (they share the
    lengths and the block tables).  Returns an int32 tensor to pass as ``plan=``; ``out`` re-uses one (a captured
    graph keeps its pointer)."""
    lib = _lib.load()
    _need(context_lens, torch.int32, "context_lens"); _need(block_tables, torch.int32, "block_tables")
    assert block_tables.stride(1) == 1 and context_lens.is_contiguous()
    nbytes = lib.tlf_paged_decode_plan_bytes()
    plan = out if out is not None else torch.empty(nbytes // 4, dtype=torch.int32, device=context_lens.device)
    assert plan.dtype == torch.int32 and plan.numel() * 4 >= nbytes and plan.is_contiguous()
    check(lib.tlf_paged_decode_plan(context_lens.data_ptr(), block_tables.data_ptr(), block_tables.stride(0),
                                    context_lens.numel(), int(block_size), block_tables.shape[1], plan.data_ptr(),
                                    plan.numel() * 4, _stream()), "tlf_paged_decode_plan")
    return plan


def paged_decode_attention(q, k_cache, v_cache, context_lens, block_tables, scale,
                           k_scale=None, v_scale=None, plan=None):
    """``q [B, Hq, Dh]`` -> ``[B, Hq*Dh]``; caches ``[nblk, bs, Hkv, Dh]``.  ``plan``: the output of
    ``paged_decode_plan`` for these lengths and tables (same bits, a shorter start)."""
    lib = _lib.load()
    _need(q, BF16, "q"); _need(context_lens, torch.int32, "context_lens")
    _need(block_tables, torch.int32, "block_tables")
    B, Hq, Dh = q.shape
    assert q.stride(2) == 1 and q.stride(1) == Dh
    nblk, bs, Hkv, _ = k_cache.shape
    assert k_cache.is_contiguous() and v_cache.is_contiguous() and block_tables.stride(1) == 1
    maxb = block_tables.shape[1]
    out = torch.empty(B, Hq * Dh, dtype=BF16, device=q.device)
    # sized for the largest batch so that one buffer serves every call (graph capture keeps its pointer)
    nbytes = lib.tlf_paged_decode_attn_workspace_bytes(max(B, 1024), Hq, Dh, maxb, bs)
    ws = _workspace(nbytes, q.device, "decode")
    args = (q.data_ptr(), q.stride(0), k_cache.data_ptr(), v_cache.data_ptr(), kv_dtype_code(k_cache),
            k_scale.data_ptr() if k_scale is not None else None,
            v_scale.data_ptr() if v_scale is not None else None,
            block_tables.data_ptr(), block_tables.stride(0), context_lens.data_ptr(), out.data_ptr(),
            B, Hq, Hkv, Dh, bs, maxb, nblk, float(scale), ws.data_ptr(), ws.numel())
    if plan is None:
        check(lib.tlf_paged_decode_attn(*args, _stream()), "tlf_paged_decode_attn")
    else:
        assert plan.dtype == torch.int32 and plan.device == q.device
        check(lib.tlf_paged_decode_attn_planned(*args, plan.data_ptr(), _stream()), "tlf_paged_decode_attn_planned")
    return out


# ------------------------------------------------------------------ a4
def varlen_prefill_attention(q, k, v, cu_seqlens_q, cu_seqlens_k, max_seqlen_q, scale,
                             block_tables=None, k_scale=None, v_scale=None):
    """``q [Sq, Hq, Dh]``; ``k``/``v`` packed ``[Sk, Hkv, Dh]`` or the paged caches with ``block_tables``."""
    lib = _lib.load()
    _need(q, BF16, "q"); _need(cu_seqlens_q, torch.int32, "cu_seqlens_q")
    _need(cu_seqlens_k, torch.int32, "cu_seqlens_k")
    Sq, Hq, Dh = q.shape
    assert q.stride(2) == 1 and q.stride(1) == Dh
    out = torch.empty(Sq, Hq * Dh, dtype=BF16, device=q.device)
    nseq = cu_seqlens_q.numel() - 1
    if block_tables is None:
        _need(k, BF16, "k"); _need(v, BF16, "v")
        Hkv = k.shape[1]
        assert k.stride(2) == 1 and k.stride(1) == Dh and v.stride(2) == 1 and v.stride(1) == Dh
        ks, vs, bs, nblk, kvd = k.stride(0), v.stride(0), 0, 0, KV_BF16
        btp, bts = None, 0
    else:
        _need(block_tables, torch.int32, "block_tables")
        nblk, bs, Hkv, _ = k.shape
        assert k.is_contiguous() and v.is_contiguous()
        ks = vs = Hkv * Dh
        kvd = kv_dtype_code(k)
        btp, bts = block_tables.data_ptr(), block_tables.stride(0)
    check(lib.tlf_varlen_prefill_attn(
        q.data_ptr(), q.stride(0), k.data_ptr(), ks, v.data_ptr(), vs, kvd,
        k_scale.data_ptr() if k_scale is not None else None,
        v_scale.data_ptr() if v_scale is not None else None,
        cu_seqlens_q.data_ptr(), cu_seqlens_k.data_ptr(), btp, bts, out.data_ptr(), nseq,
        int(max_seqlen_q), Hq, Hkv, Dh, bs, nblk, float(scale), _stream()), "tlf_varlen_prefill_attn")
    return out
