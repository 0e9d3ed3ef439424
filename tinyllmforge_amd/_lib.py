"""ctypes binding of ``libtlf_hip.so`` (the C ABI declared in ``include/tlf_hip.h``).

The library is built in-tree by ``tinyllmforge_amd/csrc/build.py``.  There is no
fallback: if the shared object is missing or a call is rejected, an exception is
raised.
"""
from __future__ import annotations

import ctypes
import os
from ctypes import c_char_p, c_float, c_int32, c_int64, c_size_t, c_uint64, c_void_p

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libtlf_hip.so")

ABI_VERSION = 1
KV_BF16 = 0
KV_FP8_E4M3 = 1

_P, _I32, _I64, _F, _SZ = c_void_p, c_int32, c_int64, c_float, c_size_t

# name -> (restype, argtypes); mirrors include/tlf_hip.h declaration by declaration
SIGNATURES = {
    "tlf_version": (c_int32, []),
    "tlf_error_string": (c_char_p, [c_int32]),
    "tlf_device_info": (c_int32, [_P, _P]),
    "tlf_kernel_launches": (c_int64, []),
    "tlf_store_kvcache": (c_int32, [_P, _I64, _P, _I64, _P, _P, _P, _I32, _I32, _I64, _P]),
    "tlf_store_kvcache_fp8": (c_int32, [_P, _I64, _P, _I64, _P, _P, _P, _I32, _I32, _I32, _P, _P, _I64, _P]),
    "tlf_rmsnorm": (c_int32, [_P, _I64, _P, _P, _I32, _I32, _I32, _F, _P]),
    "tlf_add_rmsnorm": (c_int32, [_P, _P, _P, _P, _P, _I32, _I32, _F, _P]),
    "tlf_rope": (c_int32, [_P, _P, _I64, _P, _I64, _P, _P, _P, _I32, _I32, _I32, _I32, _I32, _P]),
    "tlf_qknorm_rope_store": (c_int32, [_P, _I64, _P, _P, _F, _P, _P, _I32, _P, _P, _P, _P, _P, _P,
                                        _I64, _I32, _P, _P, _I32, _I32, _I32, _I32, _P]),
    "tlf_silu_and_mul": (c_int32, [_P, _P, _I32, _I32, _P]),
    "tlf_argmax_workspace_bytes": (_SZ, [_I32, _I32]),
    "tlf_argmax": (c_int32, [_P, _I64, _P, _I32, _I32, _P, _SZ, _P]),
    "tlf_argmax_noalloc_max_rows": (c_int32, []),
    "tlf_argmax_noalloc": (c_int32, [_P, _I64, _P, _I32, _I32, _P]),
    "tlf_sample": (c_int32, [_P, _I64, _P, _P, _I32, _I32, c_uint64, c_uint64, _P, _SZ, _P]),
    "tlf_w8a16_packed_bytes": (_SZ, [_I32, _I32]),
    "tlf_w8a16_pack_weight": (c_int32, [_P, _P, _I32, _I32, _P]),
    "tlf_w8a16_gemm_workspace_bytes": (_SZ, [_I32, _I32, _I32]),
    "tlf_w8a16_gemm": (c_int32, [_P, _I64, _P, _P, _P, _I32, _I32, _I32, _P, _SZ, _P]),
    "tlf_bf16_gemm": (c_int32, [_P, _I64, _P, _P, _I32, _I32, _I32, _P, _SZ, _P]),
    "tlf_w8a16_gemm_silu_mul": (c_int32, [_P, _I64, _P, _P, _P, _I32, _I32, _I32, _P]),
    "tlf_bf16_gemm_silu_mul": (c_int32, [_P, _I64, _P, _P, _I32, _I32, _I32, _P]),
    "tlf_gemm_plan": (c_int32, [_I32, _I32, _I32, _I32, _P]),
    "tlf_gemm_add_rmsnorm_workspace_bytes": (_SZ, [_I32, _I32, _I32]),
    "tlf_gemm_argmax_workspace_bytes": (_SZ, [_I32, _I32, _I32]),
    "tlf_gemm_qknorm_rope_store_workspace_bytes": (_SZ, [_I32, _I32, _I32]),
    "tlf_w8a16_gemm_qknorm_rope_store": (c_int32, [_P, _I64, _P, _P, _P, _P, _F, _P, _P, _I32, _P, _P, _P, _P, _P, _P,
                                                   _I64, _I32, _P, _P, _I32, _I32, _I32, _I32, _I32, _P, _SZ, _P]),
    "tlf_bf16_gemm_qknorm_rope_store": (c_int32, [_P, _I64, _P, _P, _P, _F, _P, _P, _I32, _P, _P, _P, _P, _P, _P,
                                                  _I64, _I32, _P, _P, _I32, _I32, _I32, _I32, _I32, _P, _SZ, _P]),
    "tlf_bf16_gemm_argmax": (c_int32, [_P, _I64, _P, _P, _I32, _I32, _I32, _P, _SZ, _P]),
    "tlf_w8a16_gemm_add_rmsnorm": (c_int32, [_P, _I64, _P, _P, _P, _P, _P, _P, _I32, _I32, _I32, _F, _P, _SZ, _P]),
    "tlf_bf16_gemm_add_rmsnorm": (c_int32, [_P, _I64, _P, _P, _P, _P, _P, _I32, _I32, _I32, _F, _P, _SZ, _P]),
    "tlf_paged_decode_attn_workspace_bytes": (_SZ, [_I32, _I32, _I32, _I32, _I32]),
    "tlf_paged_decode_attn": (c_int32, [_P, _I64, _P, _P, _I32, _P, _P, _P, _I64, _P, _P,
                                        _I32, _I32, _I32, _I32, _I32, _I32, _I64, _F, _P, _SZ, _P]),
    "tlf_paged_decode_plan_bytes": (_SZ, []),
    "tlf_paged_decode_plan": (c_int32, [_P, _P, _I64, _I32, _I32, _I32, _P, _SZ, _P]),
    "tlf_paged_decode_attn_planned": (c_int32, [_P, _I64, _P, _P, _I32, _P, _P, _P, _I64, _P, _P,
                                                _I32, _I32, _I32, _I32, _I32, _I32, _I64, _F, _P, _SZ, _P, _P]),
    "tlf_varlen_prefill_attn": (c_int32, [_P, _I64, _P, _I64, _P, _I64, _I32, _P, _P, _P, _P, _P, _I64,
                                          _P, _I32, _I32, _I32, _I32, _I32, _I32, _I64, _F, _P]),
    "tlf_embedding": (c_int32, [_P, _P, _P, _I32, _I32, _I32, _P]),
    "tlf_probe_read": (c_int32, [_P, _SZ, _P, _P]),
    "tlf_probe_copy": (c_int32, [_P, _P, _SZ, _P]),
    "tlf_probe_mfma": (c_int32, [_P, c_int32, c_int32, _P]),
    "tlf_probe_mix": (c_int32, [_P, _SZ, _P, _SZ, c_int32, _P, _P]),
}


class TlfError(RuntimeError):
    pass


_lib = None


def load() -> ctypes.CDLL:
    """Load the shared library once; raise if it is absent or has the wrong ABI."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise TlfError(
            f"{LIB_PATH} not found: build it with `python tinyllmforge_amd/csrc/build.py` "
            "(there is no fallback path)")
    lib = ctypes.CDLL(LIB_PATH)
    for name, (res, args) in SIGNATURES.items():
        fn = getattr(lib, name)          # AttributeError if the symbol is not exported
        fn.restype = res
        fn.argtypes = args
    if lib.tlf_version() != ABI_VERSION:
        raise TlfError(f"ABI mismatch: library {lib.tlf_version()} != binding {ABI_VERSION}")
    _lib = lib
    return lib


def check(code: int, what: str) -> None:
    if code != 0:
        msg = load().tlf_error_string(code).decode()
        raise TlfError(f"{what} failed with code {code}: {msg}")
