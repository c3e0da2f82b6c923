"""ctypes binding of ``libsana_hip.so`` (the C ABI declared in ``include/sana_hip.h``).

The library is built in-tree by ``python -m sana_amd.build``.  There is no CPU
or stock-op fallback behind these calls: a missing library raises.
"""
from __future__ import annotations

import ctypes
import os
from ctypes import c_float, c_int, c_int64, c_size_t, c_void_p

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libsana_hip.so")

DT_F32, DT_BF16, DT_F16 = 0, 1, 2
EPI_NONE, EPI_BIAS, EPI_BIAS_SILU = 0, 1, 2

# name -> (restype, argtypes); must list every symbol include/sana_hip.h declares
SIGNATURES = {
    "sana_hip_abi_version": (c_int, []),
    "sana_hip_strerror": (ctypes.c_char_p, [c_int]),
    "sana_hip_linattn_workspace_bytes": (c_size_t, [c_int, c_int, c_int, c_int, c_int, c_int]),
    "sana_hip_linattn_state": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_size_t,
                                       c_int, c_int, c_int, c_int, c_int64, c_int64,
                                       c_void_p, c_int, c_int, c_int, c_int, c_void_p]),
    "sana_hip_linattn_chunk_scan": (c_int, [c_void_p, c_int, c_int, c_int, c_int, c_void_p]),
    "sana_hip_linattn_apply": (c_int, [c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int,
                                       c_int64, c_int64, c_int64, c_int64,
                                       c_void_p, c_int, c_int, c_float, c_int, c_int, c_void_p]),
    "sana_hip_qk_rms": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int64, c_int64,
                                c_float, c_int, c_void_p]),
    "sana_hip_linattn_state_pre": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_size_t,
                                           c_int, c_int, c_int, c_int, c_int64, c_int64,
                                           c_void_p, c_int, c_int, c_int, c_int,
                                           c_void_p, c_void_p, c_void_p, c_void_p]),
    "sana_hip_litela_state": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_size_t,
                                      c_int, c_int, c_int, c_int, c_int64, c_int64, c_int,
                                      c_void_p, c_void_p, c_void_p, c_void_p]),
    "sana_hip_litela_apply": (c_int, [c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int,
                                      c_int64, c_int64, c_int64, c_int64, c_float, c_int, c_int,
                                      c_void_p, c_void_p, c_void_p, c_void_p]),
    "sana_hip_linattn_state_noalloc": (c_int, [c_void_p, c_void_p, c_void_p,
                                               c_int, c_int, c_int, c_int, c_int64, c_int64,
                                               c_void_p, c_int, c_int, c_int, c_int,
                                               c_void_p, c_void_p, c_void_p, c_void_p]),
    "sana_hip_linattn_apply_pre": (c_int, [c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int,
                                           c_int64, c_int64, c_int64, c_int64,
                                           c_void_p, c_int, c_int, c_float, c_int, c_int,
                                           c_void_p, c_void_p, c_void_p, c_void_p]),
    "sana_hip_dwconv3x3_silu_gate": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p,
                                             c_int, c_int, c_int, c_int, c_int, c_int, c_void_p]),
    "sana_hip_gemm_workspace_bytes": (c_size_t, [c_int, c_int, c_int]),
    "sana_hip_gemm_bf16": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int,
                                   c_int64, c_int64, c_int64, c_int, c_void_p, c_size_t, c_void_p]),
    "sana_hip_gemm_f16": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int,
                                  c_int64, c_int64, c_int64, c_int, c_void_p, c_size_t, c_void_p]),
    "sana_hip_gemm_gate_residual_f16": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
                                                c_int, c_int, c_int, c_int64, c_int64, c_int64, c_int64,
                                                c_int, c_int64, c_void_p, c_size_t, c_void_p]),
    "sana_hip_gemm_w8a16": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int,
                                    c_int64, c_int64, c_int64, c_int, c_void_p, c_size_t, c_void_p]),
    "sana_hip_dequant_w8": (c_int, [c_void_p, c_void_p, c_void_p, c_int, c_int, c_int64, c_int64, c_void_p]),
    "sana_hip_tconv_residual": (c_int, [c_void_p, c_void_p, c_void_p, c_int, c_int, c_int,
                                        c_int64, c_int64, c_void_p, c_int64, c_int64, c_int64, c_void_p]),
    "sana_hip_gemm_gate_residual": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
                                            c_int, c_int, c_int, c_int64, c_int64, c_int64, c_int64,
                                            c_int, c_int64, c_void_p, c_size_t, c_void_p]),
    "sana_hip_qkv_state_rows": (c_int, [c_int, c_int, c_void_p, c_int]),
    "sana_hip_gemm_qkv_state_workspace_bytes": (c_size_t, [c_int, c_int, c_int]),
    "sana_hip_gemm_qkv_state": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_size_t,
                                        c_int, c_int, c_int, c_int, c_int64, c_int64, c_int64, c_void_p]),
    "sana_hip_add_layernorm_modulate": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int64,
                                                c_int, c_int64, c_int64, c_int64, c_int64, c_int, c_int64, c_float,
                                                c_int, c_void_p]),
    "sana_hip_gate_residual": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_int64, c_int, c_int64, c_int64,
                                       c_int64, c_int, c_int64, c_int, c_void_p]),
    "sana_hip_cross_attention": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int,
                                         c_int64, c_int64, c_int64, c_int64, c_float, c_void_p]),
    "sana_hip_layernorm_modulate": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_int64, c_int,
                                            c_int64, c_int64, c_int, c_int64, c_float, c_int, c_void_p]),
}

_lib = None


class SanaHipError(RuntimeError):
    pass


def load() -> ctypes.CDLL:
    """Load the library once; raise (never fall back) when it is absent."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise SanaHipError(
                f"{LIB_PATH} is missing: build it with `python -m sana_amd.build` "
                "(there is no fallback path for the HIP kernels)")
        lib = ctypes.CDLL(LIB_PATH)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(lib, name)
            fn.restype = res
            fn.argtypes = args
        _lib = lib
    return _lib


def check(code: int, what: str) -> None:
    if code != 0:
        msg = load().sana_hip_strerror(code).decode()
        raise SanaHipError(f"{what} failed with code {code}: {msg}")
