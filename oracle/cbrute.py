"""ctypes loader for ``oracle/bruteforce.c`` (TEST INFRASTRUCTURE ONLY).

``build()`` compiles the C file with gcc into ``oracle/_build/``; the numpy
wrappers below call it.  Used by the CPU tests to pin ``sana_oracle``.
"""
from __future__ import annotations

import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_SRC = os.path.join(_HERE, "bruteforce.c")
_OUT = os.path.join(_HERE, "_build", "libbruteforce.so")
_lib = None


def build(force: bool = False) -> str:
    os.makedirs(os.path.dirname(_OUT), exist_ok=True)
    if force or not os.path.exists(_OUT) or os.path.getmtime(_OUT) < os.path.getmtime(_SRC):
        subprocess.check_call(["gcc", "-O2", "-shared", "-fPIC", "-o", _OUT, _SRC, "-lm"])
    return _OUT


def lib():
    global _lib
    if _lib is None:
        _lib = ctypes.CDLL(build())
    return _lib


def _p(a):
    return a.ctypes.data_as(ctypes.c_void_p)


def relu_attention(q, k, v, eps, chunk_of=None):
    """q, k, v: float64 [BH, N, d] token-major.  Returns [BH, N, d]."""
    q, k, v = (np.ascontiguousarray(t, dtype=np.float64) for t in (q, k, v))
    BH, N, d = q.shape
    out = np.empty_like(q)
    co = None if chunk_of is None else np.ascontiguousarray(chunk_of, dtype=np.int32)
    lib().brute_relu_attention(_p(q), _p(k), _p(v), None if co is None else _p(co),
                               ctypes.c_double(eps), BH, N, d, _p(out))
    return out


def relu_attention_rope(q, k, v, freqs, eps, chunk_of=None):
    """Rotary family: q, k, v float64 [BH, N, d]; freqs complex [N, d/2] (per-token factors
    of the channel pairs, numerator only).  Returns [BH, N, d]."""
    q, k, v = (np.ascontiguousarray(t, dtype=np.float64) for t in (q, k, v))
    BH, N, d = q.shape
    freqs = np.asarray(freqs).reshape(N, d // 2)
    f_re = np.ascontiguousarray(freqs.real, dtype=np.float64)
    f_im = np.ascontiguousarray(freqs.imag, dtype=np.float64)
    out = np.full_like(q, np.nan)
    co = None if chunk_of is None else np.ascontiguousarray(chunk_of, dtype=np.int32)
    lib().brute_relu_attention_rope(_p(q), _p(k), _p(v), _p(f_re), _p(f_im), None if co is None else _p(co),
                                    ctypes.c_double(eps), BH, N, d, _p(out))
    return out


def attention_state(k, v):
    """k, v: float64 [BH, N, d].  Returns [BH, d+1, d]."""
    k, v = (np.ascontiguousarray(t, dtype=np.float64) for t in (k, v))
    BH, N, d = k.shape
    out = np.empty((BH, d + 1, d), dtype=np.float64)
    lib().brute_attention_state(_p(k), _p(v), BH, N, d, _p(out))
    return out


def dwconv_gate(u, w, b):
    """u: [BT, H, W, 2C]; w: [2C, 3, 3]; b: [2C].  Returns [BT, H, W, C]."""
    u, w, b = (np.ascontiguousarray(t, dtype=np.float64) for t in (u, w, b))
    BT, H, W, C2 = u.shape
    out = np.empty((BT, H, W, C2 // 2), dtype=np.float64)
    lib().brute_dwconv_gate(_p(u), _p(w), _p(b), BT, H, W, C2 // 2, _p(out))
    return out
