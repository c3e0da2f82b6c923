"""CPU checks of the boundary: the library loads and exports every symbol the
header declares, argument validation works without touching a GPU."""
import ctypes
import os
import re

import pytest

from sana_amd import _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared_symbols():
    text = open(os.path.join(ROOT, "include", "sana_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(sana_hip_\w+)\s*\(", text)))


def test_library_is_built():
    assert os.path.exists(_lib.LIB_PATH), "run `python -m sana_amd.build` first"


def test_exports_every_declared_symbol():
    lib = ctypes.CDLL(_lib.LIB_PATH)
    declared = _declared_symbols()
    assert len(declared) >= 9
    for name in declared:
        assert hasattr(lib, name), f"{name} declared in include/sana_hip.h but not exported"
    assert sorted(_lib.SIGNATURES) == declared, "python signature table out of sync with the header"


def test_version_and_strerror():
    lib = _lib.load()
    assert lib.sana_hip_abi_version() == 8
    assert b"aligned" in lib.sana_hip_strerror(-3)
    assert b"unknown" in lib.sana_hip_strerror(-99)


def test_argument_validation_needs_no_gpu():
    lib = _lib.load()
    # null pointers / bad sizes are rejected before any launch
    assert lib.sana_hip_linattn_state(None, None, None, None, 0, 1, 16, 1, 32, 0, 32, None, 1, 16, 0, 1, None) == -1
    assert lib.sana_hip_linattn_state(16, 16, 16, None, 0, 1, 16, 1, 64, 0, 64, None, 1, 16, 0, 1, None) == -2  # d != 32
    assert lib.sana_hip_linattn_state(16, 16, 16, None, 0, 1, 16, 1, 32, 0, 32, None, 1, 16, 0, 7, None) == -6  # dtype
    assert lib.sana_hip_linattn_state(16, 18, 16, None, 0, 1, 16, 1, 32, 0, 32, None, 1, 16, 0, 1, None) == -3  # align
    assert lib.sana_hip_linattn_apply(16, 16, 16, 1, 16, 1, 32, 0, 32, 0, 32, None, 1, 16, 1e-8, 1, 2, None) == -6
    # head_dim 112: bf16 only (f16 for phase 1), needs its workspace, 32-bit byte offsets inside a batch entry
    F32, BF16, F16 = 0, 1, 2
    assert lib.sana_hip_linattn_state(16, 16, 16, 16, 1 << 30, 1, 16, 1, 112, 0, 112, None, 1, 16, 0, F32, None) == -6
    assert lib.sana_hip_linattn_state(16, 16, 16, None, 0, 1, 16, 1, 112, 0, 112, None, 1, 16, 0, BF16, None) == -4
    assert lib.sana_hip_linattn_state(16, 16, 16, 16, 1 << 30, 1, 1 << 20, 1, 112, 0, 1 << 12, None, 1, 1 << 20, 0,
                                      BF16, None) == -2
    assert lib.sana_hip_linattn_state(16, 16, 16, 16, 1 << 30, 1, 16, 1, 112, 0, 96, None, 1, 16, 0, BF16, None) == -1
    assert lib.sana_hip_linattn_apply(16, 16, 16, 1, 16, 1, 112, 0, 112, 0, 112, None, 1, 16, 1e-8, F16, F16, None) == -6
    assert lib.sana_hip_dwconv3x3_silu_gate(16, 16, None, 16, 1, 4, 4, 3, 1, 1, None) == -2  # odd Ch
    assert lib.sana_hip_gemm_bf16(16, 16, None, 16, 8, 8, 20, 24, 24, 8, 0, None, 0, None) == -2      # K % 8
    assert lib.sana_hip_gemm_bf16(16, 16, None, 16, 8, 8, 32, 32, 32, 8, 1, None, 0, None) == -1      # bias epilogue, no bias
    assert lib.sana_hip_gemm_w8a16(16, 16, None, None, 16, 8, 8, 32, 32, 32, 8, 0, None, 0, None) == -1  # no scale
    # temporal conv: C % 64, odd taps, the centre tap must exist for every output row
    assert lib.sana_hip_tconv_residual(16, 16, 32, 64, 96, 3, 16, 80, None, 96, 288, 96, None) == -2
    assert lib.sana_hip_tconv_residual(16, 16, 32, 64, 64, 2, 16, 80, None, 64, 128, 64, None) == -1
    assert lib.sana_hip_tconv_residual(16, 16, 32, 64, 64, 3, 16, 64, None, 64, 192, 64, None) == -1
    assert lib.sana_hip_tconv_residual(16, 16, 32, 64, 64, 3, 16, 80, None, 64, 128, 64, None) == -1   # ldw < taps * C
    assert lib.sana_hip_tconv_residual(16, 16, 32, 64, 64, 1, 16, 80, 16, 64, 64, 64, None) == -1   # chunk flags need >= 3 taps


def test_workspace_query():
    lib = _lib.load()
    # 1.6B @ 16384 tokens: 70 heads -> splits of the token axis need partial states
    n = lib.sana_hip_linattn_workspace_bytes(1, 70, 32, 1, 16384, 1)
    assert n > 0 and n % (33 * 32 * 4) == 0
    # short sequences are never split (a split is at least 256 tokens): no workspace
    assert lib.sana_hip_linattn_workspace_bytes(16, 70, 32, 1, 256, 1) == 0
    assert lib.sana_hip_linattn_workspace_bytes(64, 70, 32, 4, 300, 1) == 0
    # head_dim 112 always goes through records of token ranges: 20 heads at the video shape -> 256 // 20 = 12 ranges
    # of 2752 tokens (a multiple of 64) per head, one record per (range, chunk) pair that occurs, indexed range + chunk
    assert lib.sana_hip_linattn_workspace_bytes(1, 20, 112, 1, 32760, 1) == 20 * 12 * 113 * 112 * 4
    # 21 chunks of 1560 tokens: the same ranges, 12 + 21 - 1 records
    assert lib.sana_hip_linattn_workspace_bytes(1, 20, 112, 21, 1560, 1) == 20 * 32 * 113 * 112 * 4
    assert lib.sana_hip_linattn_workspace_bytes(1, 20, 64, 1, 32760, 1) == 0   # no kernel for this head dim


def test_gemm_split_k_workspace_query():
    """Shapes with fewer output tiles than half the compute units (256 assumed without a device) are split
    along K through fp32 partial planes; shapes that fill the chip, short K loops and int8-only shapes are not."""
    lib = _lib.load()
    # one 1024 px image at Sana-1.6B: point conv 1024 x 2240 x 5600 -> 4 x 12 tiles of 256 x 192, 88 k-tiles, 5 ranges
    assert lib.sana_hip_gemm_workspace_bytes(1024, 2240, 5600) == 5 * 1024 * 2240 * 4
    # its proj GEMM (35 k-tiles): at most one range per 8 k-tiles
    assert lib.sana_hip_gemm_workspace_bytes(1024, 2240, 2240) == 4 * 1024 * 2240 * 4
    # 256 tokens through the proj GEMM (35 k-tiles): at most one range per 8 k-tiles
    assert lib.sana_hip_gemm_workspace_bytes(256, 2240, 2240) == 4 * 256 * 2240 * 4
    # not split: grids that fill the chip, wide N or short K (the partial planes would cost more than the loop saves)
    for M, N, K in ((16384, 2240, 5600), (16384, 11200, 2240), (1024, 11200, 2240), (1024, 6720, 2240),
                    (1024, 3456, 1152), (1024, 2240, 512), (0, 8, 64), (256, 2244, 5600)):
        assert lib.sana_hip_gemm_workspace_bytes(M, N, K) == 0, (M, N, K)


def test_ops_refuse_cpu_tensors():
    import torch
    from sana_amd import ops
    x = torch.zeros(1, 32, 32)
    with pytest.raises(_lib.SanaHipError):
        ops.linattn_state(x, x)


def test_qkv_state_row_map_is_a_layout_of_the_qkv_weight():
    """sana_hip_qkv_state_rows (host code): q rows first, padded to whole 256-row tiles; then per tile of four heads
    [K h | V h | K h+1 | V h+1] twice; every row of the [3C, C] weight exactly once, the rest -1."""
    import ctypes
    lib = _lib.load()
    for heads in (1, 2, 5, 36, 70):
        C = 32 * heads
        n = lib.sana_hip_qkv_state_rows(C, heads, None, 0)
        q_pad = (C + 255) // 256 * 256
        assert n == q_pad + (heads + 3) // 4 * 256
        buf = (ctypes.c_int32 * n)()
        assert lib.sana_hip_qkv_state_rows(C, heads, ctypes.cast(buf, ctypes.c_void_p), n) == n
        rows = list(buf)
        assert rows[:C] == list(range(C)) and all(r == -1 for r in rows[C:q_pad])
        live = sorted(r for r in rows if r >= 0)
        assert live == list(range(3 * C))
        for i in range(q_pad, n):
            loc = (i - q_pad) % 256
            head = 4 * ((i - q_pad) // 256) + 2 * (loc // 128) + (loc // 64) % 2
            want = -1 if head >= heads else (1 + (loc // 32) % 2) * C + 32 * head + loc % 32
            assert rows[i] == want
    assert lib.sana_hip_qkv_state_rows(100, 3, None, 0) < 0          # C != 32 * heads
    assert lib.sana_hip_qkv_state_rows(64, 2, ctypes.cast((ctypes.c_int32 * 4)(), ctypes.c_void_p), 4) < 0
    assert lib.sana_hip_gemm_qkv_state_workspace_bytes(2, 512, 3) == 2 * 3 * 2 * 33 * 32 * 4
    assert lib.sana_hip_gemm_qkv_state_workspace_bytes(2, 500, 3) == 0
    assert lib.sana_hip_gemm_qkv_state_workspace_bytes(1, 500, 3) == 3 * 2 * 33 * 32 * 4   # one entry: a ragged last tile


def test_gemm_qkv_state_refuses_bad_arguments_before_any_launch():
    """The argument checks of sana_hip_gemm_qkv_state run on the host before anything is launched: wrong calls
    return their error code on a machine without a GPU too (the pointers below are never dereferenced)."""
    lib = _lib.load()
    P, ws = 0x10000, 1 << 30                      # a 16-byte aligned non-null "pointer", an ample workspace size
    call = lambda *a: lib.sana_hip_gemm_qkv_state(*a, None)
    good = [P, P, None, P, P, P, ws, 2, 512, 96, 3, 96, 96, 96]   # A W bias Q state ws bytes B N C heads lda ldw ldq
    bad = lambda i, v: good[:i] + [v] + good[i + 1:]
    assert call(*bad(0, None)) == -1 and call(*bad(3, None)) == -1 and call(*bad(7, 0)) == -1     # SANA_ERR_ARG
    assert call(*bad(8, 500)) == -2 and call(*bad(10, 4)) == -2                                    # SANA_ERR_SHAPE
    one = [P, P, P, P, P, P, ws, 1, 500, 96, 3, 96, 96, 96]      # one batch entry, ragged N: refused with a bias only
    assert call(*one) == -2
    assert call(*bad(11, 64)) == -1                                                                # lda < C
    assert call(*bad(0, P + 2)) == -3 and call(*bad(12, 100)) == -3                                # SANA_ERR_ALIGN
    assert call(*bad(6, 1024)) == -4 and call(*bad(5, None)) == -4                                 # SANA_ERR_WORKSPACE
