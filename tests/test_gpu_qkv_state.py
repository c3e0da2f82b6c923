"""The qkv projection with phase 1 of the linear attention in its epilogue (``sana_hip_gemm_qkv_state``): q against
the plain GEMM (bit-identical: same products in the same order), the state against the fp64 oracle on the k / v the
unfused path would store, and against the unfused pair of launches (same values, another fp32 summation order)."""
import pytest
import torch

from oracle import sana_oracle as O
from sana_amd import ops

pytestmark = pytest.mark.gpu


def rel_l2(a, b):
    return ((a.double() - b.double()).norm() / b.double().norm()).item()


def _case(B, N, C, heads, with_bias, seed, cuda):
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(B, N, C, generator=g).bfloat16().to(cuda)
    w = (torch.randn(3 * C, C, generator=g) * C ** -0.5).bfloat16().to(cuda)
    b = (torch.randn(3 * C, generator=g) * 0.5).bfloat16().to(cuda) if with_bias else None
    return x, w, b


CASES = [
    # B, N, C, heads, bias
    (1, 256, 64, 2, False),       # one token tile, half a k / v tile (two dummy heads)
    (2, 512, 96, 3, True),        # odd head count, batch boundary between token tiles
    (4, 1024, 1152, 36, True),    # cfg2 attention shape: q region padded 1152 -> 1280
    (1, 16384, 2240, 70, False),  # cfg3: 64 partial states per head
    (16, 1024, 2240, 70, False),  # 1024 px, B = 16
    (1, 4100, 2240, 70, False),   # one batch entry, no bias: a ragged last token tile (4 rows of 256 exist)
    (1, 300, 64, 2, False),
]


@pytest.mark.parametrize("B,N,C,heads,with_bias", CASES)
def test_fused_qkv_state_matches_the_unfused_pair_and_the_oracle(cuda, B, N, C, heads, with_bias):
    x, w, b = _case(B, N, C, heads, with_bias, 11 + N + C, cuda)
    wt, bt = ops.tile_qkv_weight(w, b, heads)
    print(f"gemm_qkv_state B={B} N={N} C={C} heads={heads} bias={with_bias}", flush=True)
    q, state = ops.gemm_qkv_state(x, wt, bt, heads)
    qkv = ops.gemm_bf16(x.view(B * N, C), w, b, "bias" if with_bias else None).view(B, N, 3, C)
    assert torch.equal(q, qkv[:, :, 0])
    ref_state = ops.linattn_state(qkv[:, :, 1], qkv[:, :, 2])
    assert state.shape == ref_state.shape
    kk = qkv[:, :, 1].double().view(B, N, heads, 32).permute(0, 2, 3, 1).cpu()     # [B, h, d, N]
    vv = qkv[:, :, 2].double().view(B, N, heads, 32).permute(0, 2, 3, 1).cpu()
    _, oracle_state = O.relu_linear_attention(kk, kk.transpose(-1, -2), vv, 1e-15, return_state=True)
    oracle_state = oracle_state.reshape(ref_state.shape)
    assert rel_l2(state.cpu(), oracle_state) <= 1e-5
    assert rel_l2(ref_state.cpu(), oracle_state) <= 1e-5
    err = (state.cpu().double() - oracle_state).abs().max().item()
    assert err <= 2e-5 * oracle_state.abs().max().item(), err
    # and the attention output from the fused state
    out = ops.linattn_apply(q, state, 1e-8)
    ref = ops.linattn_apply(qkv[:, :, 0], ref_state, 1e-8)
    assert rel_l2(out.cpu(), ref.cpu()) <= 1e-3


def test_fused_qkv_state_is_deterministic_and_rejects_other_shapes(cuda):
    x, w, b = _case(2, 768, 160, 5, True, 5, cuda)
    wt, bt = ops.tile_qkv_weight(w, b, 5)
    q1, s1 = ops.gemm_qkv_state(x, wt, bt, 5)
    q2, s2 = ops.gemm_qkv_state(x, wt, bt, 5)
    assert torch.equal(q1, q2) and torch.equal(s1, s2)
    with pytest.raises(ops.SanaHipError):
        ops.gemm_qkv_state(x[:, :700], wt, bt, 5)              # N % 256 != 0 with two batch entries
    with pytest.raises(ops.SanaHipError):
        ops.gemm_qkv_state(x[:1, :700], wt, bt, 5)             # ... and with one, but a bias
    q3, s3 = ops.gemm_qkv_state(x[:1, :700].contiguous(), wt, None, 5)   # one entry, no bias: taken
    assert q3.shape == (1, 700, 160) and torch.isfinite(s3).all()
    with pytest.raises(ops.SanaHipError):
        ops.gemm_qkv_state(x, wt[:-256], bt, 5)                # a weight that is not the tiled layout of these shapes
    with pytest.raises(ops.SanaHipError):
        ops.gemm_qkv_state(x, wt, bt, 4)                       # C != 32 * heads
