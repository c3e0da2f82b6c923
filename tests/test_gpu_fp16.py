"""GPU parity of the fp16 instances: the hand-written GEMM on v_mfma_f32_16x16x32_f16, the fused seams in half, and a
whole block of an fp16 model (the released Sana-600M configuration is fp16:
configs/sana_config/1024ms/Sana_600M_img1024.yaml:22) against the fp64 oracle."""
import logging

import pytest
import torch
import torch.nn.functional as F

import sana_amd as S
from oracle import sana_oracle as O
from sana_amd import ops

pytestmark = pytest.mark.gpu


def rel_l2(a, b):
    return ((a.double() - b.double()).norm() / b.double().norm()).item()


GEMM_SHAPES = [
    (4096, 2880 * 2, 1152),   # cfg2 inverted conv: 256-wide pipelined tiles
    (4096, 1152, 2880),       # cfg2 point conv: 192-wide tiles
    (1024, 2240, 5600),       # split-k
    (300, 72, 96),            # ragged rows and channels
    (260, 520, 136),          # K % 16 != 0: the generic kernel
    (129, 1000, 208),         # k tail of one k-step
    (1024, 2240, 2240),       # the 128 x 128 kernel
    (512, 11200, 2240),       # 128-wide tiles of the pipelined kernel
    (16384, 2240, 2240),      # cfg3 proj
]


def _gemm_ref(a, w, bias, epilogue):
    y = a.double() @ w.double().T
    if bias is not None:
        y = y + bias.double()
    if epilogue == "bias_silu":
        y = F.silu(y.half().double())   # the reference rounds the conv output to the io dtype, then applies SiLU
    return y


@pytest.mark.parametrize("M,N,K", GEMM_SHAPES)
@pytest.mark.parametrize("epilogue", [None, "bias", "bias_silu"])
def test_gemm_f16_matches_oracle(cuda, M, N, K, epilogue):
    g = torch.Generator().manual_seed(M + N + K)
    a = torch.randn(M, K, generator=g).half()
    w = (torch.randn(N, K, generator=g) * 0.05).half()
    bias = (torch.randn(N, generator=g) * 0.5).half() if epilogue else None
    ref = _gemm_ref(a, w, bias, epilogue)
    y = ops.gemm_bf16(a.to(cuda), w.to(cuda), None if bias is None else bias.to(cuda), epilogue)
    assert y.shape == (M, N) and y.dtype == torch.float16
    assert rel_l2(y.cpu(), ref) <= 6e-4          # half output rounding alone is ~2.8e-4
    err = (y.cpu().double() - ref).abs()
    assert (err > 2e-3 + 2 ** -9 * ref.abs()).sum().item() == 0   # a flipped rounding of the pre-activation + the output rounding


def test_gemm_f16_exact_on_integer_inputs(cuda):
    """Small-integer operands: every product and partial sum is exact, so the result is bit for bit the integer
    matrix product whatever the tile plan (pipelined, 128 x 128, generic, split-k)."""
    g = torch.Generator().manual_seed(3)
    for M, N, K in [(512, 512, 256), (200, 136, 1024), (260, 520, 136), (1024, 2240, 5600)]:
        a = torch.randint(-3, 4, (M, K), generator=g).half()
        w = torch.randint(-2, 3, (N, K), generator=g).half()
        ref = (a.double() @ w.double().T)
        assert ref.abs().max() <= 2048          # integers up to 2048 are exact in half
        y = ops.gemm_bf16(a.to(cuda), w.to(cuda))
        assert torch.equal(y.cpu().double(), ref)


@pytest.mark.parametrize("B,Ntok,C,K", [(1, 4096, 1152, 1152), (2, 1024, 2240, 5600), (3, 100, 96, 240),
                                        (7, 20, 96, 128), (2, 512, 1152, 1152)])
def test_gemm_gate_residual_f16_matches_stock_op_chain(cuda, B, Ntok, C, K):
    g = torch.Generator().manual_seed(B + K)
    a = torch.randn(B, Ntok, K, generator=g).half().to(cuda)
    w = (torch.randn(C, K, generator=g) * 0.03).half().to(cuda)
    bias = (torch.randn(C, generator=g) * 0.1).half().to(cuda)
    mod = (torch.randn(B, 6, C, generator=g) * 0.5).half().to(cuda)
    gate = mod[:, 2:3]
    res = torch.randn(B, Ntok, C, generator=g).half().to(cuda)
    out = ops.gemm_gate_residual(a, w, bias, gate, res)
    assert out.dtype == torch.float16
    y = ops.gemm_bf16(a.view(-1, K), w, bias, "bias").view(B, Ntok, C)
    assert torch.equal(out, res + gate * y)       # the reference's op chain in half: linear -> gate * y -> x + (.)
    ref = res.double() + gate.double() * (a.double() @ w.double().T + bias.double())
    assert rel_l2(out, ref) <= 6e-4


@pytest.mark.parametrize("B,Ntok,C", [(4, 1024, 1152), (2, 77, 96), (1, 2048, 2240)])
def test_seams_f16_match_stock_op_chain(cuda, B, Ntok, C):
    g = torch.Generator().manual_seed(C)
    x = (torch.randn(B, Ntok, C, generator=g) * 2 + 0.3).half().to(cuda)
    y = torch.randn(B, Ntok, C, generator=g).half().to(cuda)
    mod = (torch.randn(B, 6, C, generator=g) * 0.3).half().to(cuda)
    shift, scale, gate = mod[:, 0:1], mod[:, 1:2], mod[:, 2:3]
    out = ops.layernorm_modulate(x, scale, shift, 1e-6)
    assert out.dtype == torch.float16
    ref64 = F.layer_norm(x.double(), (C,), eps=1e-6) * (1 + scale.double()) + shift.double()
    assert rel_l2(out, ref64) <= 6e-4
    chain = F.layer_norm(x, (C,), eps=1e-6) * (1 + scale) + shift      # stock half chain (four roundings)
    diff = (out.float() - chain.float()).abs()
    mag = chain.float().abs() + shift.float().abs()
    assert (diff > 2 ** -9 * mag + 1e-6).sum().item() == 0
    assert (diff == 0).float().mean().item() > 0.97
    total, out2 = ops.add_layernorm_modulate(x, y, scale, shift, 1e-6)
    assert torch.equal(total, x + y) and torch.equal(out2, ops.layernorm_modulate(x + y, scale, shift, 1e-6))
    assert torch.equal(ops.gate_residual(y, gate, x), x + gate * y)


def test_fp16_block_runs_the_hand_written_kernels_and_matches_the_oracle(cuda, caplog):
    """cfg2's block as an fp16 model: no linear / 1x1 conv or seam leaves for a stock op (only the cross-attention,
    which is stock outside bf16, may log), and the output is within the half-precision tolerance of the fp64 oracle."""
    C, heads, B, H = 1152, 16, 4, 32
    N = H * H
    ob = O.init_block_(O.SanaMSBlock(C, heads, mlp_ratio=2.5, attn_type="linear", ffn_type="glumbconv",
                                     linear_head_dim=32), 5)
    g = torch.Generator().manual_seed(11)
    x = torch.randn(B, N, C, generator=g)
    y = torch.randn(B, 300, C, generator=g)
    t = torch.randn(B, 6 * C, generator=g) * 0.02
    hb = S.SanaMSBlock(C, heads, mlp_ratio=2.5, attn_type="linear", ffn_type="glumbconv", linear_head_dim=32)
    hb.load_state_dict(ob.state_dict())
    hb = hb.half().to(cuda).eval()
    # the oracle in fp64 on the half-rounded weights and inputs
    ob = ob.half().double().eval()
    ob.attn.fp32_attention = True
    with torch.no_grad():
        ref = ob(x.half().double(), y.half().double(), t.half().double(), None, (H, H))
    S.modules._stock_paths_seen.clear()
    with caplog.at_level(logging.WARNING, logger="sana_amd"), torch.no_grad():
        out = hb(x.half().to(cuda), y.half().to(cuda), t.half().to(cuda), None, (H, H))
    assert out.dtype == torch.float16
    logged = [r.getMessage() for r in caplog.records]
    assert not any("linear / 1x1 conv" in m or "seams" in m or "gated residual" in m for m in logged), logged
    err = (out.cpu().double() - ref).abs()
    assert rel_l2(out.cpu(), ref) <= 2e-3
    assert (err > 2e-2).sum().item() == 0
