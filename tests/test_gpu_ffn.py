"""GPU parity of the Mix-FFN kernels (depthwise+gate, GEMMs, W8A16) against the oracle."""
import pytest
import torch
import torch.nn.functional as F

from oracle import cbrute
from oracle import sana_oracle as O
from sana_amd import ops

pytestmark = pytest.mark.gpu


def rel_l2(a, b):
    return ((a.double() - b.double()).norm() / b.double().norm()).item()


def _dw_ref(u, w, b, Ch):
    """fp64 stock conv on the bf16-rounded values: dw -> split -> a * silu(g)."""
    x = u.double().permute(0, 3, 1, 2)
    t = F.conv2d(x, w.double().view(2 * Ch, 1, 3, 3), None if b is None else b.double(), padding=1, groups=2 * Ch)
    a, g = t[:, :Ch], t[:, Ch:]
    return (a * F.silu(g)).permute(0, 2, 3, 1)


@pytest.mark.parametrize("BT,H,W,Ch,dtype", [
    (4, 32, 32, 2880, torch.bfloat16),    # cfg2
    (1, 128, 128, 5600, torch.bfloat16),  # cfg3
    (2, 30, 52, 160, torch.bfloat16),     # cfg5 frame grid, ragged strips
    (1, 5, 7, 6, torch.bfloat16),
    (3, 1, 1, 2, torch.bfloat16),
    (1, 9, 3, 130, torch.float32),
    (1, 6, 11, 66, torch.float16),
])
def test_dwconv_gate_matches_oracle(cuda, BT, H, W, Ch, dtype):
    g = torch.Generator().manual_seed(H * W + Ch)
    u = torch.randn(BT, H, W, 2 * Ch, generator=g).to(dtype)
    w = (torch.randn(2 * Ch, 1, 3, 3, generator=g) * 0.3).to(dtype)
    b = (torch.randn(2 * Ch, generator=g) * 0.3).to(dtype)
    ref = _dw_ref(u, w, b, Ch)
    for round_ref in (False, True):
        y = ops.dwconv3x3_silu_gate(u.to(cuda), w.to(cuda), b.to(cuda), round_like_reference=round_ref)
        assert y.shape == (BT, H, W, Ch) and y.dtype == dtype
        tol = 1e-5 if dtype == torch.float32 else 1e-2
        assert rel_l2(y.cpu(), ref) <= tol
        if dtype == torch.bfloat16:
            err = (y.cpu().double() - ref).abs()
            assert (err <= 2e-2 + 2 ** -6 * ref.abs()).all()
    y = ops.dwconv3x3_silu_gate(u.to(cuda), w.to(cuda), None)
    ref = _dw_ref(u, w, None, Ch)
    # max-abs 2e-2 (north-star tolerance) plus a few units in the last place of the io dtype
    ulp = {torch.float32: 1e-5, torch.bfloat16: 2 ** -6, torch.float16: 2 ** -9}[dtype]
    floor = 1e-4 if dtype == torch.float32 else 2e-2
    assert ((y.cpu().double() - ref).abs() > floor + ulp * ref.abs()).sum().item() == 0


def test_dwconv_against_c_bruteforce(cuda):
    g = torch.Generator().manual_seed(1)
    BT, H, W, Ch = 2, 4, 5, 10
    u = torch.randn(BT, H, W, 2 * Ch, generator=g)
    w = torch.randn(2 * Ch, 3, 3, generator=g) * 0.3
    b = torch.randn(2 * Ch, generator=g) * 0.3
    ref = torch.from_numpy(cbrute.dwconv_gate(u.numpy(), w.numpy(), b.numpy()))
    y = ops.dwconv3x3_silu_gate(u.to(cuda), w.view(2 * Ch, 1, 3, 3).to(cuda), b.to(cuda), round_like_reference=False)
    assert rel_l2(y.cpu(), ref) <= 1e-5


def test_dwconv_reference_rounding_is_bitwise_on_exact_inputs(cuda):
    """With small-integer inputs and weights every fp32 partial sum is exact, so the
    kernel in round-like-reference mode must equal the stock bf16 op chain bit for bit."""
    g = torch.Generator().manual_seed(2)
    BT, H, W, Ch = 1, 8, 9, 64
    u = torch.randint(-3, 4, (BT, H, W, 2 * Ch), generator=g).bfloat16()
    w = torch.randint(-2, 3, (2 * Ch, 1, 3, 3), generator=g).bfloat16()
    b = torch.randint(-2, 3, (2 * Ch,), generator=g).bfloat16()
    t = F.conv2d(u.float().permute(0, 3, 1, 2), w.float(), b.float(), padding=1, groups=2 * Ch).bfloat16()
    a, gg = t[:, :Ch], t[:, Ch:]
    ref = (a * F.silu(gg)).permute(0, 2, 3, 1)
    y = ops.dwconv3x3_silu_gate(u.to(cuda), w.to(cuda), b.to(cuda), round_like_reference=True).cpu()
    # silu via exp2/rcp may differ from libm in the last fp32 bit, which can flip a bf16 rounding
    diff = (y.float() - ref.float()).abs()
    assert (diff <= 2 ** -7 * ref.float().abs() + 1e-30).all()
    assert (diff == 0).float().mean().item() > 0.97


GEMM_SHAPES = [
    (1024, 3456, 1152),   # qkv at 600M, one image of cfg2
    (4096, 5760, 1152),   # inverted conv, cfg2
    (4096, 1152, 2880),   # point conv, cfg2
    (16384, 2240, 2240),  # proj, cfg3
    (16384, 2240, 5600),  # point conv, cfg3 (K not a multiple of 64)
    (300, 72, 96),        # ragged everything
    (1, 8, 32),           # K < 64: the generic kernel
    (257, 264, 160),
    (513, 40, 64),        # a single k-tile
    (31, 24, 80),         # two k-tiles, the second with one k-step; fewer than 32 rows either side
    (260, 520, 136),      # K % 16 != 0: the generic kernel
    (129, 1000, 208),     # k tail of one k-step after three full tiles
    (1024, 2240, 2240),   # proj of one 1024 px image: the 128 x 128 kernel (144 tiles, one per CU)
    (520, 264, 1160),     # the 128 x 128 kernel with K % 16 != 0, ragged rows and channels, 19 k-tiles (not a multiple of 3)
    (200, 136, 1024),     # the 128 x 128 kernel, 16 k-tiles
]


def _gemm_ref(a, w, bias, epilogue):
    y = a.double() @ w.double().T
    if bias is not None:
        y = y + bias.double()
    if epilogue == "bias_silu":
        y = F.silu(y.bfloat16().double())   # the reference rounds the conv output, then applies SiLU
    return y


@pytest.mark.parametrize("M,N,K", GEMM_SHAPES)
@pytest.mark.parametrize("epilogue", [None, "bias", "bias_silu"])
def test_gemm_bf16_matches_oracle(cuda, M, N, K, epilogue):
    g = torch.Generator().manual_seed(M + N + K)
    a = torch.randn(M, K, generator=g).bfloat16()
    w = (torch.randn(N, K, generator=g) * 0.05).bfloat16()
    bias = (torch.randn(N, generator=g) * 0.5).bfloat16() if epilogue else None
    ref = _gemm_ref(a, w, bias, epilogue)
    y = ops.gemm_bf16(a.to(cuda), w.to(cuda), None if bias is None else bias.to(cuda), epilogue)
    assert y.shape == (M, N) and y.dtype == torch.bfloat16
    assert rel_l2(y.cpu(), ref) <= 4e-3          # bf16 output rounding alone is ~2e-3
    err = (y.cpu().double() - ref).abs()
    assert (err > 2e-2 + 2 ** -7 * ref.abs()).sum().item() == 0


def test_gemm_strided_views(cuda):
    """Row strides larger than the row length (slices of bigger buffers)."""
    g = torch.Generator().manual_seed(0)
    big_a = torch.randn(200, 320, generator=g).bfloat16().to(cuda)
    big_w = (torch.randn(136, 512, generator=g) * 0.1).bfloat16().to(cuda)
    a, w = big_a[:, 64:64 + 160], big_w[:, 128:128 + 160]
    out = torch.zeros(200, 400, dtype=torch.bfloat16, device=cuda)
    ops.gemm_bf16(a, w, out=out[:, 8:8 + 136])
    ref = a.double() @ w.double().T
    assert rel_l2(out[:, 8:144].cpu(), ref.cpu()) <= 4e-3
    assert out[:, :8].abs().max() == 0 and out[:, 144:].abs().max() == 0


@pytest.mark.parametrize("w8", [False, True])
def test_gemm_mixed_channel_tiling_is_bit_identical(cuda, w8):
    """qkv at 16384 tokens (N = 6720) runs as two launches: 24 tiles of 256 channels and 3 of 192.  Every output sums
    its k products in the same order whatever the tiling, so the first 256 rows -- which alone are one launch of one
    width -- must come out bit for bit the same; bias, SiLU, the gated residual and int8 weights ride along."""
    from sana_amd.modules import quantize_w8
    M, N, K = 16384, 6720, 192
    g = torch.Generator().manual_seed(9)
    a = torch.randn(M, K, generator=g).bfloat16().to(cuda)
    w = (torch.randn(N, K, generator=g) * 0.05).bfloat16().to(cuda)
    bias = (torch.randn(N, generator=g) * 0.5).bfloat16().to(cuda)
    if w8:
        wq, sc = quantize_w8(w)
        run = lambda x, epi: ops.gemm_w8a16(x, wq, sc, bias, epi, expand=False)
    else:
        run = lambda x, epi: ops.gemm_bf16(x, w, bias, epi)
    for epi in ("bias", "bias_silu"):
        whole, head = run(a, epi), run(a[:256], epi)
        assert torch.equal(whole[:256], head)
        # a tile row in the middle and the last one, against the same rows alone
        assert torch.equal(whole[8192:8448], run(a[8192:8448], epi))
        assert torch.equal(whole[-256:], run(a[-256:], epi))
    if not w8:
        ref = a[:512].double() @ w.double().T + bias.double()
        assert rel_l2(run(a, "bias")[:512].cpu(), ref.cpu()) <= 4e-3
        gate = (torch.randn(1, 1, N, generator=g) * 0.5).bfloat16().to(cuda)
        res = torch.randn(1, M, N, generator=g).bfloat16().to(cuda)
        whole = ops.gemm_gate_residual(a.view(1, M, K), w, bias, gate, res)
        head = ops.gemm_gate_residual(a[:256].view(1, 256, K), w, bias, gate, res[:, :256])
        assert torch.equal(whole[0, :256], head[0])


def test_gemm_128_wide_tiles_are_bit_identical_to_the_wider_ones(cuda):
    """1024 tokens x 6720 channels (qkv of one image) runs 128-wide tiles: 4 x 53 workgroups instead of 4 x 35 of 192
    channels.  The same rows inside a 16384-token call run the 256- / 192-wide tiles: same k order per output, so
    bit for bit the same; the int8-weight instances (also 128-wide here) as well; every epilogue kind."""
    from sana_amd.modules import quantize_w8
    M, N, K = 1024, 6720, 2240
    g = torch.Generator().manual_seed(19)
    big = torch.randn(16384, K, generator=g).bfloat16().to(cuda)
    a = big[5120:5120 + M]
    w = (torch.randn(N, K, generator=g) * 0.02).bfloat16()
    wq, sc = quantize_w8(w)
    w = (wq.float() * sc[:, None]).bfloat16().to(cuda)          # the dequantised weight: both routes see the same values
    bias = (torch.randn(N, generator=g) * 0.5).bfloat16().to(cuda)
    for epi in (None, "bias", "bias_silu"):
        b = bias if epi else None
        narrow = ops.gemm_bf16(a, w, b, epi)
        assert torch.equal(narrow, ops.gemm_bf16(big, w, b, epi)[5120:5120 + M]), epi
        assert torch.equal(narrow, ops.gemm_w8a16(a, wq.to(cuda), sc.to(cuda), b, epi, expand=False)), epi
    gate = (torch.randn(1, 1, N, generator=g) * 0.5).bfloat16().to(cuda)
    res = torch.randn(1, 16384, N, generator=g).bfloat16().to(cuda)
    narrow = ops.gemm_gate_residual(a.view(1, M, K), w, bias, gate, res[:, 5120:5120 + M])
    assert torch.equal(narrow[0], ops.gemm_gate_residual(big.view(1, 16384, K), w, bias, gate, res)[0, 5120:5120 + M])
    ref = a.double() @ w.double().T + bias.double()
    assert rel_l2(ops.gemm_bf16(a, w, bias, "bias").cpu(), ref.cpu()) <= 4e-3


def test_gemm_exact_on_integer_inputs(cuda):
    """Small integers: every product and partial sum is exact in fp32, the result is exact in bf16."""
    g = torch.Generator().manual_seed(3)
    a = torch.randint(-2, 3, (512, 320), generator=g).bfloat16()
    w = torch.randint(-1, 2, (264, 320), generator=g).bfloat16()
    y = ops.gemm_bf16(a.to(cuda), w.to(cuda)).cpu()
    assert torch.equal(y.float(), a.float() @ w.float().T)


@pytest.mark.parametrize("M,N,K", [(1024, 2240, 2240), (4096, 11200, 2240), (300, 72, 96), (16384, 2240, 5600),
                                   (40, 24, 64), (513, 264, 208), (9, 8, 48)])
@pytest.mark.parametrize("epilogue", [None, "bias_silu"])
def test_gemm_w8a16_equals_bf16_gemm_on_dequantised_weight(cuda, M, N, K, epilogue):
    g = torch.Generator().manual_seed(M + K)
    a = torch.randn(M, K, generator=g).bfloat16().to(cuda)
    w = torch.empty(N, K)
    torch.nn.init.trunc_normal_(w, std=0.02, generator=g)
    wq, s = O.quantize_w8(w.bfloat16())
    wd = O.dequantize_w8(wq, s)
    bias = (torch.randn(N, generator=g) * 0.5).bfloat16().to(cuda) if epilogue else None
    y16 = ops.gemm_bf16(a, wd.to(cuda), bias, epilogue)
    # both int8 routes -- conversion inside the GEMM's main loop, and the weight expanded to bf16 by a kernel of
    # its own in front of the bf16 GEMM -- reproduce (q.float()*s).bfloat16() exactly -> same kernel arithmetic
    y8 = ops.gemm_w8a16(a, wq.to(cuda), s.to(cuda), bias, epilogue, expand=False)
    assert torch.equal(y8, y16)
    assert torch.equal(ops.dequant_w8(wq.to(cuda), s.to(cuda)).cpu(), wd)
    assert torch.equal(ops.gemm_w8a16(a, wq.to(cuda), s.to(cuda), bias, epilogue, expand=True), y16)
    ref = _gemm_ref(a.cpu(), wd, None if bias is None else bias.cpu(), epilogue)
    assert rel_l2(y8.cpu(), ref) <= 4e-3


@pytest.mark.parametrize("M,N,K", [(1024, 2240, 5600),    # point conv of one 1024 px image: 4 k ranges
                                   (256, 2240, 2240),     # 4 ranges of 9, 9, 9 and 8 k-tiles
                                   (1000, 1152, 2880),    # ragged rows, 600M widths
                                   (300, 72, 1184),       # two tiles, k ranges of 10 and 9 k-tiles, a k tail of one k-step of 32
                                   (2048, 2240, 5600)])   # 2 ranges
def test_gemm_split_k(cuda, monkeypatch, M, N, K):
    """Shapes with too few output tiles run as split-k through the workspace: against the fp64 oracle to the same
    bounds as the fused path, against the unsplit kernel to fp32 summation-order noise, bit-identical between the
    bf16, int8 and gated-residual entry points (they share the plan), and exact on integer inputs."""
    from sana_amd import _lib
    assert _lib.load().sana_hip_gemm_workspace_bytes(M, N, K) > 0
    g = torch.Generator().manual_seed(M + N + K)
    a = torch.randn(M, K, generator=g).bfloat16().to(cuda)
    w = torch.empty(N, K)
    torch.nn.init.trunc_normal_(w, std=0.03, generator=g)
    wq, s = O.quantize_w8(w.bfloat16())
    wd = O.dequantize_w8(wq, s).to(cuda)
    bias = (torch.randn(N, generator=g) * 0.5).bfloat16().to(cuda)
    outs = {}
    for epilogue in (None, "bias", "bias_silu"):
        b = bias if epilogue else None
        y = ops.gemm_bf16(a, wd, b, epilogue)
        ref = _gemm_ref(a.cpu(), wd.cpu(), None if b is None else b.cpu(), epilogue)
        assert rel_l2(y.cpu(), ref) <= 4e-3
        assert ((y.cpu().double() - ref).abs() > 2e-2 + 2 ** -7 * ref.abs()).sum().item() == 0
        assert torch.equal(ops.gemm_w8a16(a, wq.to(cuda), s.to(cuda), b, epilogue, expand=False), y)
        outs[epilogue] = y
    mod = (torch.randn(1, 6, N, generator=g) * 0.5).bfloat16().to(cuda)
    res = torch.randn(1, M, N, generator=g).bfloat16().to(cuda)
    gated = ops.gemm_gate_residual(a.view(1, M, K), wd, bias, mod[:, 2:3], res)
    assert torch.equal(gated, res + mod[:, 2:3] * outs["bias"].view(1, M, N))
    monkeypatch.setattr(ops, "SPLIT_K", False)
    for epilogue, y in outs.items():
        y1 = ops.gemm_bf16(a, wd, bias if epilogue else None, epilogue)
        # same products, another fp32 summation order: the linear output moves by at most one bf16 ulp (plus fp32
        # noise where it cancels to ~0), and only on a few outputs; SiLU of an output that moved by one ulp moves by
        # up to ~|x| ulps of its own small value in the negative tail, hence the absolute term there
        diff = (y.float() - y1.float()).abs()
        floor = 2e-2 if epilogue == "bias_silu" else 1e-4
        assert (diff > 2 ** -7 * y1.float().abs() + floor).sum().item() == 0
        assert (diff > 0).float().mean().item() < 0.05
    monkeypatch.setattr(ops, "SPLIT_K", True)
    ai = torch.randint(-2, 3, (M, K), generator=g).bfloat16()
    wi = torch.randint(-1, 2, (N, K), generator=g).bfloat16()
    assert torch.equal(ops.gemm_bf16(ai.to(cuda), wi.to(cuda)).cpu(), (ai.float() @ wi.float().T).bfloat16())


# ---------------------------------------------------------------- fused seams of the block


@pytest.mark.parametrize("B,Ntok,C,K,w8", [(1, 16384, 2240, 2240, False), (2, 1024, 2240, 5600, False),
                                          (3, 100, 96, 240, False), (2, 1024, 2240, 5600, True),
                                          (7, 20, 96, 128, False),    # several gate rows inside one 32-token group
                                          (2, 512, 1152, 1152, False), (3, 100, 264, 1152, True)])  # the 128 x 128 kernel
def test_gemm_gate_residual_matches_stock_op_chain(cuda, B, Ntok, C, K, w8):
    g = torch.Generator().manual_seed(B + K)
    a = torch.randn(B, Ntok, K, generator=g).bfloat16().to(cuda)
    w = (torch.randn(C, K, generator=g) * 0.03).bfloat16()
    bias = (torch.randn(C, generator=g) * 0.1).bfloat16().to(cuda)
    mod = (torch.randn(B, 6, C, generator=g) * 0.5).bfloat16().to(cuda)   # gate is a strided view, as in the block
    gate = mod[:, 2:3]
    res = torch.randn(B, Ntok, C, generator=g).bfloat16().to(cuda)
    if w8:
        wq, s = O.quantize_w8(w)
        w = O.dequantize_w8(wq, s)
        out = ops.gemm_gate_residual(a, wq.to(cuda), bias, gate, res, s.to(cuda), expand=False)
        assert torch.equal(out, ops.gemm_gate_residual(a, wq.to(cuda), bias, gate, res, s.to(cuda), expand=True))
    else:
        out = ops.gemm_gate_residual(a, w.to(cuda), bias, gate, res)
    # the reference's op chain in bf16: linear -> gate * y -> x + (.)
    y = ops.gemm_bf16(a.view(-1, K), w.to(cuda), bias, "bias").view(B, Ntok, C)
    chain = res + gate * y
    assert torch.equal(out, chain)
    ref = res.double() + gate.double() * (a.double() @ w.double().to(cuda).T + bias.double())
    assert rel_l2(out, ref) <= 4e-3


@pytest.mark.parametrize("B,Ntok,C", [(1, 16384, 2240), (4, 1024, 1152), (2, 77, 96), (1, 5, 4096)])
def test_layernorm_modulate_matches_stock_op_chain(cuda, B, Ntok, C):
    g = torch.Generator().manual_seed(C)
    x = (torch.randn(B, Ntok, C, generator=g) * 2 + 0.3).bfloat16().to(cuda)
    mod = (torch.randn(B, 6, C, generator=g) * 0.3).bfloat16().to(cuda)
    shift, scale = mod[:, 0:1], mod[:, 1:2]
    out = ops.layernorm_modulate(x, scale, shift, 1e-6)
    ref64 = F.layer_norm(x.double(), (C,), eps=1e-6) * (1 + scale.double()) + shift.double()
    assert rel_l2(out, ref64) <= 4e-3
    chain = F.layer_norm(x, (C,), eps=1e-6) * (1 + scale) + shift      # stock bf16 chain (four roundings)
    diff = (out.float() - chain.float()).abs()
    # same rounding points: equal except where the fp32 statistics differ in the last bit; a flipped
    # rounding of the product is one bf16 ulp of the product, which the final sum may partly cancel
    mag = chain.float().abs() + shift.float().abs()
    assert (diff > 2 ** -6 * mag + 1e-6).sum().item() == 0
    assert (diff == 0).float().mean().item() > 0.98


@pytest.mark.parametrize("B,Ntok,C", [(1, 16384, 2240), (2, 77, 96), (3, 1024, 1152)])
def test_add_layernorm_modulate_equals_add_then_norm(cuda, B, Ntok, C):
    """x + y and LN(x + y) * (1 + scale) + shift in one pass: the sum is the stock bf16 add bit for bit, the
    normalised output is the plain kernel's output on that sum bit for bit."""
    g = torch.Generator().manual_seed(C + B)
    x = (torch.randn(B, Ntok, C, generator=g) * 2 + 0.3).bfloat16().to(cuda)
    y = torch.randn(B, Ntok, C, generator=g).bfloat16().to(cuda)
    mod = (torch.randn(B, 6, C, generator=g) * 0.3).bfloat16().to(cuda)
    shift, scale = mod[:, 3:4], mod[:, 4:5]
    total, out = ops.add_layernorm_modulate(x, y, scale, shift, 1e-6)
    assert torch.equal(total, x + y)
    assert torch.equal(out, ops.layernorm_modulate(x + y, scale, shift, 1e-6))


@pytest.mark.parametrize("C,T,P,B", [(64, 4, 30, 1), (128, 6, 35, 2), (2240, 3, 300, 1)])
def test_temporal_conv_residual_matches_conv2d(cuda, C, T, P, B):
    """x + t_conv(x) over frames (zero frame in front, zeros behind) against F.conv2d in fp64, with the
    reference's two roundings (conv output to bf16, then the sum)."""
    g = torch.Generator().manual_seed(C + T)
    y = torch.randn(B, T * P, C, generator=g).bfloat16()
    w = (torch.randn(C, C, 3, 1, generator=g) * (1.0 / (3 * C)) ** 0.5).bfloat16()
    xr = y.double().view(B, T, P, C).permute(0, 3, 1, 2)                          # (B, C, T, P) as the reference
    conv = F.conv2d(xr, w.double(), padding=(1, 0))
    ref = (xr + conv.bfloat16().double()).permute(0, 2, 3, 1).reshape(B, T * P, C)
    w2 = w[:, :, :, 0].permute(0, 2, 1).reshape(C, 3 * C).contiguous().to(cuda)
    buf = torch.zeros(B, (T + 1) * P, C, dtype=torch.bfloat16, device=cuda)
    buf[:, P:] = y.to(cuda)
    out = torch.stack([ops.tconv_residual(buf[b], w2, T * P, P) for b in range(B)])
    err = (out.cpu().double() - ref).abs()
    assert err.max().item() <= 2e-2 and rel_l2(out.cpu(), ref) <= 3e-3
    # all but a few results are the reference's bits (the fp32 sums of 3C products differ in order)
    assert (out.cpu().double() != ref.bfloat16().double()).double().mean().item() < 0.02
    # a chunk of frames [1, 3): the frame in front is real data, the frame behind reads as zero
    if T >= 4:
        seg = F.conv2d(torch.cat([xr[:, :, 0:3], torch.zeros_like(xr[:, :, :1])], 2), w.double(), padding=(1, 0))
        ref_c = (xr[:, :, 1:3] + seg[:, :, 1:3].bfloat16().double()).permute(0, 2, 3, 1).reshape(B, 2 * P, C)
        out_c = torch.stack([ops.tconv_residual(buf[b, P:4 * P], w2, 2 * P, P) for b in range(B)])
        assert (out_c.cpu().double() - ref_c).abs().max().item() <= 2e-2 and rel_l2(out_c.cpu(), ref_c) <= 3e-3


@pytest.mark.parametrize("C,T,P,ends", [(128, 7, 37, [0, 3, 4]), (64, 5, 300, [1]), (2240, 6, 260, [2, 4])])
def test_temporal_conv_chunk_flags_equal_per_chunk_launches(cuda, C, T, P, ends):
    """All chunks in one launch (`zero_last_tap` flags on each chunk's last frame) against one launch per chunk,
    whose buffer simply ends behind the chunk: the same products in the same order, so the same bits; and the flags
    must matter (the unflagged launch differs on exactly the flagged frames)."""
    g = torch.Generator().manual_seed(C + T)
    y = torch.randn(T * P, C, generator=g).bfloat16().to(cuda)
    w2 = (torch.randn(C, 3 * C, generator=g) * (1.0 / (3 * C)) ** 0.5).bfloat16().to(cuda)
    buf = torch.cat([torch.randn(P, C, generator=g).bfloat16().to(cuda), y])     # a real frame in front (a cache tail)
    flags = ops.frame_flags(T, ends, cuda)
    one = ops.tconv_residual(buf, w2, T * P, P, zero_last_tap=flags)
    bounds = [0] + [e + 1 for e in sorted(ends)] + ([T] if sorted(ends)[-1] + 1 < T else [])
    parts = [ops.tconv_residual(buf[f0 * P:(f1 + 1) * P], w2, (f1 - f0) * P, P) for f0, f1 in zip(bounds[:-1], bounds[1:])]
    assert torch.equal(one, torch.cat(parts))
    plain = ops.tconv_residual(buf, w2, T * P, P)
    differs = (plain != one).view(T, P * C).any(1).cpu().tolist()
    assert differs == [f in ends and f != T - 1 for f in range(T)]
    assert ops.frame_flags(T, [], cuda) is None


def test_temporal_conv_zero_weight_is_identity(cuda):
    """t_conv is zero-initialised in the reference: x + 0 must come back bit for bit."""
    C, T, P = 128, 3, 50
    y = torch.randn(T * P, C, generator=torch.Generator().manual_seed(3)).bfloat16().to(cuda)
    buf = torch.cat([torch.zeros(P, C, dtype=torch.bfloat16, device=cuda), y])
    out = ops.tconv_residual(buf, torch.zeros(C, 3 * C, dtype=torch.bfloat16, device=cuda), T * P, P)
    assert torch.equal(out, y)


@pytest.mark.parametrize("B,Ntok,C,groups", [(1, 32760, 2240, 1), (2, 120, 96, 4), (3, 77, 1152, 1), (1, 60, 128, 60)])
def test_gate_residual_equals_the_stock_op_pair(cuda, B, Ntok, C, groups):
    """res + gate * y as one pass: the bits of the two stock ops (product rounded to bf16, then the sum), with one
    gate row per batch entry or per group of consecutive tokens (per-frame conditioning)."""
    g = torch.Generator().manual_seed(C + groups)
    y = torch.randn(B, Ntok, C, generator=g).bfloat16().to(cuda)
    res = torch.randn(B, Ntok, C, generator=g).bfloat16().to(cuda)
    mod = (torch.randn(B, groups, 6, C, generator=g) * 0.7).bfloat16().to(cuda)
    gate = mod[:, :, 2:3]                                          # [B, G, 1, C], a strided view as in the blocks
    want = res + (gate * y.view(B, groups, -1, C)).view(B, Ntok, C)
    assert torch.equal(ops.gate_residual(y, gate if groups > 1 else gate[:, 0], res), want)
