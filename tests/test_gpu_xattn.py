"""Cross-attention to the text tokens: the short-key softmax attention kernel against the fp64 formula
(reference: diffusion/model/nets/sana_blocks.py:69-98, the scaled_dot_product_attention branch with its additive
padding mask), and the module built on it against the oracle module.  Tolerance: bf16 outputs, max-abs <= 2e-2 and
rel-L2 <= 1e-2 (the probabilities are rounded to bf16 before they multiply v, as fused attention kernels do)."""
import pytest
import torch

import sana_amd as S
from sana_amd import ops
from oracle import sana_oracle as O

pytestmark = pytest.mark.gpu


def rel_l2(a, b):
    return ((a.double() - b.double()).norm() / b.double().norm()).item()


def formula(q, kv, H, bias=None):
    """softmax(q k^T / sqrt(d) + bias) v per head in fp64, token-major in and out."""
    B, N, C = q.shape
    d = C // H
    qh = q.double().view(B, N, H, d).transpose(1, 2)
    k = kv.double()[:, :, :C].reshape(B, -1, H, d).transpose(1, 2)
    v = kv.double()[:, :, C:].reshape(B, -1, H, d).transpose(1, 2)
    s = qh @ k.transpose(-1, -2) * d ** -0.5
    if bias is not None:
        s = s + bias.double()[:, None, None, :]
    return (torch.softmax(s, -1) @ v).transpose(1, 2).reshape(B, N, C)


@pytest.mark.parametrize("B,N,Nk,H,d,masked", [(1, 16384, 300, 20, 112, False),   # the 4096 px latent, Sana-1.6B
                                              (2, 1024, 300, 20, 112, True),
                                              (3, 200, 77, 16, 72, True),        # Sana-600M heads, ragged query blocks
                                              (1, 37, 1, 2, 112, False),         # a single key: the output is v
                                              (2, 130, 320, 4, 104, True),       # the largest key set, another head_dim
                                              (1, 64, 33, 3, 80, False)])
def test_cross_attention_matches_the_formula(cuda, B, N, Nk, H, d, masked):
    g = torch.Generator().manual_seed(B * 1000 + N + Nk + d)
    C = H * d
    q = (torch.randn(B, N, C, generator=g) * 1.5).bfloat16()
    kv = torch.randn(B, Nk, 2 * C, generator=g).bfloat16()
    bias = None
    if masked:   # the reference's padding mask: the tail of every text is padding, of another length per batch entry
        keep = torch.ones(B, Nk)
        for b in range(B):
            keep[b, max(1, Nk - 7 * (b + 1)):] = 0
        bias = (1 - keep) * -10000.0
    out = ops.cross_attention(q.to(cuda), kv.to(cuda), H, None if bias is None else bias.to(cuda))
    ref = formula(q, kv, H, bias)
    mx = (out.cpu().double() - ref).abs().max().item()
    assert mx <= 2e-2 and rel_l2(out.cpu(), ref) <= 1e-2, (mx, rel_l2(out.cpu(), ref))
    if Nk == 1:
        assert torch.equal(out.cpu().view(B, N, H, d), kv[:, :1, C:].view(B, 1, H, d).expand(B, N, H, d))


def test_cross_attention_on_strided_rows_and_masked_keys_contribute_nothing(cuda):
    """q as a column slice of a wider buffer (row stride > C); what keys under the -10000 bias hold does not matter
    (as long as their scores stay small against 10000: the mask is additive, as in the reference)."""
    g = torch.Generator().manual_seed(5)
    B, N, Nk, H, d = 2, 300, 40, 2, 112
    C = H * d
    wide = torch.randn(B, N, C + 64, generator=g).bfloat16().to(cuda)
    kv = torch.randn(B, Nk, 2 * C, generator=g).bfloat16()
    keep = torch.ones(B, Nk)
    keep[:, 25:] = 0
    bias = ((1 - keep) * -10000.0).to(cuda)
    a = ops.cross_attention(wide[:, :, :C], kv.to(cuda), H, bias)
    kv2 = kv.clone()
    kv2[:, 25:] = 3.0
    b = ops.cross_attention(wide[:, :, :C], kv2.to(cuda), H, bias)
    assert torch.equal(a, b)
    ref = formula(wide[:, :, :C].cpu(), kv, H, bias.cpu())
    assert (a.cpu().double() - ref).abs().max().item() <= 2e-2


def test_cross_attention_rejects_what_it_cannot_hold(cuda):
    q = torch.zeros(1, 16, 256, dtype=torch.bfloat16, device=cuda)
    with pytest.raises(S.SanaHipError):
        ops.cross_attention(q, torch.zeros(1, 321, 512, dtype=torch.bfloat16, device=cuda), 2)     # 128-wide heads, 321 keys
    with pytest.raises(S.SanaHipError):
        ops.cross_attention(q, torch.zeros(1, 10, 512, dtype=torch.bfloat16, device=cuda), 8)      # head_dim 32
    with pytest.raises(S.SanaHipError):
        ops.cross_attention(q.float(), torch.zeros(1, 10, 512, device=cuda), 2)


@pytest.mark.parametrize("C,H,B,N,Nk,masked", [(2240, 20, 1, 1024, 300, False), (1152, 16, 2, 256, 120, True)])
def test_cross_attention_module_matches_oracle(cuda, C, H, B, N, Nk, masked):
    g = torch.Generator().manual_seed(C + N)
    om = O.MultiHeadCrossAttention(C, H)
    with torch.no_grad():
        for p in om.parameters():
            p.copy_(torch.nn.init.trunc_normal_(torch.empty(p.shape), std=0.02, generator=g))
    om = om.bfloat16()
    hm = S.modules.MultiHeadCrossAttention(C, H).bfloat16()
    hm.load_state_dict(om.state_dict())
    hm = hm.to(cuda)
    x = torch.randn(B, N, C, generator=g).bfloat16()
    y = torch.randn(B, Nk, C, generator=g).bfloat16()
    mask = None
    if masked:
        mask = torch.ones(B, Nk, dtype=torch.int64)
        mask[0, Nk // 2:] = 0
    with torch.no_grad():
        out = hm(x.to(cuda), y.to(cuda), None if mask is None else mask.to(cuda))
        ref = om.float()(x.float(), y.float(), mask)
    mx = (out.cpu().double() - ref.double()).abs().max().item()
    assert mx <= 2e-2 and rel_l2(out.cpu(), ref) <= 1e-2, (mx, rel_l2(out.cpu(), ref))


def test_residual_add_inside_the_projection_gemm(cuda):
    """x + cross_attn(x, y): from 4096 rows on the add is the projection GEMM's epilogue (two roundings, as the stock
    linear + add); against the oracle module's output plus x, and against the unfused composition of this module (same
    products, another fp32 summation order inside the two GEMMs: at most one bf16 ulp of the sum apart)."""
    C, H, B, N, Nk = 2240, 20, 2, 2048, 300
    g = torch.Generator().manual_seed(3)
    om = O.MultiHeadCrossAttention(C, H)
    with torch.no_grad():
        for p in om.parameters():
            p.copy_(torch.nn.init.trunc_normal_(torch.empty(p.shape), std=0.02, generator=g))
    om = om.bfloat16()
    hm = S.modules.MultiHeadCrossAttention(C, H).bfloat16()
    hm.load_state_dict(om.state_dict())
    hm = hm.to(cuda)
    assert B * N >= hm.RESIDUAL_GEMM_MIN_ROWS
    x = torch.randn(B, N, C, generator=g).bfloat16()
    y = torch.randn(B, Nk, C, generator=g).bfloat16()
    with torch.no_grad():
        fused = hm.forward_residual(x.to(cuda), y.to(cuda))
        plain = x.to(cuda) + hm(x.to(cuda), y.to(cuda))
        ref = x.float() + om.float()(x.float(), y.float())
    assert (fused.float() - plain.float()).abs().max().item() <= 2 ** -7 * plain.float().abs().max().item()
    mx = (fused.cpu().double() - ref.double()).abs()
    assert (mx > 2e-2 + 2.0 ** -7 * ref.double().abs()).sum().item() == 0 and rel_l2(fused.cpu(), ref) <= 1e-2
    small = hm.forward_residual(x[:, :64].to(cuda), y.to(cuda))       # below the threshold: the composition itself
    assert torch.equal(small, x[:, :64].to(cuda) + hm(x[:, :64].to(cuda), y.to(cuda)))
