"""Pins for the oracle's ReLU linear attention (LiteLA.attn_matmul and LiteLA.forward).

None of these retypes the oracle's formula: the C brute force is the quadratic
form, the invariants are properties of the mathematics.
"""
import numpy as np
import pytest
import torch

from oracle import cbrute
from oracle import sana_oracle as O


def _qkv(B, h, d, N, seed, dtype=torch.float64):
    g = torch.Generator().manual_seed(seed)
    q = torch.randn(B, h, d, N, generator=g, dtype=torch.float64).to(dtype)
    k = torch.randn(B, h, N, d, generator=g, dtype=torch.float64).to(dtype)
    v = torch.randn(B, h, d, N, generator=g, dtype=torch.float64).to(dtype)
    return q, k, v


def _token_major(q, k, v):
    B, h, d, N = q.shape
    return (q.permute(0, 1, 3, 2).reshape(B * h, N, d).numpy(),
            k.reshape(B * h, N, d).numpy(),
            v.permute(0, 1, 3, 2).reshape(B * h, N, d).numpy())


@pytest.mark.parametrize("B,h,d,N,eps", [(1, 2, 32, 48, 1e-15), (2, 3, 8, 17, 1e-8), (1, 1, 4, 1, 1e-15)])
def test_matches_quadratic_bruteforce(B, h, d, N, eps):
    q, k, v = _qkv(B, h, d, N, seed=B * 100 + N)
    out, state = O.relu_linear_attention(q, k, v, eps, return_state=True)
    qn, kn, vn = _token_major(q, k, v)
    ref = cbrute.relu_attention(qn, kn, vn, eps).reshape(B, h, N, d).transpose(0, 1, 3, 2)
    np.testing.assert_allclose(out.numpy(), ref, rtol=1e-10, atol=1e-12)
    sref = cbrute.attention_state(kn, vn).reshape(B, h, d + 1, d)
    np.testing.assert_allclose(state.numpy(), sref, rtol=1e-11, atol=1e-12)


def test_state_last_row_is_relu_k_sum():
    q, k, v = _qkv(1, 2, 8, 33, seed=3)
    _, state = O.relu_linear_attention(q, k, v, 1e-15, return_state=True)
    torch.testing.assert_close(state[:, :, -1], torch.relu(k).sum(dim=2))


def test_token_permutation_invariance_and_equivariance():
    q, k, v = _qkv(1, 2, 8, 40, seed=4)
    perm = torch.randperm(40, generator=torch.Generator().manual_seed(0))
    base = O.relu_linear_attention(q, k, v, 1e-15)
    # permuting keys/values together changes nothing
    out = O.relu_linear_attention(q, k[:, :, perm], v[..., perm], 1e-15)
    torch.testing.assert_close(out, base, rtol=1e-11, atol=1e-12)
    # permuting queries permutes the output
    out = O.relu_linear_attention(q[..., perm], k, v, 1e-15)
    torch.testing.assert_close(out, base[..., perm], rtol=1e-11, atol=1e-12)


def test_linear_in_v_and_constant_v():
    q, k, v = _qkv(1, 2, 8, 40, seed=5)
    v2 = torch.randn_like(v)
    f = lambda vv: O.relu_linear_attention(q, k, vv, 0.0)
    torch.testing.assert_close(f(2.5 * v - v2), 2.5 * f(v) - f(v2), rtol=1e-10, atol=1e-11)
    # v == c  =>  out == c * den / (den + eps)
    eps = 0.3
    c = 1.75
    den = torch.einsum("bhnj,bhjm->bhm", torch.relu(k), torch.relu(q))  # sum over keys of <k, q_m>
    out = O.relu_linear_attention(q, k, torch.full_like(v, c), eps)
    torch.testing.assert_close(out, (c * den / (den + eps))[:, :, None].expand_as(out), rtol=1e-10, atol=1e-12)


def test_all_negative_query_gives_zero():
    q, k, v = _qkv(1, 1, 8, 12, seed=6)
    q[..., 5] = -q[..., 5].abs() - 0.1
    out = O.relu_linear_attention(q, k, v, 1e-15)
    assert torch.all(out[..., 5] == 0)


def test_state_additive_over_token_subsets():
    q, k, v = _qkv(1, 2, 8, 64, seed=7)
    _, s_all = O.relu_linear_attention(q, k, v, 1e-15, return_state=True)
    _, s_a = O.relu_linear_attention(q, k[:, :, :20], v[..., :20], 1e-15, return_state=True)
    _, s_b = O.relu_linear_attention(q, k[:, :, 20:], v[..., 20:], 1e-15, return_state=True)
    torch.testing.assert_close(s_a + s_b, s_all, rtol=1e-11, atol=1e-12)


def test_eps_is_a_runtime_value():
    q, k, v = _qkv(1, 1, 4, 6, seed=8)
    a = O.relu_linear_attention(q, k, v, 1e-15)
    b = O.relu_linear_attention(q, k, v, 10.0)
    assert (a - b).abs().max() > 1e-3


def test_bf16_dtype_flow():
    """fp32_attention: fp32 matmuls of bf16-valued operands; otherwise both matmul
    results are rounded to bf16 before the fp32 divide (sana_blocks.py:251-261)."""
    q, k, v = _qkv(1, 2, 32, 256, seed=9, dtype=torch.bfloat16)
    exact = O.relu_linear_attention(q.double(), k.double(), v.double(), 1e-8)
    hi = O.relu_linear_attention(q, k, v, 1e-8, fp32_attention=True)
    lo = O.relu_linear_attention(q, k, v, 1e-8, fp32_attention=False)
    assert hi.dtype == torch.float32 and lo.dtype == torch.float32
    rel = lambda a: ((a.double() - exact).norm() / exact.norm()).item()
    assert rel(hi) < 1e-6
    assert 1e-4 < rel(lo) < 1e-2


def test_module_layout_head_is_channel_div_d():
    """qkv(x).reshape(B,N,3,C): q|k|v are the three C-blocks of the output
    features and head = channel // d (pinned by the checkpoint converter's
    torch.chunk(qkv.weight, 3, dim=0): tools/convert_scripts/convert_sana_to_diffusers.py:160-163)."""
    torch.manual_seed(0)
    B, N, C, d = 2, 24, 64, 16
    m = O.LiteLA(C, C, dim=d, eps=1e-8).double()
    x = torch.randn(B, N, C, dtype=torch.float64)
    wq, wk, wv = torch.chunk(m.qkv.weight, 3, dim=0)
    q = (x @ wq.T).view(B, N, C // d, d).permute(0, 2, 1, 3).reshape(-1, N, d)
    k = (x @ wk.T).view(B, N, C // d, d).permute(0, 2, 1, 3).reshape(-1, N, d)
    v = (x @ wv.T).view(B, N, C // d, d).permute(0, 2, 1, 3).reshape(-1, N, d)
    att = cbrute.relu_attention(q.detach().numpy(), k.detach().numpy(), v.detach().numpy(), 1e-8)
    att = torch.from_numpy(att).view(B, C // d, N, d).permute(0, 2, 1, 3).reshape(B, N, C)
    ref = att @ m.proj.weight.T + m.proj.bias
    torch.testing.assert_close(m(x, HW=(4, 6)), ref, rtol=1e-9, atol=1e-11)


def test_module_state_dict_keys():
    m = O.LiteLA(64, 64, dim=32)
    assert sorted(m.state_dict()) == ["proj.bias", "proj.weight", "qkv.weight"]
    m = O.LiteLA(64, 64, dim=32, qk_norm=True)
    assert sorted(m.state_dict()) == ["k_norm.weight", "proj.bias", "proj.weight", "q_norm.weight", "qkv.weight"]
    assert m.dim == 32 and m.heads == 2 and m.eps == 1e-15


def test_rmsnorm_closed_form():
    n = O.RMSNorm(8, eps=1e-5)
    with torch.no_grad():
        n.weight.copy_(torch.arange(1, 9).float())
    x = torch.tensor([[3.0, -4.0, 0, 0, 0, 0, 0, 0]])
    rms = (25.0 / 8 + 1e-5) ** 0.5
    torch.testing.assert_close(n(x), torch.tensor([[3 / rms, -8 / rms, 0, 0, 0, 0, 0, 0]]))


def test_rotary_real_is_a_rotation_of_channel_pairs():
    B, h, d, N = 1, 2, 8, 5
    x = torch.randn(B, h, d, N, dtype=torch.float64)
    theta = torch.rand(N, d // 2, dtype=torch.float64) * 6
    cos = torch.cos(theta).repeat_interleave(2, dim=1)
    sin = torch.sin(theta).repeat_interleave(2, dim=1)
    y = O.rotary_real(x, (cos, sin))
    xc = torch.view_as_complex(x.permute(0, 1, 3, 2).reshape(B, h, N, d // 2, 2).contiguous())
    yc = xc * torch.polar(torch.ones_like(theta), theta)
    ref = torch.view_as_real(yc).reshape(B, h, N, d).permute(0, 1, 3, 2)
    torch.testing.assert_close(y, ref.to(y.dtype), rtol=1e-6, atol=1e-6)
    # and the complex form used by the ReLU->RoPE family agrees with it
    y2 = O.rotary_complex(x, torch.polar(torch.ones_like(theta), theta)[None, None])
    torch.testing.assert_close(y2, ref, rtol=1e-12, atol=1e-12)


def test_guidance_processors_restate_the_attention_forward():
    """SelfAttnProcessorLiteLA is LiteLA.forward on the module's parts; the PAG processors run it on the
    unperturbed part of the batch and proj(v_linear(x)) (identity attention) on the perturbed part
    (sana_blocks.py:575-717)."""
    torch.manual_seed(0)
    C, N = 64, 24
    attn = O.LiteLA(C, C, heads=2, eps=1e-8, qk_norm=True).double()
    with torch.no_grad():
        for p in attn.parameters():
            p.normal_(0, 0.2)
    x = torch.randn(3, N, C, dtype=torch.float64)
    plain = attn(x)
    torch.testing.assert_close(O.SelfAttnProcessorLiteLA(attn)(x), plain, rtol=1e-12, atol=1e-12)
    v_only = attn.proj(x @ attn.qkv.weight[2 * C:].T)
    out3 = O.PAGCFGIdentitySelfAttnProcessorLiteLA(attn)(x)
    torch.testing.assert_close(out3[:2], plain[:2], rtol=1e-12, atol=1e-12)
    torch.testing.assert_close(out3[2:], v_only[2:], rtol=1e-12, atol=1e-12)
    out2 = O.PAGIdentitySelfAttnProcessorLiteLA(attn)(x[:2])
    torch.testing.assert_close(out2[:1], plain[:1], rtol=1e-12, atol=1e-12)
    torch.testing.assert_close(out2[1:], v_only[1:2], rtol=1e-12, atol=1e-12)
