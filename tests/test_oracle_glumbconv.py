"""Pins for the oracle's GLUMBConv (Mix-FFN): brute-force taps in C, library
reductions (1x1 conv == linear) and the a/g split."""
import numpy as np
import torch
import torch.nn.functional as F

from oracle import cbrute
from oracle import sana_oracle as O


def _mlp(C, Hd, seed=0):
    torch.manual_seed(seed)
    m = O.GLUMBConv(C, Hd, use_bias=(True, True, False), norm=(None, None, None), act=("silu", "silu", None)).double()
    with torch.no_grad():
        for p in m.parameters():
            p.copy_(torch.randn_like(p) * 0.3)
    return m


def test_state_dict_keys_and_shapes():
    m = O.GLUMBConv(16, 40, use_bias=(True, True, False))
    sd = m.state_dict()
    assert sorted(sd) == ["depth_conv.conv.bias", "depth_conv.conv.weight", "inverted_conv.conv.bias",
                          "inverted_conv.conv.weight", "point_conv.conv.weight"]
    assert sd["inverted_conv.conv.weight"].shape == (80, 16, 1, 1)
    assert sd["depth_conv.conv.weight"].shape == (80, 1, 3, 3)
    assert sd["point_conv.conv.weight"].shape == (16, 40, 1, 1)


def test_against_bruteforce_taps_on_4x5_grid():
    C, Hd, B, Hh, Ww = 6, 10, 2, 4, 5
    m = _mlp(C, Hd)
    x = torch.randn(B, Hh * Ww, C, dtype=torch.float64)
    # stage 1 by library reduction: 1x1 conv == linear, then SiLU
    w1 = m.inverted_conv.conv.weight.flatten(1)
    u = F.silu(x @ w1.T + m.inverted_conv.conv.bias)                      # [B, N, 2H] channels-last
    # stage 2 by brute force in C
    y = cbrute.dwconv_gate(u.view(B, Hh, Ww, 2 * Hd).detach().numpy(),
                           m.depth_conv.conv.weight.view(2 * Hd, 3, 3).detach().numpy(),
                           m.depth_conv.conv.bias.detach().numpy())
    # stage 3: 1x1 conv == linear, no bias
    ref = torch.from_numpy(y).view(B, Hh * Ww, Hd) @ m.point_conv.conv.weight.flatten(1).T
    torch.testing.assert_close(m(x, HW=(Hh, Ww)), ref, rtol=1e-10, atol=1e-12)


def test_gate_is_on_the_second_half():
    """Zeroing the depthwise filter+bias of the FIRST half zeroes the output;
    zeroing the second half gives a * silu(0) = 0 as well, but a bias of +40 on
    the second half (silu(g) ~= g) must scale the output, not gate it off."""
    C, Hd = 4, 6
    m = _mlp(C, Hd, seed=1)
    x = torch.randn(1, 9, C, dtype=torch.float64)
    with torch.no_grad():
        m.depth_conv.conv.weight[Hd:].zero_()
        m.depth_conv.conv.bias[Hd:].fill_(40.0)
    y40 = m(x, HW=(3, 3))
    with torch.no_grad():
        m.depth_conv.conv.bias[Hd:].fill_(20.0)
    y20 = m(x, HW=(3, 3))
    torch.testing.assert_close(y40, 2 * y20, rtol=1e-6, atol=1e-9)
    with torch.no_grad():
        m.depth_conv.conv.weight[:Hd].zero_()
        m.depth_conv.conv.bias[:Hd].zero_()
    assert m(x, HW=(3, 3)).abs().max() == 0


def test_video_hw_is_per_frame():
    """HW=(T,H,W) applies the 3x3 independently per frame (basic_modules.py:187-189)."""
    C, Hd, T, Hh, Ww = 4, 6, 3, 3, 4
    m = _mlp(C, Hd, seed=2)
    x = torch.randn(2, T * Hh * Ww, C, dtype=torch.float64)
    y = m(x, HW=(T, Hh, Ww))
    per_frame = torch.cat([m(x[:, t * Hh * Ww:(t + 1) * Hh * Ww], HW=(Hh, Ww)) for t in range(T)], dim=1)
    torch.testing.assert_close(y, per_frame, rtol=1e-12, atol=1e-12)


def test_autochunk_splits_are_transparent(monkeypatch):
    C, Hd = 4, 6
    m = _mlp(C, Hd, seed=3)
    x = torch.randn(5, 12, C, dtype=torch.float64)
    y = m(x, HW=(3, 4))
    monkeypatch.setattr(O, "INT32_SAFE_CONV_ELEMENTS", 2 * 2 * Hd * 12)  # two images per call
    torch.testing.assert_close(m(x, HW=(3, 4)), y, rtol=0, atol=0)


def test_bf16_rounding_points():
    """Six roundings in bf16 (each torch op returns bf16): conv1x1+bias, SiLU,
    depthwise+bias, SiLU(g), a*g, conv1x1 — reproduced by hand with fp32 math
    between explicit bf16 round trips."""
    C, Hd, Hh, Ww = 32, 80, 6, 7
    torch.manual_seed(5)
    m = O.GLUMBConv(C, Hd, use_bias=(True, True, False)).bfloat16()
    with torch.no_grad():
        for p in m.parameters():
            p.copy_((torch.randn(p.shape) * 0.2).bfloat16())
    x = torch.randn(1, Hh * Ww, C).bfloat16()
    y = m(x, HW=(Hh, Ww))
    r = lambda t: t.bfloat16().float()
    w1 = m.inverted_conv.conv.weight.flatten(1).float()
    u = r(F.silu(r(x.float() @ w1.T + m.inverted_conv.conv.bias.float())))
    un = u.view(1, Hh, Ww, 2 * Hd).permute(0, 3, 1, 2)
    dw = r(F.conv2d(un, m.depth_conv.conv.weight.float(), m.depth_conv.conv.bias.float(), padding=1, groups=2 * Hd))
    a, g = dw[:, :Hd], dw[:, Hd:]
    z = r(a * r(F.silu(g)))
    ref = r(z.permute(0, 2, 3, 1).reshape(1, Hh * Ww, Hd) @ m.point_conv.conv.weight.flatten(1).float().T)
    err = (y.float() - ref).abs().max().item()
    # identical up to fp32 accumulation order inside the library GEMM/conv: at most an ulp of bf16 here and there
    assert err <= 2 ** -7 * ref.abs().max().item(), err
    assert ((y.float() - ref).norm() / ref.norm()).item() < 2e-3


# ---------------------------------------------------------------- temporal variants (basic_modules.py:200-399)

def _temp(cls, C, Hd, seed):
    torch.manual_seed(seed)
    m = cls(C, Hd, use_bias=(True, True, False)).double()
    with torch.no_grad():
        for p in m.parameters():
            p.normal_(0, 0.3)
    return m


def test_temporal_conv_is_zero_initialised_and_then_the_module_is_the_plain_mix_ffn():
    C, Hd, T, Hh, Ww = 8, 20, 3, 2, 5
    torch.manual_seed(0)
    m = O.GLUMBConvTemp(C, Hd, use_bias=(True, True, False)).double()
    assert m.t_conv.weight.abs().max().item() == 0.0 and m.t_conv.bias is None
    plain = O.GLUMBConv(C, Hd, use_bias=(True, True, False)).double()
    plain.load_state_dict({k: v for k, v in m.state_dict().items() if not k.startswith("t_conv")})
    x = torch.randn(2, T * Hh * Ww, C, dtype=torch.float64)
    torch.testing.assert_close(m(x, HW=(T, Hh, Ww)), plain(x, HW=(T, Hh, Ww)), rtol=0, atol=0)


def test_temporal_conv_against_explicit_loops():
    """out[b, t, p, :] = y[b, t, p, :] + sum_dt W[:, :, dt] y[b, t + dt - 1, p, :] with zero frames outside."""
    C, Hd, T, Hh, Ww = 4, 6, 4, 2, 3
    m = _temp(O.GLUMBConvTemp, C, Hd, 1)
    x = torch.randn(2, T * Hh * Ww, C, dtype=torch.float64)
    plain = O.GLUMBConv(C, Hd, use_bias=(True, True, False)).double()
    plain.load_state_dict({k: v for k, v in m.state_dict().items() if not k.startswith("t_conv")})
    y = plain(x, HW=(T, Hh, Ww)).view(2, T, Hh * Ww, C)
    Wt = m.t_conv.weight[:, :, :, 0]   # [co, ci, dt]
    ref = y.clone()
    for t in range(T):
        for dt in range(3):
            ts = t + dt - 1
            if 0 <= ts < T:
                ref[:, t] += y[:, ts] @ Wt[:, :, dt].T
    torch.testing.assert_close(m(x, HW=(T, Hh, Ww)), ref.view(2, -1, C), rtol=1e-12, atol=1e-12)


def test_cached_stream_equals_chunked_temporal_conv_and_frame_mask():
    C, Hd, T, Hh, Ww = 6, 10, 7, 3, 2
    P = Hh * Ww
    chunked = _temp(O.ChunkGLUMBConvTemp, C, Hd, 2)
    cached = O.CachedGLUMBConvTemp(C, Hd, use_bias=(True, True, False)).double()
    cached.load_state_dict(chunked.state_dict())
    x = torch.randn(2, T * P, C, dtype=torch.float64)
    bounds = [0, 2, 3, 7]
    full = chunked(x, HW=(T, Hh, Ww), chunk_index=bounds[:-1])
    cache, outs = [None, None, None], []
    for a, b in zip(bounds[:-1], bounds[1:]):
        o, cache = cached(x[:, a * P:b * P], HW=(b - a, Hh, Ww), save_kv_cache=True, kv_cache=cache)
        assert cache[0] is None and cache[1] is None and cache[-1].shape == (2, C, 1, P)
        outs.append(o)
    torch.testing.assert_close(torch.cat(outs, 1), full, rtol=1e-12, atol=1e-12)
    # one chunk = the unchunked module; a chunk boundary changes only the frame in front of it
    whole = O.GLUMBConvTemp(C, Hd, use_bias=(True, True, False)).double()
    whole.load_state_dict(chunked.state_dict())
    w = whole(x, HW=(T, Hh, Ww))
    torch.testing.assert_close(chunked(x, HW=(T, Hh, Ww), chunk_index=[0]), w, rtol=1e-12, atol=1e-12)
    diff = (full - w).view(2, T, P, C).abs().amax(dim=(0, 2, 3))
    assert (diff[[1, 2]] > 1e-6).all() and diff[[0, 3, 4, 5, 6]].max().item() < 1e-12
    # masked frames are zero on the way in and on the way out
    mask = torch.ones(2, T)
    mask[:, 5:] = 0
    wm = whole(x, HW=(T, Hh, Ww), frame_valid_mask=mask).view(2, T, P, C)
    assert wm[:, 5:].abs().max().item() == 0.0
    torch.testing.assert_close(wm[:, :4], w.view(2, T, P, C)[:, :4], rtol=1e-12, atol=1e-12)


# ---- GLUMBConvLinear (basic_modules_linear.py:133-311): the same function with nn.Linear parameters


def _linear_twin(conv_module, linear_cls, **kw):
    """A *Linear module holding conv_module's weights under the mapping stated at basic_modules_linear.py:142-146."""
    from sana_amd import checkpoint as ck
    twin = linear_cls(**kw).double()
    twin.load_state_dict(ck.ffn_conv_to_linear(conv_module.state_dict()), strict=True)
    return twin


def test_linear_variant_is_the_same_function_as_the_conv_variant():
    """A 1x1 convolution over a channels-first image is a matmul over its pixels: with the stated weight mapping
    GLUMBConvLinear must reproduce GLUMBConv (itself pinned by the brute-force taps above) on image and video HW,
    and its HW=None default must be the square grid."""
    kw = dict(in_features=24, hidden_features=40, use_bias=(True, True, False))
    conv = O.GLUMBConv(**kw).double()
    g = torch.Generator().manual_seed(3)
    with torch.no_grad():
        for p in conv.parameters():
            p.copy_(torch.randn(p.shape, generator=g, dtype=torch.float64) * 0.3)
    lin = _linear_twin(conv, O.GLUMBConvLinear, **kw)
    assert sorted(lin.state_dict()) == ["depth_conv.conv.bias", "depth_conv.conv.weight", "inverted_conv.linear.bias",
                                        "inverted_conv.linear.weight", "point_conv.linear.weight"]
    assert lin.state_dict()["inverted_conv.linear.weight"].shape == (80, 24)
    x = torch.randn(2, 36, 24, generator=g, dtype=torch.float64)
    for hw in [(6, 6), (4, 9), (2, 3, 6), (3, 4, 3)]:
        torch.testing.assert_close(lin(x, HW=hw), conv(x, HW=hw), rtol=1e-12, atol=1e-12)
    torch.testing.assert_close(lin(x), conv(x, HW=(6, 6)), rtol=1e-12, atol=1e-12)
    # a non-square grid must differ from the square default (the reshape is not a no-op)
    assert (lin(x, HW=(4, 9)) - lin(x)).abs().max() > 1e-3


def test_linear_temporal_variant_matches_the_conv_temporal_variant():
    kw = dict(in_features=16, hidden_features=24, use_bias=(True, True, False))
    conv = O.GLUMBConvTemp(**kw).double()
    g = torch.Generator().manual_seed(4)
    with torch.no_grad():
        for p in conv.parameters():
            p.copy_(torch.randn(p.shape, generator=g, dtype=torch.float64) * 0.3)
    lin = _linear_twin(conv, O.GLUMBConvLinearTemp, **kw)
    assert "t_conv.weight" in lin.state_dict()
    x = torch.randn(2, 5 * 12, 16, generator=g, dtype=torch.float64)
    torch.testing.assert_close(lin(x, HW=(5, 3, 4)), conv(x, HW=(5, 3, 4)), rtol=1e-12, atol=1e-12)
