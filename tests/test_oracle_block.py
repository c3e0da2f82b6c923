"""Pins for the oracle's SanaMSBlock wiring, cross-attention and chunk-causal family."""
import numpy as np
import pytest
import torch
import torch.nn.functional as F

from oracle import cbrute
from oracle import sana_oracle as O


def _block(C=64, heads=4, seed=0, dtype=torch.float64):
    blk = O.SanaMSBlock(C, heads, mlp_ratio=2.5, attn_type="linear", ffn_type="glumbconv", linear_head_dim=32)
    O.init_block_(blk, seed)
    with torch.no_grad():
        for n, p in blk.named_parameters():
            if n.endswith("bias"):
                p.copy_(torch.randn(p.shape, generator=torch.Generator().manual_seed(len(n))) * 0.1)
    return blk.to(dtype)


def test_block_keys_and_defaults():
    blk = O.SanaMSBlock(64, 4, mlp_ratio=2.5, attn_type="linear", ffn_type="glumbconv")
    keys = set(blk.state_dict())
    assert keys == {
        "scale_shift_table", "attn.qkv.weight", "attn.proj.weight", "attn.proj.bias",
        "cross_attn.q_linear.weight", "cross_attn.q_linear.bias", "cross_attn.kv_linear.weight",
        "cross_attn.kv_linear.bias", "cross_attn.proj.weight", "cross_attn.proj.bias",
        "mlp.inverted_conv.conv.weight", "mlp.inverted_conv.conv.bias", "mlp.depth_conv.conv.weight",
        "mlp.depth_conv.conv.bias", "mlp.point_conv.conv.weight"}
    assert blk.attn.eps == 1e-8  # the block overrides LiteLA's 1e-15 default (sana_multi_scale.py:90)
    assert blk.mlp.inverted_conv.conv.out_channels == 2 * 160


def test_zero_gates_reduce_block_to_cross_attention_residual():
    C = 64
    blk = _block(C)
    x, y, t = (a.double() for a in O.block_inputs(2, 16, C, n_text=7))
    with torch.no_grad():
        blk.scale_shift_table[2].zero_()
        blk.scale_shift_table[5].zero_()
    t = t.view(2, 6, C).clone()
    t[:, 2] = 0
    t[:, 5] = 0
    out = blk(x, y, t.view(2, 6 * C), HW=(4, 4))
    torch.testing.assert_close(out, x + blk.cross_attn(x, y), rtol=1e-12, atol=1e-12)


def test_block_composition_by_hand():
    C = 64
    blk = _block(C, seed=1)
    x, y, t = (a.double() for a in O.block_inputs(2, 16, C, n_text=5))
    sst = (blk.scale_shift_table[None] + t.view(2, 6, C))
    sh1, sc1, g1, sh2, sc2, g2 = [sst[:, i:i + 1] for i in range(6)]
    ln = lambda z: (z - z.mean(-1, keepdim=True)) / torch.sqrt(z.var(-1, unbiased=False, keepdim=True) + 1e-6)
    h = x + g1 * blk.attn(ln(x) * (1 + sc1) + sh1, HW=(4, 4))
    h = h + blk.cross_attn(h, y)
    h = h + g2 * blk.mlp(ln(h) * (1 + sc2) + sh2, HW=(4, 4))
    torch.testing.assert_close(blk(x, y, t, HW=(4, 4)), h, rtol=1e-10, atol=1e-11)


def test_cross_attention_closed_form_and_mask():
    torch.manual_seed(0)
    C, nh = 32, 4
    ca = O.MultiHeadCrossAttention(C, nh).double()
    x = torch.randn(2, 6, C, dtype=torch.float64)
    y = torch.randn(2, 5, C, dtype=torch.float64)
    q = (x @ ca.q_linear.weight.T + ca.q_linear.bias).view(2, 6, nh, C // nh)
    kv = y @ ca.kv_linear.weight.T + ca.kv_linear.bias
    k, v = kv[..., :C].reshape(2, 5, nh, C // nh), kv[..., C:].reshape(2, 5, nh, C // nh)
    att = torch.einsum("bqhd,bkhd->bhqk", q, k) / (C // nh) ** 0.5
    ref = torch.einsum("bhqk,bkhd->bqhd", att.softmax(-1), v).reshape(2, 6, C) @ ca.proj.weight.T + ca.proj.bias
    torch.testing.assert_close(ca(x, y), ref, rtol=1e-10, atol=1e-12)
    # a 2-d mask removes padded text tokens
    mask = torch.tensor([[1, 1, 1, 0, 0], [1, 1, 1, 1, 1]])
    out = ca(x, y, mask)
    y2 = y.clone()
    y2[0, 3:] = 123.0  # masked tokens must not matter
    torch.testing.assert_close(ca(x, y2, mask), out, rtol=1e-9, atol=1e-9)


# ---------------------------------------------------------------- chunk-causal family


def _attn_inputs(cls, C=64, d=32, N=24, seed=0):
    torch.manual_seed(seed)
    m = cls(C, C, dim=d, eps=1e-8).double()
    x = torch.randn(2, N, C, dtype=torch.float64)
    return m, x


def test_relurope_with_unit_rotary_equals_litela():
    m, x = _attn_inputs(O.LiteLAReLURope)
    ref = O.LiteLA(64, 64, dim=32, eps=1e-8).double()
    ref.load_state_dict(m.state_dict())
    unit = torch.ones(1, 1, 24, 16, dtype=torch.complex128)
    torch.testing.assert_close(m(x, rotary_emb=unit), ref(x), rtol=1e-10, atol=1e-12)
    torch.testing.assert_close(m(x, rotary_emb=None), ref(x), rtol=1e-10, atol=1e-12)


def test_chunk_causal_single_chunk_equals_relurope():
    m, x = _attn_inputs(O.ChunkCausalAttention)
    base = O.LiteLAReLURope(64, 64, dim=32, eps=1e-8).double()
    base.load_state_dict(m.state_dict())
    theta = torch.rand(24, 16, dtype=torch.float64)
    rot = torch.polar(torch.ones_like(theta), theta)[None, None]
    torch.testing.assert_close(m(x, HW=(4, 2, 3), rotary_emb=rot, chunk_index=[0]),
                               base(x, rotary_emb=rot), rtol=1e-10, atol=1e-12)


@pytest.mark.parametrize("chunk_index", [[0, 1, 2, 3], [0, 3], [0, 1, 3]])
def test_chunk_causal_matches_masked_quadratic_form(chunk_index):
    C, d, f, hh, ww = 64, 32, 4, 2, 3
    N = f * hh * ww
    m, x = _attn_inputs(O.ChunkCausalAttention, C, d, N, seed=3)
    out = m(x, HW=(f, hh, ww), rotary_emb=None, chunk_index=list(chunk_index))
    qkv = (x @ m.qkv.weight.T).view(2, N, 3, C // d, d)
    tm = lambda i: qkv[:, :, i].permute(0, 2, 1, 3).reshape(-1, N, d).detach().numpy()
    bounds = list(chunk_index) + [f]
    chunk_of = np.zeros(N, dtype=np.int32)
    for ci, (a, b) in enumerate(zip(bounds[:-1], bounds[1:])):
        chunk_of[a * hh * ww:b * hh * ww] = ci
    att = cbrute.relu_attention(tm(0), tm(1), tm(2), 1e-8, chunk_of)
    att = torch.from_numpy(att).view(2, C // d, N, d).permute(0, 2, 1, 3).reshape(2, N, C)
    ref = att @ m.proj.weight.T + m.proj.bias
    torch.testing.assert_close(out, ref, rtol=1e-9, atol=1e-11)


def test_cached_causal_stream_equals_chunk_causal():
    """Feeding chunks one by one with the caller accumulating the saved states
    (diffusion/longsana/pipeline/sana_inference_pipeline.py:242-263) reproduces
    the one-shot chunk-causal forward."""
    C, d, f, hh, ww = 64, 32, 3, 2, 2
    N = f * hh * ww
    m, x = _attn_inputs(O.ChunkCausalAttention, C, d, N, seed=4)
    full = m(x, HW=(f, hh, ww), chunk_index=[0, 1, 2])
    cm = O.CachedCausalAttention(C, C, dim=d, eps=1e-8).double()
    cm.load_state_dict(m.state_dict())
    acc = [None, None]
    outs = []
    for c in range(f):
        cache = [acc[0], acc[1]]
        o, cache = cm(x[:, c * 4:(c + 1) * 4], save_kv_cache=True, kv_cache=cache)
        acc = [cache[0] if acc[0] is None else acc[0] + cache[0],
               cache[1] if acc[1] is None else acc[1] + cache[1]]
        outs.append(o)
    torch.testing.assert_close(torch.cat(outs, 1), full, rtol=1e-10, atol=1e-12)


def _rope_case(cls, d, f, hh, ww, seed):
    """Module, input, generic (non-unit) complex factors and the token-major q/k/v of every (batch, head)."""
    heads = 2
    C = heads * d
    N = f * hh * ww
    m, x = _attn_inputs(cls, C, d, N, seed=seed)
    g = torch.Generator().manual_seed(100 + seed)
    theta = (torch.rand(N, d // 2, generator=g, dtype=torch.float64) - 0.5) * 6.0
    radius = 0.5 + torch.rand(N, d // 2, generator=g, dtype=torch.float64)      # not on the unit circle
    rot = torch.polar(radius, theta)[None, None]
    qkv = (x @ m.qkv.weight.T).view(2, N, 3, heads, d)
    tm = lambda i: qkv[:, :, i].permute(0, 2, 1, 3).reshape(-1, N, d).detach().numpy()
    return m, x, rot, (tm(0), tm(1), tm(2)), (C, N, heads)


def _proj_of(att, m, C, N, heads, d):
    att = torch.from_numpy(att).view(2, heads, N, d).permute(0, 2, 1, 3).reshape(2, N, C)
    return att @ m.proj.weight.T + m.proj.bias


@pytest.mark.parametrize("d", [32, 112])
def test_relurope_matches_rotated_numerator_quadratic_form(d):
    """Pins WHICH operands are rotated (sana_blocks.py:378-381): numerator rotated, denominator not.
    Generic angles and radii, so a rotated denominator (or an unrotated numerator) gives other numbers."""
    m, x, rot, (q, k, v), (C, N, heads) = _rope_case(O.LiteLAReLURope, d, 3, 2, 3, seed=5)
    out = m(x, rotary_emb=rot)
    ref = _proj_of(cbrute.relu_attention_rope(q, k, v, rot[0, 0].numpy(), 1e-8), m, C, N, heads, d)
    torch.testing.assert_close(out, ref, rtol=1e-9, atol=1e-11)
    # the two plausible mistakes are far away from the brute force: both sides rotated / none rotated
    plain = _proj_of(cbrute.relu_attention(q, k, v, 1e-8), m, C, N, heads, d)
    assert (plain - ref).abs().max() > 1e-3


@pytest.mark.parametrize("d", [32, 112])
@pytest.mark.parametrize("chunk_index", [[0, 1, 2, 3], [0, 3], [0, 1, 3]])
def test_chunk_causal_rope_matches_masked_rotated_quadratic_form(d, chunk_index):
    """sana_blocks.py:481-489 with a rotary embedding: cumulative rotated vk, cumulative UNROTATED k sum."""
    f, hh, ww = 4, 2, 3
    m, x, rot, (q, k, v), (C, N, heads) = _rope_case(O.ChunkCausalAttention, d, f, hh, ww, seed=6)
    out = m(x, HW=(f, hh, ww), rotary_emb=rot, chunk_index=list(chunk_index))
    bounds = list(chunk_index) + [f]
    chunk_of = np.zeros(N, dtype=np.int32)
    for ci, (a, b) in enumerate(zip(bounds[:-1], bounds[1:])):
        chunk_of[a * hh * ww:b * hh * ww] = ci
    ref = _proj_of(cbrute.relu_attention_rope(q, k, v, rot[0, 0].numpy(), 1e-8, chunk_of), m, C, N, heads, d)
    torch.testing.assert_close(out, ref, rtol=1e-9, atol=1e-11)


@pytest.mark.parametrize("d", [32, 112])
def test_cached_causal_rope_stream_matches_masked_rotated_quadratic_form(d):
    """sana_blocks.py:544-562 streamed chunk by chunk (each call gets its own slice of the factors, the caller
    accumulates the saved states) against the brute force on the whole sequence."""
    f, hh, ww = 3, 2, 2
    P = hh * ww
    m, x, rot, (q, k, v), (C, N, heads) = _rope_case(O.CachedCausalAttention, d, f, hh, ww, seed=7)
    acc = [None, None]
    outs = []
    for c in range(f):
        cache = [acc[0], acc[1]]
        o, cache = m(x[:, c * P:(c + 1) * P], rotary_emb=rot[:, :, c * P:(c + 1) * P], save_kv_cache=True,
                     kv_cache=cache)
        acc = [cache[0] if acc[0] is None else acc[0] + cache[0],
               cache[1] if acc[1] is None else acc[1] + cache[1]]
        outs.append(o)
    chunk_of = np.repeat(np.arange(f, dtype=np.int32), P)
    ref = _proj_of(cbrute.relu_attention_rope(q, k, v, rot[0, 0].numpy(), 1e-8, chunk_of), m, C, N, heads, d)
    torch.testing.assert_close(torch.cat(outs, 1), ref, rtol=1e-9, atol=1e-11)


def test_rotated_brute_force_reduces_to_the_plain_one_for_unit_factors():
    rng = np.random.default_rng(0)
    q, k, v = (rng.standard_normal((3, 10, 8)) for _ in range(3))
    ones = np.ones((10, 4), dtype=np.complex128)
    np.testing.assert_allclose(cbrute.relu_attention_rope(q, k, v, ones, 1e-8), cbrute.relu_attention(q, k, v, 1e-8),
                               rtol=1e-13, atol=1e-14)
    # a rotation common to all tokens leaves <rot k, rot q> unchanged (it is orthogonal): same answer
    same = np.full((10, 4), np.exp(0.7j))
    np.testing.assert_allclose(cbrute.relu_attention_rope(q, k, v, same, 1e-8), cbrute.relu_attention(q, k, v, 1e-8),
                               rtol=1e-12, atol=1e-13)


# ---------------------------------------------------------------- W8A16 quantiser


def test_quantiser_closed_form():
    w = torch.tensor([[1.27, -0.64, 0.004, 0.0], [-2.0, 0.5, 0.25, 1.0]])
    wq, s = O.quantize_w8(w)
    torch.testing.assert_close(s, torch.tensor([0.01, 2.0 / 127]))
    assert wq.dtype == torch.int8
    assert wq[0].tolist() == [127, -64, 0, 0]
    assert wq[1].tolist() == [-127, 32, 16, 64]  # round-half-even of 31.75, 15.875, 63.5
    assert wq.abs().max() <= 127


def test_quantiser_is_exact_on_grid_weights_and_idempotent():
    g = torch.Generator().manual_seed(0)
    k = torch.randint(-127, 128, (8, 16), generator=g)
    k[:, 0] = 127
    s = 2.0 ** torch.randint(-8, -3, (8,), generator=g).float()
    w = (k.float() * s[:, None] * 1.0)
    wq, s2 = O.quantize_w8(w.bfloat16())
    torch.testing.assert_close(s2, s)
    assert torch.equal(wq, k.to(torch.int8))
    assert torch.equal(O.dequantize_w8(wq, s2), w.bfloat16())
    # quantising the dequantised weight is a fixed point
    wq3, s3 = O.quantize_w8(O.dequantize_w8(wq, s2))
    assert torch.equal(wq3, wq) and torch.equal(s3, s2)


def test_dequantized_block_state_touches_only_the_four_gemm_weights():
    blk = _block(64, dtype=torch.bfloat16)
    sd = blk.state_dict()
    dq = O.dequantized_block_state(sd)
    for key in sd:
        if key in O.W8A16_KEYS:
            assert not torch.equal(sd[key], dq[key])
            assert ((sd[key].float() - dq[key].float()).abs().max() <= sd[key].float().abs().max() / 127 * 0.51 + 1e-3)
        else:
            assert torch.equal(sd[key], dq[key])


# ---- SanaVideoMSBlock (sana_multi_scale_video.py:66-333): pinned by reductions to what is already pinned


def _video_pair(attn_type, ffn_type, seed=0, **kw):
    blk = O.SanaVideoMSBlock(64, 4, mlp_ratio=2.5, attn_type=attn_type, ffn_type=ffn_type, **kw).double()
    O.init_block_(blk, seed)
    with torch.no_grad():
        for n, p in blk.named_parameters():
            if n.endswith("bias") or n.endswith("t_conv.weight"):
                p.copy_(torch.randn(p.shape, generator=torch.Generator().manual_seed(seed + 7), dtype=torch.float64) * 0.05)
    return blk


def test_video_block_with_image_options_is_the_image_block():
    """attn_type="linear", ffn_type="glumbconv", flat t: the video block's forward is SanaMSBlock's (same wiring,
    same keys), so the two restatements must agree exactly on the same weights."""
    vb = _video_pair("linear", "glumbconv")
    ib = O.SanaMSBlock(64, 4, mlp_ratio=2.5, attn_type="linear", ffn_type="glumbconv").double()
    assert list(ib.state_dict()) == list(vb.state_dict())
    ib.load_state_dict(vb.state_dict(), strict=True)
    x, y, t = (a.double() for a in O.block_inputs(2, 6 * 5, 64, n_text=9, seed=1))
    torch.testing.assert_close(vb(x, y, t, THW=(6, 5)), ib(x, y, t, HW=(6, 5)), rtol=0, atol=0)


def test_video_block_frame_aware_conditioning():
    """One modulation row per frame ([B, 1, F, 6C]): equal rows reduce to the flat-t forward; different rows act on
    their own frames only through the modulation (zero gates for one frame leave that frame's residual stream with
    the cross-attention update alone)."""
    vb = _video_pair("chunkcausal", "ChunkGLUMBConvTemp", seed=2, qk_norm=True)
    B, (T, H, W), C = 2, (4, 3, 5), 64
    x, y, t = (a.double() for a in O.block_inputs(B, T * H * W, C, n_text=9, seed=2))
    flat = vb(x, y, t, THW=(T, H, W), chunk_index=[0, 2])
    tf = t.view(B, 1, 1, 6 * C).expand(B, 1, T, 6 * C).contiguous()
    torch.testing.assert_close(vb(x, y, tf, THW=(T, H, W), chunk_index=[0, 2]), flat, rtol=1e-12, atol=1e-12)
    # frame 1 gets gates that cancel the table's: its tokens then only receive x + cross_attn(x, y)
    tf2 = tf.clone().view(B, 1, T, 6, C)
    tf2[:, :, 1, 2] = -vb.scale_shift_table[2]
    tf2[:, :, 1, 5] = -vb.scale_shift_table[5]
    out = vb(x, y, tf2.view(B, 1, T, 6 * C), THW=(T, H, W), chunk_index=[0, 2])
    P = H * W
    want = (x + vb.cross_attn(x, y))[:, P:2 * P]
    torch.testing.assert_close(out[:, P:2 * P], want, rtol=1e-12, atol=1e-12)
    assert (out[:, :P] - (x + vb.cross_attn(x, y))[:, :P]).abs().max() > 1e-3


def test_video_block_streaming_cache_equals_the_chunked_block():
    """cachedcausal + CachedGLUMBConvTemp fed chunk by chunk with the accumulated cache (the pipeline's bookkeeping,
    sana_inference_pipeline.py:242-263) reproduces chunkcausal + ChunkGLUMBConvTemp on the whole sequence, given
    rotary factors that depend on the absolute token position."""
    chunked = _video_pair("chunkcausal", "ChunkGLUMBConvTemp", seed=3)
    cached = O.SanaVideoMSBlock(64, 4, mlp_ratio=2.5, attn_type="cachedcausal", ffn_type="CachedGLUMBConvTemp").double()
    cached.load_state_dict(chunked.state_dict(), strict=True)
    B, (T, H, W), C = 1, (5, 2, 3), 64
    P = H * W
    x, y, t = (a.double() for a in O.block_inputs(B, T * P, C, n_text=9, seed=3))
    theta = torch.rand(T * P, 16, generator=torch.Generator().manual_seed(5), dtype=torch.float64) * 6.283
    freqs = torch.polar(torch.ones_like(theta), theta)[None, None]
    whole = chunked(x, y, t, THW=(T, H, W), rotary_emb=freqs, chunk_index=[0, 2, 3])
    acc, outs = None, []
    for a, b in ((0, 2), (2, 3), (3, 5)):
        cache = [None, None, None] if acc is None else [acc[0], acc[1], acc[2]]
        o, saved = cached(x[:, a * P:b * P], y, t, THW=(b - a, H, W), rotary_emb=freqs[:, :, a * P:b * P],
                          save_kv_cache=True, kv_cache=cache)
        outs.append(o)
        if acc is None:
            acc = [saved[0], saved[1], saved[2]]
        else:   # states add up, the temporal-conv tail is replaced
            acc = [acc[0] + saved[0], acc[1] + saved[1], saved[2]]
    torch.testing.assert_close(torch.cat(outs, 1), whole, rtol=1e-9, atol=1e-9)
