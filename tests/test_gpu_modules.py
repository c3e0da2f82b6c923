"""GPU parity of the drop-in modules against the oracle modules (same state_dict, same seeded inputs)."""
import pytest
import torch

import sana_amd as S
from oracle import sana_oracle as O

pytestmark = pytest.mark.gpu


def rel_l2(a, b):
    return ((a.double() - b.double()).norm() / b.double().norm()).item()


def check(out, ref, what="", block=False):
    """north-star tolerance for the bf16 LiteLA / GLUMBConv outputs: max-abs 2e-2 and
    rel-L2 1e-2.  A whole-block output carries the residual stream (|x| up to ~5,
    where one bf16 unit in the last place is already 3.1e-2), so there the
    max-abs bound is 2e-2 plus one bf16 ulp of the reference value."""
    err = (out.double().cpu() - ref.double()).abs()
    rl = rel_l2(out.cpu(), ref)
    if block:
        bad = (err > 2e-2 + 2.0 ** -7 * ref.double().abs()).sum().item()
        assert bad == 0 and rl <= 1e-2, f"{what}: {bad} elements over tolerance, rel-L2 {rl:.3e}"
    else:
        mx = err.max().item()
        assert mx <= 2e-2 and rl <= 1e-2, f"{what}: max-abs {mx:.3e} rel-L2 {rl:.3e}"


def _pair(C, heads, seed=0):
    ob = O.init_block_(O.SanaMSBlock(C, heads, mlp_ratio=2.5, attn_type="linear", ffn_type="glumbconv", linear_head_dim=32), seed)
    with torch.no_grad():   # non-zero biases exercise every epilogue
        g = torch.Generator().manual_seed(seed + 1)
        for n, p in ob.named_parameters():
            if n.endswith("bias"):
                p.copy_(torch.randn(p.shape, generator=g) * 0.05)
    ob = ob.bfloat16()
    hb = S.SanaMSBlock(C, heads, mlp_ratio=2.5, attn_type="linear", ffn_type="glumbconv", linear_head_dim=32).bfloat16()
    hb.load_state_dict(ob.state_dict(), strict=True)
    return ob, hb


def _ref64(module, *args, **kw):
    """The oracle in fp64 on the bf16-valued weights and inputs: the exact result."""
    import copy
    m = copy.deepcopy(module).double()
    conv = lambda a: a.double() if torch.is_tensor(a) and a.is_floating_point() else a
    return m(*[conv(a) for a in args], **{k: conv(v) for k, v in kw.items()})


@pytest.mark.parametrize("B,HW,C,heads", [(2, (16, 16), 1152, 16), (1, (8, 12), 96, 4)])
def test_litela_and_glumbconv_modules(cuda, B, HW, C, heads):
    ob, hb = _pair(C, heads)
    hb = hb.to(cuda)
    N = HW[0] * HW[1]
    x = torch.randn(B, N, C, generator=torch.Generator().manual_seed(5)).bfloat16()
    with torch.no_grad():
        # attention
        ref = ob.attn.double()(x.double(), HW=HW)
        out = hb.attn(x.to(cuda), HW=HW)
        assert out.dtype == torch.bfloat16 and out.shape == (B, N, C)
        check(out, ref, "LiteLA")
        # attn_matmul, called the way the PAG processor does (channel-major views of the fused buffer)
        qkv = hb.attn.qkv(x.to(cuda)).reshape(B, N, 3, C)
        q, k, v = (t.transpose(-1, -2).reshape(B, C // 32, 32, N) for t in qkv.unbind(2))
        am = hb.attn.attn_matmul(torch.relu(q), torch.relu(k).transpose(-1, -2), v)
        assert am.dtype == torch.float32 and am.shape == (B, C // 32, 32, N)
        am_ref = O.relu_linear_attention(q.double().cpu(), k.double().cpu().transpose(-1, -2), v.double().cpu(), 1e-8)
        assert rel_l2(am.cpu(), am_ref) <= 1e-5
        am.to(torch.bfloat16).view(B, C, N)   # the reshape the PAG processor performs must be a view
        # Mix-FFN
        ref = ob.mlp.double()(x.double(), HW=HW)
        out = hb.mlp(x.to(cuda), HW=HW)
        check(out, ref, "GLUMBConv")
        hb.mlp.round_like_reference = False
        check(hb.mlp(x.to(cuda), HW=HW), ref, "GLUMBConv single rounding")


def test_block_cfg2_shape(cuda):
    """One SanaMSBlock at Sana-600M width, B=4, 32x32 latent, 300 text tokens."""
    C, heads, B, HW = 1152, 16, 4, (32, 32)
    ob, hb = _pair(C, heads, seed=2)
    hb = hb.to(cuda)
    x, y, t = (a.bfloat16() for a in O.block_inputs(B, HW[0] * HW[1], C, seed=2))
    with torch.no_grad():
        ref = _ref64(ob, x, y, t, HW=HW)
        out = hb(x.to(cuda), y.to(cuda), t.to(cuda), HW=HW)
        check(out, ref, "SanaMSBlock vs fp64 oracle", block=True)
        # and against the oracle run as the reference would run it: bf16 on its own device
        ob.attn.fp32_attention = True
        ref16 = ob(x, y, t, HW=HW)
        assert rel_l2(out.cpu(), ref16) <= 1e-2
        # text mask path
        mask = torch.ones(B, 300, dtype=torch.long)
        mask[:, 200:] = 0
        out_m = hb(x.to(cuda), y.to(cuda), t.to(cuda), mask=mask.to(cuda), HW=HW)
        check(out_m, _ref64(ob, x, y, t, mask=mask, HW=HW), "masked text", block=True)


def test_block_qk_norm_and_rope(cuda):
    C, heads, B, HW = 96, 4, 2, (6, 8)
    N = HW[0] * HW[1]
    ob = O.init_block_(O.SanaMSBlock(C, heads, mlp_ratio=2.5, attn_type="linear", ffn_type="glumbconv", qk_norm=True), 3).bfloat16()
    hb = S.SanaMSBlock(C, heads, mlp_ratio=2.5, attn_type="linear", ffn_type="glumbconv", qk_norm=True).bfloat16()
    hb.load_state_dict(ob.state_dict(), strict=True)
    hb = hb.to(cuda)
    x, y, t = (a.bfloat16() for a in O.block_inputs(B, N, C, n_text=20, seed=3))
    theta = torch.rand(N, 16, generator=torch.Generator().manual_seed(0)) * 6
    rope = (torch.cos(theta).repeat_interleave(2, 1), torch.sin(theta).repeat_interleave(2, 1))
    with torch.no_grad():
        ob.attn.fp32_attention = True
        ref = ob(x, y, t, HW=HW, image_rotary_emb=rope)
        out = hb(x.to(cuda), y.to(cuda), t.to(cuda), HW=HW, image_rotary_emb=tuple(r.to(cuda) for r in rope))
        assert rel_l2(out.cpu(), ref) <= 1e-2


def test_w8a16_block_matches_dequantised_reference(cuda):
    """cfg4 contract at a reduced batch: the W8A16 block equals the bf16 block
    (and the oracle) run on the dequantised weights."""
    C, heads, B, HW = 2240, 20, 2, (32, 32)
    ob, hb = _pair(C, heads, seed=4)
    dq = O.dequantized_block_state(ob.state_dict())
    ob.load_state_dict(dq)
    hb_dq = S.SanaMSBlock(C, heads, mlp_ratio=2.5, attn_type="linear", ffn_type="glumbconv").bfloat16()
    hb_dq.load_state_dict(dq)
    hb_dq = hb_dq.to(cuda)
    hb = hb.quantize_w8_().to(cuda)   # quantised on the host, like the oracle's dequantised target
    assert hb.attn.qkv.weight is None and hb.attn.qkv.weight_q.dtype == torch.int8
    x, y, t = (a.bfloat16() for a in O.block_inputs(B, HW[0] * HW[1], C, seed=4))
    with torch.no_grad():
        out8 = hb(x.to(cuda), y.to(cuda), t.to(cuda), HW=HW)
        out16 = hb_dq(x.to(cuda), y.to(cuda), t.to(cuda), HW=HW)
        assert torch.equal(out8, out16)       # in-register dequantisation is exact
        check(out8, _ref64(ob, x, y, t, HW=HW), "W8A16 block vs dequantised fp64 oracle", block=True)


def test_chunk_causal_module_and_video_ffn(cuda):
    """cfg5 structure at a reduced width: 21 frames x 30x52 tokens, chunk-causal
    attention followed by the per-frame Mix-FFN."""
    C, B, HW = 96, 1, (21, 30, 52)
    N = HW[0] * HW[1] * HW[2]
    torch.manual_seed(0)
    oa = O.ChunkCausalAttention(C, C, dim=32, eps=1e-8).bfloat16()
    ha = S.ChunkCausalAttention(C, C, dim=32, eps=1e-8).bfloat16()
    ha.load_state_dict(oa.state_dict(), strict=True)
    ha = ha.to(cuda)
    x = torch.randn(B, N, C, generator=torch.Generator().manual_seed(1)).bfloat16()
    with torch.no_grad():
        for chunk_index in ([0, 11], list(range(21)), None):
            ref = oa.double()(x.double(), HW=HW, chunk_index=chunk_index)
            out = ha(x.to(cuda), HW=HW, chunk_index=chunk_index)
            check(out, ref, f"chunk-causal {chunk_index}")
        om = O.GLUMBConv(C, 240, use_bias=(True, True, False)).bfloat16()
        hm = S.GLUMBConv(C, 240, use_bias=(True, True, False)).bfloat16()
        hm.load_state_dict(om.state_dict(), strict=True)
        check(hm.to(cuda)(x.to(cuda), HW=HW), om.double()(x.double(), HW=HW), "per-frame Mix-FFN")


def test_fp16_model_uses_library_gemm_and_hip_attention(cuda):
    C, heads, B, HW = 96, 4, 1, (8, 8)
    ob = O.init_block_(O.SanaMSBlock(C, heads, mlp_ratio=2.5, attn_type="linear", ffn_type="glumbconv"), 6).half()
    hb = S.SanaMSBlock(C, heads, mlp_ratio=2.5, attn_type="linear", ffn_type="glumbconv").half()
    hb.load_state_dict(ob.state_dict(), strict=True)
    hb = hb.to(cuda)
    x, y, t = (a.half() for a in O.block_inputs(B, 64, C, n_text=10, seed=6))
    with torch.no_grad():
        ref = ob.double()(x.double(), y.double(), t.double(), HW=HW)
        out = hb(x.to(cuda), y.to(cuda), t.to(cuda), HW=HW)
    assert rel_l2(out.cpu(), ref) <= 2e-3


def _temp_pair(name, C, Hd, seed):
    om = getattr(O, name)(C, Hd, use_bias=(True, True, False))
    g = torch.Generator().manual_seed(seed)
    with torch.no_grad():
        for n, p in om.named_parameters():
            p.copy_(torch.randn(p.shape, generator=g) * (0.05 if n.endswith("bias") else 0.25 / p[0].numel() ** 0.5 * 2))
    om = om.bfloat16()
    hm = getattr(S, name)(C, Hd, use_bias=(True, True, False)).bfloat16()
    assert list(hm.state_dict()) == list(om.state_dict())
    hm.load_state_dict(om.state_dict(), strict=True)
    return om, hm


@pytest.mark.parametrize("C,Hd", [(96, 240), (128, 320)])
def test_temporal_mix_ffn_variants(cuda, C, Hd):
    """GLUMBConvTemp / ChunkGLUMBConvTemp against the fp64 oracle, and the cached stream against the chunked call.
    C = 128 takes the temporal conv as a GEMM over the token-major frames, C = 96 (not a multiple of the k-tile)
    and the masked call the stock convolution."""
    (T, H, W), B = (6, 5, 7), 2
    P = H * W
    x = torch.randn(B, T * P, C, generator=torch.Generator().manual_seed(11)).bfloat16()
    with torch.no_grad():
        om, hm = _temp_pair("GLUMBConvTemp", C, Hd, 1)
        hm = hm.to(cuda)
        check(hm(x.to(cuda), HW=(T, H, W)), _ref64(om, x, HW=(T, H, W)), "GLUMBConvTemp")
        mask = torch.ones(B, T)
        mask[:, 4:] = 0
        check(hm(x.to(cuda), HW=(T, H, W), frame_valid_mask=mask.to(cuda)),
              _ref64(om, x, HW=(T, H, W), frame_valid_mask=mask), "GLUMBConvTemp masked")
        om, hm = _temp_pair("ChunkGLUMBConvTemp", C, Hd, 2)
        hm = hm.to(cuda)
        full = hm(x.to(cuda), HW=(T, H, W), chunk_index=[0, 1, 4])
        check(full, _ref64(om, x, HW=(T, H, W), chunk_index=[0, 1, 4]), "ChunkGLUMBConvTemp")
        cm = S.CachedGLUMBConvTemp(C, Hd, use_bias=(True, True, False)).bfloat16()
        cm.load_state_dict(om.state_dict(), strict=True)
        cm = cm.to(cuda)
        cache, outs = [None, None, None], []
        for a, b in ((0, 1), (1, 4), (4, 6)):
            o, cache = cm(x[:, a * P:b * P].to(cuda), HW=(b - a, H, W), save_kv_cache=True, kv_cache=cache)
            outs.append(o)
        assert (torch.cat(outs, 1).float() - full.float()).abs().max().item() <= 2 ** -6


@pytest.mark.parametrize("mode", ["pag", "pag_cfg"])
def test_guidance_processor_patched_over_attn_forward(cuda, mode):
    """The sampler's way of enabling perturbed-attention guidance: patch a processor over
    ``block.attn.forward`` (dpm_solver.py:486-524), run the tripled / doubled batch, restore."""
    from sana_amd import pag
    C, heads, HW = 96, 4, (6, 8)
    N = HW[0] * HW[1]
    ob, hb = _pair(C, heads, seed=5)
    hb = hb.to(cuda)
    nb = 2 if mode == "pag" else 3
    x, y, t = (a.bfloat16() for a in O.block_inputs(nb, N, C, n_text=20, seed=5))
    name = "PAGIdentitySelfAttnProcessorLiteLA" if mode == "pag" else "PAGCFGIdentitySelfAttnProcessorLiteLA"
    with torch.no_grad():
        import copy
        o64 = copy.deepcopy(ob).double()
        o64.attn.forward = getattr(O, name)(o64.attn)
        ref = o64(x.double(), y.double(), t.double(), HW=HW)
        plain = hb(x.to(cuda), y.to(cuda), t.to(cuda), HW=HW)
        hb.attn.forward = getattr(pag, name)(hb.attn)
        out = hb(x.to(cuda), y.to(cuda), t.to(cuda), HW=HW)
        check(out, ref, name, block=True)
        # the unperturbed part is what the block computes without the processor; the perturbed part is not
        assert (out[:nb - 1].float() - plain[:nb - 1].float()).abs().max().item() <= 2 ** -5
        assert (out[nb - 1:].float() - plain[nb - 1:].float()).abs().max().item() > 1e-2
        hb.attn.forward = pag.SelfAttnProcessorLiteLA(hb.attn)     # what the sampler leaves behind
        assert torch.equal(hb(x.to(cuda), y.to(cuda), t.to(cuda), HW=HW), plain) or \
            (hb(x.to(cuda), y.to(cuda), t.to(cuda), HW=HW).float() - plain.float()).abs().max().item() <= 2 ** -5


def test_glumbconv_linear_block_and_temporal_variant(cuda):
    """ffn_type="glumbconv_linear" (nn.Linear parameters, basic_modules_linear.py:133-311): the block, the module with
    the HW=None square default, the W8A16 form and the temporal variant against the fp64 oracle."""
    C, heads, B, HW = 256, 8, 2, (12, 12)
    ob = O.init_block_(O.SanaMSBlock(C, heads, mlp_ratio=2.5, attn_type="linear", ffn_type="glumbconv_linear"), 3)
    with torch.no_grad():
        g = torch.Generator().manual_seed(4)
        for n, p in ob.named_parameters():
            if n.endswith("bias"):
                p.copy_(torch.randn(p.shape, generator=g) * 0.05)
    ob = ob.bfloat16()
    hb = S.SanaMSBlock(C, heads, mlp_ratio=2.5, attn_type="linear", ffn_type="glumbconv_linear").bfloat16()
    hb.load_state_dict(ob.state_dict(), strict=True)
    hb = hb.to(cuda)
    x, y, t = (a.bfloat16() for a in O.block_inputs(B, HW[0] * HW[1], C, seed=3))
    with torch.no_grad():
        check(hb(x.to(cuda), y.to(cuda), t.to(cuda), HW=HW), _ref64(ob, x, y, t, HW=HW), "block, linear FFN", block=True)
        ref = _ref64(ob.mlp, x, HW=HW)
        check(hb.mlp(x.to(cuda), HW=HW), ref, "GLUMBConvLinear")
        check(hb.mlp(x.to(cuda)), ref, "GLUMBConvLinear, HW=None")
        check(hb.mlp(x.to(cuda), HW=(2, 12, 6)), _ref64(ob.mlp, x, HW=(2, 12, 6)), "GLUMBConvLinear, video HW")
        # W8A16 against the oracle holding the dequantised weights
        sd = dict(ob.mlp.state_dict())
        for k in ("inverted_conv.linear.weight", "point_conv.linear.weight"):
            sd[k] = O.dequantize_w8(*O.quantize_w8(sd[k]))
        oq = O.GLUMBConvLinear(C, int(C * 2.5), use_bias=(True, True, False)).bfloat16()
        oq.load_state_dict(sd, strict=True)
        hb.mlp.quantize_w8_()
        check(hb.mlp(x.to(cuda), HW=HW), _ref64(oq, x, HW=HW), "GLUMBConvLinear W8A16")
        (T, H, W) = (4, 5, 6)
        om, hm = _temp_pair("GLUMBConvLinearTemp", 128, 320, 7)
        xt = torch.randn(1, T * H * W, 128, generator=torch.Generator().manual_seed(12)).bfloat16()
        check(hm.to(cuda)(xt.to(cuda), HW=(T, H, W)), _ref64(om, xt, HW=(T, H, W)), "GLUMBConvLinearTemp")


def test_empty_inputs(cuda):
    """No batch entries / no tokens: the stock ops of the reference return empty tensors (and a sum over no tokens
    is zero); the drop-in answers the same way without a launch."""
    from sana_amd import ops
    C, heads = 128, 4
    ob, hb = _pair(C, heads)
    hb = hb.to(cuda)
    with torch.no_grad():
        # (the block itself cannot take B = 0: `t.reshape(B, 6, -1)` of sana_multi_scale.py:147 is ambiguous there)
        x0 = torch.zeros(0, 16, C, dtype=torch.bfloat16, device=cuda)
        assert hb.attn(x0, HW=(4, 4)).shape == (0, 16, C)
        assert hb.mlp(x0, HW=(4, 4)).shape == (0, 16, C)
        xn = torch.zeros(2, 0, C, dtype=torch.bfloat16, device=cuda)
        assert hb.attn(xn, HW=(0, 0)).shape == (2, 0, C)
        assert hb.mlp(xn, HW=(0, 0)).shape == (2, 0, C)
        st = ops.linattn_state(xn, xn)
        assert st.shape == (2, C // 32, 1, 33, 32) and st.abs().max().item() == 0.0
        assert ops.linattn_apply(xn, st, 1e-8).shape == (2, 0, C)
        rq, rk = ops.qk_rms(xn, xn, 1e-5)
        assert rq.shape == (2, 0)
        # the oracle agrees on the shapes
        assert ob.attn(x0.cpu(), HW=(4, 4)).shape == (0, 16, C) and ob.mlp(x0.cpu(), HW=(4, 4)).shape == (0, 16, C)


def test_block_replays_from_a_hip_graph(cuda):
    """The whole block (hand-written kernels, stock cross-attention, the cached workspace) captured once into a HIP
    graph: every replay, with eager launches and synchronisations between them, reproduces the eager result bit
    for bit, also after the input buffer's contents change."""
    C, heads, B, HW = 256, 8, 2, (16, 16)
    ob, hb = _pair(C, heads, seed=5)
    hb = hb.to(cuda)
    x, y, t = (a.bfloat16().to(cuda) for a in O.block_inputs(B, HW[0] * HW[1], C, seed=5))
    with torch.no_grad():
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):           # warm-up off the default stream, as capture requires
            for _ in range(2):
                hb(x, y, t, HW=HW)
        torch.cuda.current_stream().wait_stream(side)
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            out = hb(x, y, t, HW=HW)
        for r in range(3):
            if r == 2:
                x.copy_(torch.randn(x.shape, generator=torch.Generator().manual_seed(9)).bfloat16())
            graph.replay()
            torch.cuda.synchronize()
            eager = hb(x, y, t, HW=HW)
            torch.cuda.synchronize()
            assert torch.equal(out, eager), f"replay {r}"
        check(out, _ref64(ob, x.cpu(), y.cpu(), t.cpu(), HW=HW), "graph replay vs fp64 oracle", block=True)


def test_glumbconv_with_dilation_takes_the_logged_stock_depthwise(cuda, caplog):
    """dilation = 2 (`glumbconv_dilate`): no depthwise kernel, so that one stage is the stock convolution -- said
    once on the logger -- between the two MFMA GEMMs; same keys, same result as the oracle."""
    import logging
    from sana_amd import modules as M
    C, Hd, B, HW = 64, 160, 2, (9, 7)
    om = O.GLUMBConv(C, Hd, use_bias=(True, True, False), norm=(None, None, None), act=("silu", "silu", None), dilation=2)
    g = torch.Generator().manual_seed(3)
    with torch.no_grad():
        for p in om.parameters():
            p.copy_(torch.randn(p.shape, generator=g) * 0.2)
    om = om.bfloat16()
    hm = S.GLUMBConv(C, Hd, use_bias=(True, True, False), norm=(None, None, None), act=("silu", "silu", None),
                     dilation=2).bfloat16()
    hm.load_state_dict(om.state_dict(), strict=True)
    hm = hm.to(cuda)
    x = torch.randn(B, HW[0] * HW[1], C, generator=g).bfloat16()
    M._stock_paths_seen.clear()
    with torch.no_grad(), caplog.at_level(logging.WARNING, logger="sana_amd"):
        out = hm(x.to(cuda), HW=HW)
        hm(x.to(cuda), HW=HW)
        ref = _ref64(om, x, HW=HW)
    check(out, ref, "GLUMBConv dilation 2")
    assert sum("dilation 2" in r.getMessage() for r in caplog.records) == 1


def test_graphed_call_replays_a_chain_of_blocks(cuda):
    """sana_amd.GraphedCall: two chained blocks captured once; replays with new inputs equal the eager chain bit for
    bit, with eager work and synchronisations between the replays."""
    C, heads, B, HW = 256, 8, 2, (16, 16)
    blocks = []
    for seed in (11, 12):
        _, hb = _pair(C, heads, seed=seed)
        blocks.append(hb.to(cuda))
    chain = lambda x, y, t: blocks[1](blocks[0](x, y, t, HW=HW), y, t, HW=HW)
    x, y, t = (a.bfloat16().to(cuda) for a in O.block_inputs(B, HW[0] * HW[1], C, seed=13))
    graphed = S.GraphedCall(chain, (x, y, t))
    with torch.no_grad():
        for r in range(3):
            xr = torch.randn(x.shape, generator=torch.Generator().manual_seed(20 + r)).bfloat16().to(cuda)
            out = graphed(xr, y, t)
            torch.cuda.synchronize()
            eager = chain(xr, y, t)
            torch.cuda.synchronize()
            assert torch.equal(out, eager), f"replay {r}"
    with pytest.raises(ValueError):
        graphed(x[:1], y, t)


def test_graphed_call_with_shared_conditioning_and_the_fused_routes(cuda):
    """Two blocks at 4096 rows -- the qkv GEMM with the attention state in its epilogue, the cross-attention's
    residual add in its projection GEMM -- with their StepConditioning evaluated inside the captured step: replays
    equal the eager step bit for bit (every derived weight copy exists before the capture: GraphedCall warms up)."""
    C, heads, B, HW = 288, 3, 2, (64, 32)          # cross-attention heads of 96, linear-attention heads of 32
    blocks = []
    for seed in (21, 22):
        _, hb = _pair(C, heads, seed=seed)
        blocks.append(hb.to(cuda))
    cond = S.StepConditioning(blocks)
    assert B * HW[0] * HW[1] >= blocks[0].attn.STATE_IN_QKV_GEMM_MIN_ROWS

    def step(x, y, t):
        for blk, c in zip(blocks, cond(y, t)):
            x = blk(x, y, t, None, HW, None, **c)
        return x

    x, y, t = (a.bfloat16().to(cuda) for a in O.block_inputs(B, HW[0] * HW[1], C, seed=23))
    graphed = S.GraphedCall(step, (x, y, t))
    with torch.no_grad():
        for r in range(3):
            xr = torch.randn(x.shape, generator=torch.Generator().manual_seed(30 + r)).bfloat16().to(cuda)
            yr = torch.randn(y.shape, generator=torch.Generator().manual_seed(40 + r)).bfloat16().to(cuda)
            out = graphed(xr, yr, t)
            torch.cuda.synchronize()
            eager = step(xr, yr, t)
            torch.cuda.synchronize()
            assert torch.equal(out, eager), f"replay {r}"
        ref_blocks = [b for b in blocks]
        own = xr
        for blk in ref_blocks:                       # and the step without the shared conditioning: same function
            own = blk(own, yr, t, None, HW, None)
        assert ((eager.float() - own.float()).norm() / own.float().norm()).item() <= 2e-3


def test_graph_replay_survives_a_larger_eager_shape(cuda):
    """A captured block holds the raw addresses of the scratch buffers it used (attention partial states, split-k
    planes).  A later, larger eager call makes the library take bigger buffers; the captured ones must stay alive
    and untouched by the allocator, so a replay still reproduces the eager result bit for bit."""
    from sana_amd import ops
    C, heads = 2240, 20
    hb = S.SanaMSBlock(C, heads, mlp_ratio=2.5, attn_type="linear", ffn_type="glumbconv").bfloat16()
    hb.load_state_dict(O.init_block_(O.SanaMSBlock(C, heads, mlp_ratio=2.5, attn_type="linear", ffn_type="glumbconv"),
                                     8).bfloat16().state_dict())
    hb = hb.to(cuda)
    small, big = (32, 32), (64, 64)
    x, y, t = (a.bfloat16().to(cuda) for a in O.block_inputs(1, small[0] * small[1], C, seed=8))
    xb, yb, tb = (a.bfloat16().to(cuda) for a in O.block_inputs(2, big[0] * big[1], C, seed=9))
    lib = ops._lib.load()
    assert lib.sana_hip_linattn_workspace_bytes(1, C // 32, 32, 1, 1024, 1) > 0       # both kinds of scratch are in play
    assert lib.sana_hip_gemm_workspace_bytes(1024, C, 5600) > 0
    with torch.no_grad():
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            for _ in range(2):
                hb(x, y, t, HW=small)
        torch.cuda.current_stream().wait_stream(side)
        want = hb(x, y, t, HW=small).clone()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            out = hb(x, y, t, HW=small)
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out, want)
        held = sum(len(v) for v in ops._workspaces.values())
        for r in range(3):
            hb(xb, yb, tb, HW=big)                    # larger scratch on the eager stream
            junk = [torch.full((1 << 22,), float(r), device=cuda) for _ in range(8)]   # takes whatever was freed
            torch.cuda.synchronize()
            out.zero_()
            graph.replay()
            torch.cuda.synchronize()
            assert torch.equal(out, want), f"replay {r} after a larger eager call"
            del junk
        assert sum(len(v) for v in ops._workspaces.values()) >= held   # nothing the graph may point at was dropped


def test_conditioning_in_another_dtype_is_never_misread(cuda):
    """t in fp32 with a bf16 x: the stock op chain promotes (scale_shift_table + t is fp32) and then fails in its
    first linear, as the reference does; the fused kernels would misread the fp32 rows as bf16 and return garbage.
    The block must end in an error, not a result, and the op wrappers themselves refuse such rows."""
    from sana_amd import ops
    from sana_amd._lib import SanaHipError
    C, heads, B, HW = 96, 4, 2, (8, 12)
    ob, hb = _pair(C, heads, seed=6)
    hb = hb.to(cuda)
    x, y, t = O.block_inputs(B, HW[0] * HW[1], C, n_text=16, seed=6)
    x, y = x.bfloat16(), y.bfloat16()
    with torch.no_grad():
        with pytest.raises(RuntimeError):
            hb(x.to(cuda), y.to(cuda), t.to(cuda), HW=HW)       # t stays fp32
        with pytest.raises(RuntimeError):
            ob(x, y, t, HW=HW)                                  # the stock composition fails the same way
    xd = x.to(cuda)
    rows32 = torch.zeros(B, 1, C, device=cuda)
    with pytest.raises(SanaHipError):
        ops.layernorm_modulate(xd, rows32, rows32)
    w = torch.zeros(C, C, dtype=torch.bfloat16, device=cuda)
    g16 = torch.zeros(B, 1, C, dtype=torch.bfloat16, device=cuda)
    with pytest.raises(SanaHipError):
        ops.gemm_gate_residual(xd, w, torch.zeros(C, device=cuda), g16, xd)                   # fp32 bias
    with pytest.raises(SanaHipError):
        ops.gemm_gate_residual(xd, w.to(torch.int8), None, g16, xd)                           # int8 weight, no scale
    with pytest.raises(SanaHipError):
        ops.gemm_gate_residual(xd, w, None, rows32, xd)                                       # fp32 gate


def test_four_images_at_the_full_shape_equal_one_at_a_time(cuda):
    """B = 4 at the cfg3 shape (65536 tokens x 2240 channels, 4x the benchmark size: 1.5 GB hidden activation, row
    offsets past 2^31 bytes): images do not interact, so the batched block must reproduce the per-image calls --
    the GEMMs, depthwise conv and norms bit for bit per element, the attention up to the fp32 summation order of
    its token splits (which depends on the grid)."""
    C, heads, B, HW = 2240, 20, 4, (128, 128)
    hb = S.SanaMSBlock(C, heads, mlp_ratio=2.5, attn_type="linear", ffn_type="glumbconv").bfloat16()
    hb.load_state_dict(O.init_block_(O.SanaMSBlock(C, heads, mlp_ratio=2.5, attn_type="linear", ffn_type="glumbconv"),
                                     7).bfloat16().state_dict())
    hb = hb.to(cuda)
    x, y, t = (a.bfloat16().to(cuda) for a in O.block_inputs(B, HW[0] * HW[1], C, seed=7))
    with torch.no_grad():
        full = hb(x, y, t, HW=HW)
        ffn = hb.mlp(x, HW=HW)
        for b in range(B):
            one = hb(x[b:b + 1], y[b:b + 1], t[b:b + 1], HW=HW)
            assert rel_l2(full[b:b + 1], one) <= 2e-3
            # a one-ulp flip of an attention output travels through two more GEMMs: a few bf16 ulps at the end
            assert ((full[b:b + 1].float() - one.float()).abs() > 2 ** -5 * one.float().abs() + 4e-3).sum().item() == 0
            assert torch.equal(ffn[b:b + 1], hb.mlp(x[b:b + 1], HW=HW))
        assert torch.isfinite(full.float()).all()


def _video_blocks(C, heads, attn_type, ffn_type, seed, **kw):
    ob = O.SanaVideoMSBlock(C, heads, mlp_ratio=2.5, attn_type=attn_type, ffn_type=ffn_type, **kw)
    O.init_block_(ob, seed)
    with torch.no_grad():
        g = torch.Generator().manual_seed(seed + 1)
        for n, p in ob.named_parameters():
            if n.endswith("bias"):
                p.copy_(torch.randn(p.shape, generator=g) * 0.05)
            elif n.endswith("t_conv.weight"):
                p.copy_(torch.randn(p.shape, generator=g) * (0.3 / p.shape[1]) ** 0.5)
    ob = ob.bfloat16()
    hb = S.SanaVideoMSBlock(C, heads, mlp_ratio=2.5, attn_type=attn_type, ffn_type=ffn_type, **kw).bfloat16()
    hb.load_state_dict(ob.state_dict(), strict=True)
    return ob, hb


def _freqs(N, d, seed):
    theta = torch.rand(N, d // 2, generator=torch.Generator().manual_seed(seed), dtype=torch.float64) * 6.283
    return torch.polar(torch.ones_like(theta), theta)[None, None]


@pytest.mark.parametrize("attn_type,ffn_type,d,C", [("chunkcausal", "ChunkGLUMBConvTemp", 32, 128),
                                                    ("LiteLAReLURope", "GLUMBConvTemp", 112, 224),
                                                    ("ChunkedLiteLAReLURope", "glumbconv", 32, 96),
                                                    ("linear", "glumbconv", 32, 128)])
def test_video_block_matches_oracle(cuda, attn_type, ffn_type, d, C):
    """SanaVideoMSBlock (sana_multi_scale_video.py:66-333) against the fp64 oracle: flat conditioning, one
    modulation row per frame, text mask, block_hook."""
    B, (T, H, W) = 2, (4, 5, 6)
    N = T * H * W
    ob, hb = _video_blocks(C, 4, attn_type, ffn_type, seed=d, qk_norm=True, linear_head_dim=d)
    hb = hb.to(cuda)
    x, y, t = (a.bfloat16() for a in O.block_inputs(B, N, C, n_text=40, seed=d))
    # LiteLA takes the real-valued (cos, sin) form of the rotary embedding, applied before the ReLU: none here
    freqs = _freqs(N, d, 3) if attn_type != "linear" else None
    kw = {"chunk_index": [0, 1, 3]} if attn_type == "chunkcausal" else {}
    with torch.no_grad():
        ref = _ref64(ob, x, y, t, THW=(T, H, W), rotary_emb=freqs, **kw)
        seen = {}
        hb.block_hook = lambda **feats: seen.update(feats)
        dfreqs = None if freqs is None else freqs.to(cuda)
        out = hb(x.to(cuda), y.to(cuda), t.to(cuda), THW=(T, H, W), rotary_emb=dfreqs, **kw)
        check(out, ref, f"{attn_type}/{ffn_type}", block=True)
        assert set(seen) == {"x_in", "x_self_attn", "x_cross_attn", "x_ffn"} and torch.equal(seen["x_ffn"], out)
        hb.block_hook = None
        tf = (torch.randn(B, 1, T, 6 * C, generator=torch.Generator().manual_seed(8)) * 0.3).bfloat16()
        mask = torch.ones(B, 40, dtype=torch.long)
        mask[:, 25:] = 0
        ref = _ref64(ob, x, y, tf, mask=mask, THW=(T, H, W), rotary_emb=freqs, **kw)
        out = hb(x.to(cuda), y.to(cuda), tf.to(cuda), mask=mask.to(cuda), THW=(T, H, W), rotary_emb=dfreqs, **kw)
        check(out, ref, f"{attn_type}/{ffn_type}, per-frame conditioning", block=True)


def test_video_block_streaming_cache_equals_chunked_block(cuda):
    """cachedcausal + CachedGLUMBConvTemp fed chunk by chunk with the accumulated cache against chunkcausal +
    ChunkGLUMBConvTemp on the whole sequence (both on the HIP path), and the whole against the fp64 oracle."""
    C, d, B, (T, H, W) = 128, 32, 1, (5, 4, 6)
    P = H * W
    ob, hb = _video_blocks(C, 4, "chunkcausal", "ChunkGLUMBConvTemp", seed=11, linear_head_dim=d)
    hc = S.SanaVideoMSBlock(C, 4, mlp_ratio=2.5, attn_type="cachedcausal", ffn_type="CachedGLUMBConvTemp",
                            linear_head_dim=d).bfloat16()
    hc.load_state_dict(hb.state_dict(), strict=True)
    hb, hc = hb.to(cuda), hc.to(cuda)
    x, y, t = (a.bfloat16() for a in O.block_inputs(B, T * P, C, n_text=20, seed=11))
    freqs = _freqs(T * P, d, 4)
    with torch.no_grad():
        whole = hb(x.to(cuda), y.to(cuda), t.to(cuda), THW=(T, H, W), rotary_emb=freqs.to(cuda), chunk_index=[0, 2, 3])
        check(whole, _ref64(ob, x, y, t, THW=(T, H, W), rotary_emb=freqs, chunk_index=[0, 2, 3]), "chunked video block",
              block=True)
        acc, outs = None, []
        for a, b in ((0, 2), (2, 3), (3, 5)):
            cache = [None, None, None] if acc is None else list(acc)
            o, saved = hc(x[:, a * P:b * P].to(cuda), y.to(cuda), t.to(cuda), THW=(b - a, H, W),
                          rotary_emb=freqs[:, :, a * P:b * P].to(cuda), save_kv_cache=True, kv_cache=cache)
            outs.append(o)
            acc = S.accumulate_kv_cache(acc, saved)
        stream = torch.cat(outs, 1)
        assert rel_l2(stream, whole) <= 3e-3
        assert ((stream.float() - whole.float()).abs() > 2 ** -5 * whole.float().abs() + 4e-3).sum().item() == 0
