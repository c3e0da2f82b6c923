"""The benchmark configurations at their FULL sizes, worded as the configurations word them, against the oracle
run on the host in fp32 with ``fp32_attention = True`` (the reference's arithmetic with exact products; every
weight and input is a bf16 value, so the only differences are the HIP path's bf16 roundings and summation order):

  cfg3  one SanaMSBlock at B=1, N=128x128, C=2240 -- and all 20 blocks of the denoising step ``bench.py`` times,
        each against the oracle block on the same input, plus the drift of the free-running chain
  cfg4  W8A16 at B=16, N=1024 (16384 rows: the route that expands the int8 weight per call) against the oracle
        on the dequantised weights
  cfg5  chunk-causal attention at C=2240 (70 heads of 32), 21 x 30 x 52 tokens, chunk_index [0, 11] and one chunk
        per frame, followed by the per-frame Mix-FFN
  io-dtype attention (``fp32_attention = False``, sana_blocks.py:251-260): the measured distance between the HIP
        kernels (always fp32 state) and the reference's bf16-state mode
"""
import math

import pytest
import torch

import bench
import sana_amd as S
from oracle import sana_oracle as O

pytestmark = pytest.mark.gpu

C, HEADS_X = bench.C, bench.HEADS_X


def rel_l2(a, b):
    return ((a.double() - b.double()).norm() / b.double().norm()).item()


def check_block(out, ref, what):
    """Whole-block tolerance: rel-L2 1e-2 and max-abs 2e-2 plus one bf16 ulp of the value (the residual stream
    reaches |x| of several units, where one bf16 ulp alone exceeds 2e-2)."""
    err = (out.double().cpu() - ref.double()).abs()
    rl = rel_l2(out.cpu(), ref)
    bad = (err > 2e-2 + 2.0 ** -7 * ref.double().abs()).sum().item()
    assert bad == 0 and rl <= 1e-2, f"{what}: {bad} elements over tolerance, max-abs {err.max().item():.3e}, rel-L2 {rl:.3e}"
    return rl


def check_module(out, ref, what):
    mx = (out.double().cpu() - ref.double()).abs().max().item()
    rl = rel_l2(out.cpu(), ref)
    assert mx <= 2e-2 and rl <= 1e-2, f"{what}: max-abs {mx:.3e} rel-L2 {rl:.3e}"
    return mx, rl


def oracle_block(state):
    ob = O.SanaMSBlock(C, HEADS_X, mlp_ratio=bench.MLP_RATIO, attn_type="linear", ffn_type="glumbconv")
    ob.load_state_dict({k: v.float() for k, v in state.items()})
    ob.attn.fp32_attention = True
    return ob


def hip_block(state, dev):
    hb = S.SanaMSBlock(C, HEADS_X, mlp_ratio=bench.MLP_RATIO, attn_type="linear", ffn_type="glumbconv").bfloat16()
    hb.load_state_dict(state)
    return hb.to(dev)


def test_cfg3_all_twenty_blocks_and_chain_drift(cuda):
    """The 20 blocks bench.py chains (same seeds, same inputs).  Block i of the HIP path and of the oracle both
    take the oracle chain's running activation (rounded to bf16, as the reference's own bf16 chain hands it on):
    per-block parity at the full shape.  Beside it the HIP chain runs freely from x0; its distance from the oracle
    chain is the accumulated drift: bounded by 3e-3 * sqrt(blocks) in rel-L2 (one block contributes ~2e-3, mostly
    the bf16 rounding of the residual stream it hands on; independent roundings add in quadrature: measured
    1.8e-3 after one block, 1.06e-2 after all twenty).
    A third chain shows whose drift that is: the oracle itself in bf16 on the GPU (stock PyTorch ops with
    ``fp32_attention``: the reference's own arithmetic at the precision it runs in), free-running from the same x0.
    The HIP chain must end no further from the fp32 chain than 1.1 x that stock bf16 chain does."""
    HW = (128, 128)
    x, y, t = (a.bfloat16() for a in bench.make_inputs(1, HW[0] * HW[1]))
    yd, td = y.to(cuda), t.to(cuda)
    ref_run, hip_run, stock_run = x.float(), x.to(cuda), x.to(cuda)
    drift = stock_drift = 0.0
    with torch.no_grad():
        for i in range(bench.DEPTH):
            state = bench.make_state(i)
            ob, hb = oracle_block(state), hip_block(state, cuda)
            xin = ref_run.bfloat16()
            ref_run = ob(xin.float(), y.float(), t.float(), HW=HW)
            rl = check_block(hb(xin.to(cuda), yd, td, HW=HW), ref_run, f"cfg3 block {i}")
            hip_run = hb(hip_run, yd, td, HW=HW)
            drift = rel_l2(hip_run.cpu(), ref_run)
            ob16 = ob.bfloat16().to(cuda)             # the same block as stock bf16 ops on the GPU
            ob16.attn.fp32_attention = True
            stock_run = ob16(stock_run, yd, td, HW=HW)
            stock_drift = rel_l2(stock_run.cpu(), ref_run)
            print(f"block {i:2d}: rel-L2 on the oracle's input {rl:.2e}; free-running chain drift {drift:.2e} "
                  f"(stock bf16 chain: {stock_drift:.2e}); |x| rms {ref_run.pow(2).mean().sqrt().item():.2f}", flush=True)
            assert drift <= 3e-3 * math.sqrt(i + 1), f"chain drift after {i + 1} blocks: {drift:.3e}"
            del ob, hb, ob16
    assert drift <= 1.1 * stock_drift, f"HIP chain drift {drift:.3e} against the stock bf16 chain's {stock_drift:.3e}"


def test_step_conditioning_shared_by_the_blocks(cuda):
    """Three blocks of the step with their text keys / values and modulation rows computed at once
    (``StepConditioning``: one GEMM over the stacked kv_linear weights, one add), each against the oracle block on
    the oracle chain's running activation and against the same block computing its own: the modulation rows are the same add (bit-identical), the keys /
    values one bf16 ulp apart at most (same products, another fp32 summation order), and a changed parameter is
    picked up by the next call.  B=2 with a text mask; 4096 rows and 1024 rows (both cross-attention routes)."""
    states = [bench.make_state(i) for i in range(3)]
    obs = [oracle_block(st) for st in states]
    hbs = [hip_block(st, cuda) for st in states]
    cond = S.StepConditioning(hbs)
    for B, HW in ((2, (64, 32)), (1, (32, 32))):
        x, y, t = (a.bfloat16() for a in bench.make_inputs(B, HW[0] * HW[1]))
        mask = torch.ones(B, y.shape[1], dtype=torch.int64)
        mask[-1, 200:] = 0
        xd, yd, td, md = x.to(cuda), y.to(cuda), t.to(cuda), mask.to(cuda)
        with torch.no_grad():
            cs = cond(yd, td)
            assert len(cs) == 3
            ref = x.float()
            for i, (ob, hb, c) in enumerate(zip(obs, hbs, cs)):
                assert torch.equal(c["modulation"], hb.scale_shift_table[None] + td.reshape(B, 6, -1))
                kv = torch.nn.functional.linear(yd, hb.cross_attn.kv_linear.weight, hb.cross_attn.kv_linear.bias)
                assert c["text_kv"].shape == kv.shape
                assert ((c["text_kv"].float() - kv.float()).abs() <= 2.0 ** -7 * kv.float().abs() + 1e-5).all()
                xin = ref.bfloat16()                      # every block on the oracle chain's running activation
                ref = ob(xin.float(), y.float(), t.float(), mask=mask, HW=HW)
                h_shared = hb(xin.to(cuda), yd, td, md, HW, **c)
                check_block(h_shared, ref, f"block {i} with shared conditioning, B={B}")
                assert rel_l2(h_shared.cpu(), hb(xin.to(cuda), yd, td, md, HW).cpu()) <= 2e-3
    with torch.no_grad():
        hbs[1].cross_attn.kv_linear.bias.add_(1.0)
        hbs[2].scale_shift_table.mul_(2.0)
        cs = cond(yd, td)
        kv = torch.nn.functional.linear(yd, hbs[1].cross_attn.kv_linear.weight, hbs[1].cross_attn.kv_linear.bias)
        assert ((cs[1]["text_kv"].float() - kv.float()).abs() <= 2.0 ** -7 * kv.float().abs() + 1e-5).all()
        assert torch.equal(cs[2]["modulation"], hbs[2].scale_shift_table[None] + td.reshape(1, 6, -1))
        assert cond(yd.float(), td.float()) == [{}, {}, {}]          # outside bf16: the blocks compute their own


def test_cfg4_w8a16_block_at_batch_16(cuda):
    """Every qkv / proj / 1x1-conv weight int8 per output channel, B=16 images of 1024 tokens: 16384 rows, so the
    GEMMs take the route that expands the int8 weight to bf16 once per call.  Bit-identical to the bf16 block on
    the dequantised weights, and within the block tolerance of the oracle on the dequantised weights."""
    B, HW = 16, (32, 32)
    state = bench.make_state(3)
    g = torch.Generator().manual_seed(11)
    for k in state:
        if k.endswith("bias"):
            state[k] = (torch.randn(state[k].shape, generator=g) * 0.05).bfloat16()
    dq = O.dequantized_block_state(state)
    ob = oracle_block(dq)
    hb_dq = hip_block(dq, cuda)
    hb = S.SanaMSBlock(C, HEADS_X, mlp_ratio=bench.MLP_RATIO, attn_type="linear", ffn_type="glumbconv").bfloat16()
    hb.load_state_dict(state)
    hb = hb.quantize_w8_().to(cuda)
    assert hb.mlp.inverted_conv.conv.weight is None and hb.attn.proj.weight_q.dtype == torch.int8
    x, y, t = (a.bfloat16() for a in bench.make_inputs(B, HW[0] * HW[1], seed=44))
    with torch.no_grad():
        out8 = hb(x.to(cuda), y.to(cuda), t.to(cuda), HW=HW)
        out16 = hb_dq(x.to(cuda), y.to(cuda), t.to(cuda), HW=HW)
        assert torch.equal(out8, out16)
        ref = ob(x.float(), y.float(), t.float(), HW=HW)
    rl = check_block(out8, ref, "cfg4 W8A16 block, B=16")
    print(f"cfg4 B=16: rel-L2 {rl:.2e} vs the dequantised fp32 oracle", flush=True)


@pytest.mark.parametrize("chunk_index", [[0, 11], list(range(21))], ids=["chunks_0_11", "one_chunk_per_frame"])
def test_cfg5_chunk_causal_attention_and_per_frame_ffn_at_full_width(cuda, chunk_index):
    """C=2240, 70 heads x 32, 21 frames x 30x52 tokens (N=32760), B=1, bf16 I/O with fp32 state: every frame-chunk
    attends to the running sum of the states of all previous chunks plus its own; then the Mix-FFN with the
    depthwise 3x3 per frame."""
    T, H, W = 21, 30, 52
    N = T * H * W
    state = bench.make_state(5)
    g = torch.Generator().manual_seed(12)
    oa = O.ChunkCausalAttention(C, C, heads=C // 32, eps=1e-8)
    oa.load_state_dict({"qkv.weight": state["attn.qkv.weight"].float(), "proj.weight": state["attn.proj.weight"].float(),
                        "proj.bias": (torch.randn(C, generator=g) * 0.05).bfloat16().float()})
    oa.fp32_attention = True
    ha = S.ChunkCausalAttention(C, C, heads=C // 32, eps=1e-8).bfloat16()
    ha.load_state_dict({k: v.bfloat16() for k, v in oa.state_dict().items()})
    ha = ha.to(cuda)
    om = O.GLUMBConv(C, bench.HID, use_bias=(True, True, False), norm=(None, None, None), act=("silu", "silu", None))
    om.load_state_dict({k[4:]: (v.float() if not k.endswith("bias") else
                                (torch.randn(v.shape, generator=g) * 0.05).bfloat16().float())
                        for k, v in state.items() if k.startswith("mlp.")})
    hm = S.GLUMBConv(C, bench.HID, use_bias=(True, True, False), norm=(None, None, None),
                     act=("silu", "silu", None)).bfloat16()
    hm.load_state_dict({k: v.bfloat16() for k, v in om.state_dict().items()})
    hm = hm.to(cuda)
    x = torch.randn(1, N, C, generator=g).bfloat16()
    with torch.no_grad():
        ref_a = oa(x.float(), HW=(T, H, W), chunk_index=list(chunk_index))
        out_a = ha(x.to(cuda), HW=(T, H, W), chunk_index=list(chunk_index))
        mx, rl = check_module(out_a, ref_a, f"cfg5 attention {chunk_index[:3]}..")
        print(f"cfg5 attention, {len(chunk_index)} chunks: max-abs {mx:.2e} rel-L2 {rl:.2e}", flush=True)
        # the Mix-FFN on the attention's output (rounded to bf16: what the next module of a bf16 model receives)
        h = ref_a.bfloat16()
        ref_m = om(h.float(), HW=(T, H, W))
        out_m = hm(h.to(cuda), HW=(T, H, W))
        mx, rl = check_module(out_m, ref_m, "cfg5 per-frame Mix-FFN")
        print(f"cfg5 per-frame Mix-FFN: max-abs {mx:.2e} rel-L2 {rl:.2e}", flush=True)


def test_io_dtype_attention_mode_measured_distance(cuda):
    """``fp32_attention`` False (forced for bf16 inference by app/sana_pipeline.py:141) makes the reference round
    the state ``vk`` and the numerator / denominator to bf16 before the fp32 divide (sana_blocks.py:251-260).
    The HIP kernels always keep the fp32 state.  This records how far apart the two modes are at the cfg2
    attention shape (B=4, N=1024, C=1152) and holds the HIP output to the tolerance against BOTH."""
    B, N, Cc = 4, 1024, 1152
    g = torch.Generator().manual_seed(21)
    om = O.LiteLA(Cc, Cc, heads=Cc // 32, eps=1e-8)
    with torch.no_grad():
        for p in om.parameters():
            p.copy_(torch.nn.init.trunc_normal_(torch.empty(p.shape), std=0.02, generator=g))
    om = om.bfloat16()
    hm = S.LiteLA(Cc, Cc, heads=Cc // 32, eps=1e-8).bfloat16()
    hm.load_state_dict(om.state_dict())
    hm = hm.to(cuda)
    x = torch.randn(B, N, Cc, generator=g).bfloat16()
    with torch.no_grad():
        out = hm(x.to(cuda)).cpu()
        om.fp32_attention = False
        ref_io = om(x)                       # bf16 module, bf16 state: the io-dtype mode as the reference runs it
        om.fp32_attention = True
        ref_32 = om(x)                       # bf16 module, fp32 state
        import copy
        exact = copy.deepcopy(om).double()(x.double())
    d_io, d_32, modes = rel_l2(out, ref_io), rel_l2(out, ref_32), rel_l2(ref_io, ref_32)
    e_hip, e_io, e_32 = rel_l2(out, exact), rel_l2(ref_io, exact), rel_l2(ref_32, exact)
    print(f"rel-L2: HIP vs io-dtype mode {d_io:.2e}, HIP vs fp32-attention mode {d_32:.2e}, the two reference modes "
          f"apart {modes:.2e}; against fp64: HIP {e_hip:.2e}, io-dtype {e_io:.2e}, fp32-attention {e_32:.2e}", flush=True)
    for ref, what in ((ref_io, "io-dtype mode"), (ref_32, "fp32-attention mode")):
        mx = (out.double() - ref.double()).abs().max().item()
        assert mx <= 2e-2 and rel_l2(out, ref) <= 1e-2, f"LiteLA vs {what}: max-abs {mx:.3e}"
    assert e_hip <= e_io * 1.05   # keeping the fp32 state is never the less accurate choice
