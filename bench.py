#!/usr/bin/env python3
"""Benchmark of the SanaMSBlock hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

A *step* is one denoising step of the Sana-1.6B DiT blocks at 4096x4096:
20 random-init SanaMSBlocks chained on one batch (B=1, N=128x128=16384 tokens,
C=2240, 70 heads x 32, Mix-FFN hidden 5600, 300 text tokens), bf16, inputs
resident in HBM.  ``value`` is the block forward latency in ms (step / 20).

The JSON line also carries, measured in the same run with HIP events on the
launch stream:
  roofline       the dominant kernel (the inverted-conv GEMM) against the
                 MI355X dense bf16 MFMA peak,
  kernels        every hand-written kernel of the block against its roofline
                 (HBM 8 TB/s for the attention pair, the depthwise kernel and
                 the LayerNorm+modulate kernel, 2.5 PFLOP/s for the GEMMs),
  images_per_s   B / (20 x block latency) at the 1024px shape (B=16, N=1024),
                 bf16 and W8A16: DiT blocks of ONE denoising step only,
  cpu_baseline   the oracle block (stock PyTorch, fp32) on the host cores, one
                 block of the same workload.

``--kernels-only`` runs just the per-kernel section (the command the rocprofv3
summaries under profiles/ were taken with).  ``roofline.traffic`` is not
measurable from inside the process: it is the HBM byte count of one launch of
the dominant kernel from two ``rocprofv3 --pmc`` runs of ``--kernels-only --cfg3-only``
(FETCH_SIZE, WRITE_SIZE), read at run time from profiles/kernels_cfg3_hbm_traffic.txt.
``configs`` holds the other configurations of the benchmark definition beside the
headline: cfg1 (the LiteLA op alone, fp32, eps 1e-15), cfg2 (one Sana-600M block,
B=4), cfg4 (the W8A16 block at B=16 x 1024 tokens) and cfg5 (chunk-causal attention
with 70 heads of 32 on 21 x 30 x 52 tokens + the per-frame Mix-FFN), each with the
oracle timed on the host cores; ``kernels`` also lists cfg2's four GEMMs with the
library's time beside each.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

import torch

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

TRAFFIC_PROFILE = os.path.join(ROOT, "profiles", "kernels_cfg3_hbm_traffic.txt")
DOMINANT_KERNEL_ROW = "gemm4_kernel<false, 2, 4>"   # the inverted-conv GEMM (bias + SiLU epilogue, 256-wide channel tile)


def dominant_kernel_traffic_bytes():
    """HBM-side bytes per launch of the dominant kernel, read from the committed rocprofv3 --pmc summary (columns
    read_MB and write_MB of its row: FETCH_SIZE / WRITE_SIZE scaled by what a plain copy of known size reads
    on the same counters).  None when the summary or the row is missing."""
    try:
        for line in open(TRAFFIC_PROFILE):
            if line.startswith(DOMINANT_KERNEL_ROW):
                cols = line.split()[-7:]   # FETCH_SIZE read_MB alg_rd_MB WRITE_SIZE write_MB alg_wr_MB traffic/alg
                return int(round((float(cols[1]) + float(cols[4])) * 1e6))   # read_MB + write_MB
    except (OSError, ValueError, IndexError):
        pass
    return None


HBM_PEAK_GBS = 8000.0          # MI355X HBM3E, published
MFMA_BF16_PEAK_TFLOPS = 2500.0  # MI355X dense bf16, published

DEPTH, C, HEADS_X, MLP_RATIO, N_TEXT = 20, 2240, 20, 2.5, 300   # Sana-1.6B (depth 20, width 2240, 20 cross-attn heads)
HID = int(C * MLP_RATIO)


def make_state(seed: int, dtype=torch.bfloat16) -> dict:
    """Random init of one block: trunc-normal(std 0.02) weights, zero biases,
    scale_shift_table = randn(6, C) / sqrt(C)."""
    g = torch.Generator().manual_seed(seed)

    def tn(*shape):
        w = torch.empty(*shape)
        torch.nn.init.trunc_normal_(w, std=0.02, generator=g)
        return w.to(dtype)

    z = lambda *s: torch.zeros(*s, dtype=dtype)
    return {
        "scale_shift_table": (torch.randn(6, C, generator=g) / C ** 0.5).to(dtype),
        "attn.qkv.weight": tn(3 * C, C), "attn.proj.weight": tn(C, C), "attn.proj.bias": z(C),
        "cross_attn.q_linear.weight": tn(C, C), "cross_attn.q_linear.bias": z(C),
        "cross_attn.kv_linear.weight": tn(2 * C, C), "cross_attn.kv_linear.bias": z(2 * C),
        "cross_attn.proj.weight": tn(C, C), "cross_attn.proj.bias": z(C),
        "mlp.inverted_conv.conv.weight": tn(2 * HID, C, 1, 1), "mlp.inverted_conv.conv.bias": z(2 * HID),
        "mlp.depth_conv.conv.weight": tn(2 * HID, 1, 3, 3), "mlp.depth_conv.conv.bias": z(2 * HID),
        "mlp.point_conv.conv.weight": tn(C, HID, 1, 1),
    }


def make_inputs(B: int, N: int, seed: int = 1000):
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(B, N, C, generator=g)
    y = torch.randn(B, N_TEXT, C, generator=g)
    t = torch.randn(B, 6 * C, generator=g) * 0.02
    return x, y, t


def event_time_us(fn, iters: int, warmup: int, repeats: int = 3) -> float:
    """Average duration of one call, HIP events on the stream the kernels are launched on.  The chip
    idles (and drops its clocks) while the host prepares the next operand set, so the warm-up runs
    for at least 0.1 s of GPU time, and the figure is the median of ``repeats`` timed regions of
    ``iters`` back-to-back calls each."""
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    done, spent_ms = 0, 0.0
    while done < warmup or spent_ms < 100.0:
        n = max(warmup - done, 5)
        e0.record()
        for _ in range(n):
            fn()
        e1.record()
        torch.cuda.synchronize()
        spent_ms += e0.elapsed_time(e1)
        done += n
    times = []
    for _ in range(repeats):
        e0.record()
        for _ in range(iters):
            fn()
        e1.record()
        torch.cuda.synchronize()
        times.append(e0.elapsed_time(e1) * 1e3 / iters)
    return sorted(times)[len(times) // 2]


def kernel_rooflines(dev, iters=50, warmup=10, stock_conv=False, cfg3_only=False):
    """Each hand-written kernel alone at the cfg3 shape (B=1, N=16384)."""
    from sana_amd import ops

    B, N, M = 1, 16384, 16384
    g = torch.Generator().manual_seed(7)
    rows = []

    def add(name, bound, work, t_us, note):
        if bound == "hbm":
            ach, peak, unit = work / t_us / 1e3, HBM_PEAK_GBS, "GB/s"
        else:
            ach, peak, unit = work / t_us / 1e6, MFMA_BF16_PEAK_TFLOPS, "TFLOP/s"
        rows.append({"kernel": name, "bound": bound, "us": round(t_us, 2), "achieved": round(ach, 1), "peak": peak,
                     "unit": unit, "frac": round(ach / peak, 4), "work": work, "note": note})

    qkv = torch.randn(B, N, 3, C, generator=g).bfloat16().to(dev)
    q, k, v = qkv[:, :, 0], qkv[:, :, 1], qkv[:, :, 2]
    state = ops.linattn_state(k, v)
    out = torch.empty(B, N, C, dtype=torch.bfloat16, device=dev)
    la_bytes = 2 * M * C * 2 + B * (C // 32) * 33 * 32 * 4
    add("linattn_state", "hbm", la_bytes, event_time_us(lambda: ops.linattn_state(k, v), iters, warmup),
        "2*M*C*2 B (K,V read) + state write")
    add("linattn_apply", "hbm", la_bytes,
        event_time_us(lambda: ops.linattn_apply(q, state, 1e-8, out=out), iters, warmup),
        "M*C*2 B (Q read) + M*C*2 B (out write) + state read")
    if not cfg3_only:
        _kernel_rooflines_other_shapes(dev, add, qkv, state, out, la_bytes, g, iters, warmup)
    _kernel_rooflines_ffn(dev, add, rows, g, iters, warmup, stock_conv, cfg3_only)
    if not cfg3_only:
        _kernel_rows_qk_norm_and_cfg2(dev, add, rows, g)
    # plain device copy as a bandwidth yardstick of this box
    src = torch.empty(256 << 20, dtype=torch.uint8, device=dev)
    dst = torch.empty_like(src)
    t_us = event_time_us(lambda: dst.copy_(src), 20, 5)
    copy_gbs = 2 * src.numel() / t_us / 1e3
    for r in rows:   # the HBM-bound rows once more against what a plain copy reaches on this box
        if r["bound"] == "hbm":
            r["frac_of_copy_rate"] = round(r["achieved"] / copy_gbs, 3)
    return rows, round(copy_gbs, 1)


def _kernel_rooflines_other_shapes(dev, add, qkv, state, out, la_bytes, g, iters, warmup):
    """The attention phases with q/k norm + rotary embedding on load, the chunk-causal video shape and the
    112-wide heads (skipped by --cfg3-only, so a counter run sees every template instance at one shape only)."""
    from sana_amd import ops

    B, N, M = 1, 16384, 16384
    q, k, v = qkv[:, :, 0], qkv[:, :, 1], qkv[:, :, 2]
    # the same two phases with q/k RMSNorm and the rotary embedding applied on load (LiteLAReLURope), plus
    # the statistics pass they need; and the chunk-causal video shape (21 frames x 30x52 tokens, one chunk per frame)
    wn = (1 + 0.1 * torch.randn(C, generator=g)).bfloat16().to(dev)
    theta = torch.rand(N, 16, generator=g, dtype=torch.float64) * 6.283
    rope = ops.rope_table(torch.polar(torch.ones_like(theta), theta), N, dev)
    rq, rk = ops.qk_rms(q, k, 1e-5)
    add("qk_rms", "hbm", 2 * M * C * 2 + 2 * M * 4, event_time_us(lambda: ops.qk_rms(q, k, 1e-5), iters, warmup),
        "2*M*C*2 B (Q,K read) + 2*M*4 B")
    pre_k, pre_q = ops.QkPre(rk, wn, rope), ops.QkPre(rq, wn, rope)
    rope_bytes = M * 16 * 2 * 4 + M * 4
    add("linattn_state_norm_rope", "hbm", la_bytes + rope_bytes,
        event_time_us(lambda: ops.linattn_state(k, v, pre=pre_k), iters, warmup),
        "as linattn_state + rope table (128 B/token) + 1/rms (4 B/token)")
    add("linattn_apply_norm_rope", "hbm", la_bytes + rope_bytes,
        event_time_us(lambda: ops.linattn_apply(q, state, 1e-8, out=out, pre=pre_q), iters, warmup),
        "as linattn_apply + rope table + 1/rms")
    Nv, hw = 21 * 30 * 52, 30 * 52
    qkv5 = torch.randn(1, Nv, 3, C, generator=g).bfloat16().to(dev)
    starts = [f * hw for f in range(21)]
    st5 = ops.linattn_state(qkv5[:, :, 1], qkv5[:, :, 2], starts, causal=True)
    out5 = torch.empty(1, Nv, C, dtype=torch.bfloat16, device=dev)
    la5 = 2 * Nv * C * 2 + 21 * (C // 32) * 33 * 32 * 4
    add("linattn_state_chunk_causal_cfg5", "hbm", la5,
        event_time_us(lambda: ops.linattn_state(qkv5[:, :, 1], qkv5[:, :, 2], starts, causal=True), iters, warmup),
        "cfg5: N=32760, 21 chunks; K,V read + 21 states")
    add("linattn_apply_chunk_causal_cfg5", "hbm", la5,
        event_time_us(lambda: ops.linattn_apply(qkv5[:, :, 0], st5, 1e-8, starts, out=out5), iters, warmup),
        "cfg5: Q read + out write + 21 states")
    # the reference's own chunking of that shape: two chunks, frames [0, 11) and [11, 21)
    starts2 = [0, 11 * hw]
    st5b = ops.linattn_state(qkv5[:, :, 1], qkv5[:, :, 2], starts2, causal=True)
    la5b = 2 * Nv * C * 2 + 2 * (C // 32) * 33 * 32 * 4
    add("linattn_state_chunk_causal_cfg5_chunks_0_11", "hbm", la5b,
        event_time_us(lambda: ops.linattn_state(qkv5[:, :, 1], qkv5[:, :, 2], starts2, causal=True), iters, warmup),
        "cfg5: N=32760, chunk_index [0, 11]; K,V read + 2 states")
    add("linattn_apply_chunk_causal_cfg5_chunks_0_11", "hbm", la5b,
        event_time_us(lambda: ops.linattn_apply(qkv5[:, :, 0], st5b, 1e-8, starts2, out=out5), iters, warmup),
        "cfg5: chunk_index [0, 11]; Q read + out write + 2 states")
    del st5b
    # the same video shape with 112-wide heads (linear_head_dim = 112: 20 heads at C = 2240), q/k RMSNorm and rotary
    # embedding on load as the video blocks use them; whole sequence as one chunk, and 21 causal chunks
    D2 = 112
    h2 = C // D2
    rq5, rk5 = ops.qk_rms(qkv5[:, :, 0], qkv5[:, :, 1], 1e-5)
    theta = torch.rand(Nv, D2 // 2, generator=g, dtype=torch.float64) * 6.283
    rope5 = ops.rope_table(torch.polar(torch.ones_like(theta), theta), Nv, dev, head_dim=D2)
    pk5, pq5 = ops.QkPre(rk5, wn, rope5), ops.QkPre(rq5, wn, rope5)
    se2 = h2 * (D2 + 1) * D2 * 4
    st112 = ops.linattn_state(qkv5[:, :, 1], qkv5[:, :, 2], head_dim=D2)
    add("linattn_state_d112", "hbm", 2 * Nv * C * 2 + se2,
        event_time_us(lambda: ops.linattn_state(qkv5[:, :, 1], qkv5[:, :, 2], head_dim=D2), iters, warmup),
        "N=32760, 20 heads of 112; K,V read + state")
    add("linattn_apply_d112", "hbm", 2 * Nv * C * 2 + se2,
        event_time_us(lambda: ops.linattn_apply(qkv5[:, :, 0], st112, 1e-8, out=out5), iters, warmup),
        "N=32760, 20 heads of 112; Q read + out write + state")
    rope_bytes5 = Nv * (D2 // 2) * 2 * 4 + Nv * 4
    add("linattn_state_d112_norm_rope_chunk_causal", "hbm", la5 - 21 * (C // 32) * 33 * 32 * 4 + 21 * se2 + rope_bytes5,
        event_time_us(lambda: ops.linattn_state(qkv5[:, :, 1], qkv5[:, :, 2], starts, causal=True, pre=pk5,
                                                head_dim=D2), iters, warmup),
        "cfg5 with 112-wide heads: K,V read + 21 states + rope table (448 B/token) + 1/rms")
    st112c = ops.linattn_state(qkv5[:, :, 1], qkv5[:, :, 2], starts, causal=True, pre=pk5, head_dim=D2)
    add("linattn_apply_d112_norm_rope_chunk_causal", "hbm", la5 - 21 * (C // 32) * 33 * 32 * 4 + 21 * se2 + rope_bytes5,
        event_time_us(lambda: ops.linattn_apply(qkv5[:, :, 0], st112c, 1e-8, starts, out=out5, pre=pq5), iters, warmup),
        "cfg5 with 112-wide heads: Q read + out write + 21 states + rope table + 1/rms")
    del qkv5, out5, st112, st112c, rope5


def _kernel_rooflines_ffn(dev, add, rows, g, iters, warmup, stock_conv, cfg3_only):
    from sana_amd import ops

    B, N, M = 1, 16384, 16384
    u = torch.randn(B, 128, 128, 2 * HID, generator=g).bfloat16().to(dev)
    dw = (torch.randn(2 * HID, 1, 3, 3, generator=g) * 0.3).bfloat16().to(dev)
    db = torch.zeros(2 * HID, dtype=torch.bfloat16, device=dev)
    add("dwconv3x3_silu_gate", "hbm", M * 2 * HID * 2 + M * HID * 2 + 2 * HID * 10 * 2,
        event_time_us(lambda: ops.dwconv3x3_silu_gate(u, dw, db, True), iters, warmup),
        "M*2H*2 B read + M*H*2 B write + weights")
    del u
    # cross-attention to 300 text tokens, 20 heads of 112 (the block's num_heads): two products of 2*M*300*C flops
    xq = torch.randn(B, N, C, generator=g).bfloat16().to(dev)
    xkv = torch.randn(B, 300, 2 * C, generator=g).bfloat16().to(dev)
    xo = torch.empty_like(xq)
    add("cross_attention_300_keys", "mfma", 4 * M * 300 * C,
        event_time_us(lambda: ops.cross_attention(xq, xkv, HEADS_X, out=xo), iters, warmup),
        "4*M*Nk*C flops (q k^T and p v), Nk=300, 20 heads of 112; also moves 2*M*C*2 B (147 MB)")
    del xq, xo
    x_ln = torch.randn(B, N, C, generator=g).bfloat16().to(dev)
    mod = (torch.randn(B, 6, C, generator=g) * 0.5).bfloat16().to(dev)
    add("layernorm_modulate", "hbm", 2 * M * C * 2,
        event_time_us(lambda: ops.layernorm_modulate(x_ln, mod[:, 1:2], mod[:, 0:1], 1e-6), iters, warmup),
        "M*C*2 B read + M*C*2 B write")
    for name, Nn, Kk, epi in (("gemm_qkv", 3 * C, C, None), ("gemm_proj_gate_residual", C, C, "gate_res"),
                              ("gemm_inverted", 2 * HID, C, "bias_silu"),
                              ("gemm_inverted_bias_only", 2 * HID, C, "bias"),   # what the library figure beside it computes
                              ("gemm_point_gate_residual", C, HID, "gate_res"),
                              ("gemm_inverted_w8a16", 2 * HID, C, "w8_bias_silu"),
                              ("gemm_inverted_w8a16_in_loop", 2 * HID, C, "w8_bias_silu_fused")):
        a = torch.randn(M, Kk, generator=g).bfloat16().to(dev)
        w = (torch.randn(Nn, Kk, generator=g) * 0.02).bfloat16().to(dev)
        bias = torch.zeros(Nn, dtype=torch.bfloat16, device=dev) if epi else None
        o = torch.empty(M, Nn, dtype=torch.bfloat16, device=dev)
        lib_extra = ""
        if epi == "gate_res":     # x + gate * (a @ w.T + bias): the two gated residual seams of the block
            fn = lambda: ops.gemm_gate_residual(a.view(B, N, Kk), w, bias, mod[:, 2:3], x_ln)
        elif epi in ("w8_bias_silu", "w8_bias_silu_fused"):
            # int8 weights: expanded to bf16 by a kernel of its own in front of the bf16 GEMM (what the library
            # picks at this M), or converted inside the GEMM's main loop (the path for small M)
            from sana_amd.modules import quantize_w8
            wq, sc = quantize_w8(w)
            fused = epi.endswith("_fused")
            fn = lambda: ops.gemm_w8a16(a, wq, sc, bias, "bias_silu", out=o, expand=not fused)
        else:
            fn = lambda: ops.gemm_bf16(a, w, bias, epi, out=o)
        t_us = event_time_us(fn, 20, 5)
        add(name, "mfma", 2 * M * Nn * Kk, t_us, f"2*M*K*N, M={M} N={Nn} K={Kk}")
        t_lib = event_time_us(lambda: torch.nn.functional.linear(a, w, bias), 20, 5)
        rows[-1]["library_gemm_us"] = round(t_lib, 2)   # hipBLASLt, plain GEMM(+bias) of the same shape, for scale only
        if name == "gemm_qkv":
            # the same projection with phase 1 of the attention in its epilogue (k, v never stored): one launch + the
            # sum of the 64 per-tile partial states, against this row + linattn_state above
            wt_, _ = ops.tile_qkv_weight(w, None, C // 32)
            t_f = event_time_us(lambda: ops.gemm_qkv_state(a.view(B, N, Kk), wt_, None, C // 32), 20, 5)
            add("gemm_qkv_with_attention_state", "mfma", 2 * M * Nn * Kk + 2 * M * C * 33, t_f,
                f"2*M*K*N + 2*M*C*33 (state), M={M} N={Nn} K={Kk}; replaces gemm_qkv + linattn_state")
            del wt_
        del a, w, o
    if cfg3_only:
        return
    # temporal (3, 1) conv of the video Mix-FFN (GLUMBConvTemp) + its residual at the cfg5 frame grid, as one GEMM over
    # the token-major frames; the stock convolution on the reference's (B, C, T, HW) view beside it
    Tf, Pf = 21, 30 * 52
    buf = torch.randn((Tf + 1) * Pf, C, generator=g).bfloat16().to(dev)
    buf[:Pf].zero_()
    wt = (torch.randn(C, 3 * C, generator=g) * 0.01).bfloat16().to(dev)
    ot = torch.empty(Tf * Pf, C, dtype=torch.bfloat16, device=dev)
    add("tconv_residual_cfg5", "mfma", 2 * Tf * Pf * 3 * C * C,
        event_time_us(lambda: ops.tconv_residual(buf, wt, Tf * Pf, Pf, out=ot), 10, 3),
        f"2*M*3C*C, M={Tf * Pf} (21 frames of 1560 tokens), C={C}")
    if stock_conv:
        # off by default: on a fresh machine the convolution library first times its candidate kernels for this
        # shape, a naive one among them that runs ~14 s per call -- about two minutes before the first result
        xr = buf[Pf:].view(1, Tf, Pf, C).permute(0, 3, 1, 2)
        w4 = wt.view(C, 3, C).permute(0, 2, 1).unsqueeze(-1).contiguous()
        rows[-1]["library_conv_us"] = round(event_time_us(
            lambda: xr + torch.nn.functional.conv2d(xr, w4, padding=(1, 0)), 3, 1), 2)
        del xr
    del buf, ot


def _kernel_rows_qk_norm_and_cfg2(dev, add, rows, g):
    """litela_qk_norm_cfg3: what LiteLA with qk_norm=True (every Sana-1.5 configuration) runs between its qkv GEMM
    and its proj GEMM -- the per-token 1/rms pass and the two attention phases with the norm applied on load --
    as one timed sequence.  Then the four GEMMs of cfg2 (Sana-600M width, B=4 x 1024 tokens = 4096 rows) with
    the library's plain GEMM of the same shape beside each."""
    from sana_amd import ops

    B, N, M = 1, 16384, 16384
    qkv = torch.randn(B, N, 3, C, generator=g).bfloat16().to(dev)
    q, k, v = qkv[:, :, 0], qkv[:, :, 1], qkv[:, :, 2]
    wn = (1 + 0.1 * torch.randn(C, generator=g)).bfloat16().to(dev)
    out = torch.empty(B, N, C, dtype=torch.bfloat16, device=dev)

    def qk_norm_attention():
        rq, rk = ops.qk_rms(q, k, 1e-5)
        st = ops.linattn_state(k, v, pre=ops.QkPre(rk, wn, None))
        ops.linattn_apply(q, st, 1e-8, out=out, pre=ops.QkPre(rq, wn, None))

    add("litela_qk_norm_cfg3", "hbm", 2 * M * C * 2 + 2 * (2 * M * C * 2) + 3 * 2 * M * 4 + 2 * (C // 32) * 33 * 32 * 4,
        event_time_us(qk_norm_attention, 30, 5),
        "qk_rms + linattn_state + linattn_apply with q/k RMSNorm on load (4 launches): q, k read twice, v read, out "
        "written; beyond the plain qkv GEMM (the fused qkv+state route needs the whole k row's 1/rms before it can "
        "contract a token, so it does not apply)")
    del qkv, out
    Cc, Hc, Mc = 1152, 2880, 4096
    x_res = torch.randn(4, 1024, Cc, generator=g).bfloat16().to(dev)
    mod = (torch.randn(4, 6, Cc, generator=g) * 0.5).bfloat16().to(dev)
    for name, Nn, Kk, epi in (("cfg2_gemm_qkv", 3 * Cc, Cc, None), ("cfg2_gemm_proj_gate_residual", Cc, Cc, "gate_res"),
                              ("cfg2_gemm_inverted", 2 * Hc, Cc, "bias_silu"),
                              ("cfg2_gemm_point_gate_residual", Cc, Hc, "gate_res")):
        a = torch.randn(Mc, Kk, generator=g).bfloat16().to(dev)
        w = (torch.randn(Nn, Kk, generator=g) * 0.02).bfloat16().to(dev)
        bias = torch.zeros(Nn, dtype=torch.bfloat16, device=dev) if epi else None
        o = torch.empty(Mc, Nn, dtype=torch.bfloat16, device=dev)
        if epi == "gate_res":
            fn = lambda: ops.gemm_gate_residual(a.view(4, 1024, Kk), w, bias, mod[:, 2:3], x_res)
        else:
            fn = lambda: ops.gemm_bf16(a, w, bias, epi, out=o)
        add(name, "mfma", 2 * Mc * Nn * Kk, event_time_us(fn, 50, 10), f"2*M*K*N, M={Mc} N={Nn} K={Kk} (cfg2: B=4 x 1024 tokens)")
        rows[-1]["library_gemm_us"] = round(event_time_us(lambda: torch.nn.functional.linear(a, w, bias), 50, 10), 2)
        if name == "cfg2_gemm_qkv":
            wt_, _ = ops.tile_qkv_weight(w, None, Cc // 32)
            add("cfg2_gemm_qkv_with_attention_state", "mfma", 2 * Mc * Nn * Kk + 2 * Mc * Cc * 33,
                event_time_us(lambda: ops.gemm_qkv_state(a.view(4, 1024, Kk), wt_, None, Cc // 32), 50, 10),
                f"2*M*K*N + state, M={Mc} N={Nn} K={Kk}: the route the cfg2 block takes (replaces cfg2_gemm_qkv + phase 1)")
            del wt_
        del a, w, o


_STATES = {}


def make_blocks(dev, w8: bool = False):
    """The DEPTH blocks of Sana-1.6B (random init, one seed per block), bf16 or W8A16."""
    import sana_amd as S

    blocks = []
    for i in range(DEPTH):
        blk = S.SanaMSBlock(C, HEADS_X, mlp_ratio=MLP_RATIO, attn_type="linear", ffn_type="glumbconv").bfloat16()
        if i not in _STATES:
            _STATES[i] = make_state(i)
        blk.load_state_dict(_STATES[i])
        blk = blk.to(dev)
        blocks.append(blk.quantize_w8_() if w8 else blk)
    return blocks


def chain_step(blocks, cond, x, y, t, HW):
    """One denoising step's block loop (sana_multi_scale.py:368-383); ``cond``: the blocks' StepConditioning,
    evaluated inside the step (text keys / values and modulation rows of all blocks in two launches)."""
    h = x
    for blk, c in zip(blocks, cond(y, t)):
        h = blk(h, y, t, None, HW, None, **c)
    return h


def images_per_s(dev, blocks, steps: int, warmup: int, B: int = 16, graphed: bool = False) -> float:
    """1024px shape of Sana-1.6B: B images of N=1024 tokens; the DEPTH DiT blocks of one denoising step only.
    ``graphed``: the step's launches replayed from one captured HIP graph (sana_amd.GraphedCall) instead of being
    issued from Python."""
    import sana_amd as S

    HW = (32, 32)
    cond = S.StepConditioning(blocks)
    x, y, t = (a.bfloat16().to(dev) for a in make_inputs(B, HW[0] * HW[1]))
    with torch.no_grad():
        if graphed:
            step = S.GraphedCall(lambda a, b, c: chain_step(blocks, cond, a, b, c, HW), (x, y, t))
            t_us = event_time_us(lambda: step(x, y, t), steps, warmup)
        else:
            t_us = event_time_us(lambda: chain_step(blocks, cond, x, y, t, HW), steps, warmup)
    return B / (t_us * 1e-6)


def video_block_ms(dev, steps: int = 10, warmup: int = 3) -> float:
    """One SanaVideoMSBlock forward at the video shape (21 x 30 x 52 tokens, C = 2240, 20 heads of 112, q/k norm,
    rotary embedding, chunk_index [0, 11], temporal Mix-FFN): the reference's released video configuration."""
    import sana_amd as S

    T, H, W, d = 21, 30, 52, 112
    N = T * H * W
    g = torch.Generator().manual_seed(5)
    blk = S.SanaVideoMSBlock(C, HEADS_X, mlp_ratio=MLP_RATIO, attn_type="chunkcausal", ffn_type="ChunkGLUMBConvTemp",
                             qk_norm=True, linear_head_dim=d).bfloat16()
    with torch.no_grad():
        for n, p in blk.named_parameters():
            if n != "scale_shift_table" and p.dim() > 1:
                p.copy_(torch.nn.init.trunc_normal_(torch.empty(p.shape), std=0.02, generator=g))
    blk = blk.to(dev)
    x, y, t = (a.bfloat16().to(dev) for a in make_inputs(1, N))
    theta = torch.rand(N, d // 2, generator=g, dtype=torch.float64) * 6.283
    freqs = torch.polar(torch.ones_like(theta), theta)[None, None].to(dev)
    with torch.no_grad():
        t_us = event_time_us(lambda: blk(x, y, t, THW=(T, H, W), rotary_emb=freqs, chunk_index=[0, 11]), steps, warmup)
    return t_us / 1e3


def cpu_baseline(iters: int = 5):
    """The oracle (stock PyTorch restatement of the reference block) on the host
    cores: one block of the cfg3 workload in fp32 (bf16 GEMM/conv on CPU is not a
    fair or stable baseline), same seeded weights and inputs."""
    from oracle import sana_oracle as O

    threads = torch.get_num_threads()
    blk = O.SanaMSBlock(C, HEADS_X, mlp_ratio=MLP_RATIO, attn_type="linear", ffn_type="glumbconv")
    blk.load_state_dict(make_state(0, torch.float32))
    blk.attn.fp32_attention = True
    x, y, t = make_inputs(1, 16384)
    with torch.no_grad():
        blk(x, y, t, HW=(128, 128))
        t0 = time.perf_counter()
        for _ in range(iters):
            blk(x, y, t, HW=(128, 128))
        dt = (time.perf_counter() - t0) / iters
    model = ""
    try:
        for line in open("/proc/cpuinfo"):
            if line.startswith("model name"):
                model = line.split(":", 1)[1].strip()
                break
    except OSError:
        pass
    return {"value": round(dt * 1e3, 2), "unit": "ms per block forward", "cores": threads, "kind": "port",
            "sample": f"1 of the 20 blocks at the same shape (B=1, N=16384, C=2240), fp32, {iters} timed "
                      f"iterations after 1 warm-up; os.cpu_count()={os.cpu_count()}, cpu='{model}'"}


def small_configs(dev):
    """The two small configurations of the benchmark definition, GPU and host side by side.
    cfg1: the LiteLA attention op alone (state + apply), fp32, B=1, 36 heads x 32, N=1024, q, k, v ~ N(0, 1), eps 1e-15;
    host: the oracle's two-matmul form of the same op (LiteLA.attn_matmul), fp32.
    cfg2: one SanaMSBlock at Sana-600M width, bf16, B=4, N=32x32, C=1152, hidden 2880, 300 text tokens;
    host: the oracle block in fp32 (bf16 GEMM / conv on the host is neither fair nor stable)."""
    import sana_amd as S
    from oracle import sana_oracle as O
    from sana_amd import ops

    threads = torch.get_num_threads()
    res = {}
    # ---- cfg1
    B, h, d, N = 1, 36, 32, 1024
    g = torch.Generator().manual_seed(0)
    qkv = torch.randn(B, N, 3, h * d, generator=g)
    qd = qkv.to(dev)
    out = torch.empty(B, N, h * d, device=dev)

    def gpu_op():
        st = ops.linattn_state(qd[:, :, 1], qd[:, :, 2])
        ops.linattn_apply(qd[:, :, 0], st, 1e-15, out=out)

    t_gpu = event_time_us(gpu_op, 200, 20)
    q4, k4, v4 = (qkv[:, :, i].reshape(B, N, h, d).permute(0, 2, 3, 1) for i in range(3))   # (B, h, d, N) views
    with torch.no_grad():
        O.relu_linear_attention(q4, k4.transpose(-1, -2), v4, 1e-15)
        t0 = time.perf_counter()
        for _ in range(50):
            O.relu_linear_attention(q4, k4.transpose(-1, -2), v4, 1e-15)
        t_cpu = (time.perf_counter() - t0) / 50 * 1e6
    bytes1 = 4 * N * h * d * 4 + 2 * h * (d + 1) * d * 4
    res["cfg1"] = {"workload": "LiteLA ReLU linear attention op alone, fp32, B=1, 36 heads x 32, N=1024, eps 1e-15",
                   "gpu_us": round(t_gpu, 2), "gpu_launches": 3, "algorithmic_bytes": bytes1,
                   "achieved_GBps": round(bytes1 / t_gpu / 1e3, 1),
                   "cpu_baseline": {"value": round(t_cpu, 1), "unit": "us per op", "cores": threads, "kind": "port",
                                    "sample": "the whole workload, 50 timed iterations after 1 warm-up"},
                   "note": "three launches of a few microseconds each: bound by launch latency, not by HBM"}
    # ---- cfg2
    Cc, heads, Bb, HW = 1152, 16, 4, (32, 32)
    ob = O.init_block_(O.SanaMSBlock(Cc, heads, mlp_ratio=2.5, attn_type="linear", ffn_type="glumbconv"), 0)
    ob.attn.fp32_attention = True
    hb = S.SanaMSBlock(Cc, heads, mlp_ratio=2.5, attn_type="linear", ffn_type="glumbconv").bfloat16()
    hb.load_state_dict({k_: v_.bfloat16() for k_, v_ in ob.state_dict().items()})
    hb = hb.to(dev)
    x, y, t = O.block_inputs(Bb, HW[0] * HW[1], Cc, seed=2)
    xd, yd, td = (a.bfloat16().to(dev) for a in (x, y, t))
    with torch.no_grad():
        t_gpu = event_time_us(lambda: hb(xd, yd, td, HW=HW), 50, 10)
        graphed = S.GraphedCall(lambda a, b, c: hb(a, b, c, HW=HW), (xd, yd, td))
        t_graph = event_time_us(lambda: graphed(xd, yd, td), 50, 10)
        ob(x, y, t, HW=HW)
        t0 = time.perf_counter()
        for _ in range(5):
            ob(x, y, t, HW=HW)
        t_cpu = (time.perf_counter() - t0) / 5 * 1e3
    res["cfg2"] = {"workload": "one SanaMSBlock at Sana-600M width, bf16, B=4, N=32x32=1024, C=1152, hidden 2880, "
                               "300 text tokens, random init",
                   "gpu_block_ms": round(t_gpu / 1e3, 4), "gpu_block_ms_hip_graph": round(t_graph / 1e3, 4),
                   "note": "eager issue of the block's ~25 launches from Python is host-bound at this size; "
                           "gpu_block_ms_hip_graph replays the same launches from one captured HIP graph (sana_amd.GraphedCall)",
                   "cpu_baseline": {"value": round(t_cpu, 2), "unit": "ms per block forward", "cores": threads,
                                    "kind": "port", "sample": "the whole workload in fp32, 5 timed iterations after 1 warm-up"}}
    return res


def _cpu_model() -> str:
    try:
        for line in open("/proc/cpuinfo"):
            if line.startswith("model name"):
                return line.split(":", 1)[1].strip()
    except OSError:
        pass
    return ""


def config4(dev, ips_w8: float, ips_bf16: float):
    """cfg4: W8A16 Sana-1.6B at 1024px, B=16 x 1024 tokens; GPU figures from the images/s legs, host: ONE oracle
    block on the dequantised weights in fp32 at the same shape."""
    from oracle import sana_oracle as O

    B, HW = 16, (32, 32)
    blk = O.SanaMSBlock(C, HEADS_X, mlp_ratio=MLP_RATIO, attn_type="linear", ffn_type="glumbconv")
    blk.load_state_dict({k: v.float() for k, v in O.dequantized_block_state(make_state(0)).items()})
    blk.attn.fp32_attention = True
    x, y, t = make_inputs(B, HW[0] * HW[1])
    with torch.no_grad():
        blk(x, y, t, HW=HW)
        t0 = time.perf_counter()
        for _ in range(3):
            blk(x, y, t, HW=HW)
        t_cpu = (time.perf_counter() - t0) / 3 * 1e3
    return {"workload": "W8A16 (int8 per-output-channel qkv / proj / 1x1-conv weights, bf16 activations) Sana-1.6B block, "
                        "B=16 images of N=32x32=1024 tokens, C=2240, 300 text tokens, random init",
            "gpu_block_ms": round(B / ips_w8 / DEPTH * 1e3, 4), "gpu_block_ms_bf16_weights": round(B / ips_bf16 / DEPTH * 1e3, 4),
            "images_per_s": round(ips_w8, 2),
            "note": "gpu_block_ms = step time of the 20 chained W8A16 blocks / 20 (the images_per_s_1024px leg)",
            "cpu_baseline": {"value": round(t_cpu, 2), "unit": "ms per block forward", "cores": torch.get_num_threads(),
                             "kind": "port", "sample": "1 of the 20 blocks at the same shape (B=16, N=1024) on the dequantised "
                                                       f"weights, fp32, 3 timed iterations after 1 warm-up; cpu='{_cpu_model()}'"}}


def config5(dev):
    """cfg5: ChunkCausalAttention at C=2240 with 70 heads of 32 on 21 x 30 x 52 tokens, then the GLUMBConv Mix-FFN with
    the depthwise 3x3 per frame -- the two modules as the configuration words them, GPU and host (oracle, fp32)."""
    import sana_amd as S
    from oracle import sana_oracle as O

    T, H, W = 21, 30, 52
    N = T * H * W
    g = torch.Generator().manual_seed(9)

    def tn(p):
        return torch.nn.init.trunc_normal_(torch.empty(p.shape), std=0.02, generator=g)

    oa = O.ChunkCausalAttention(C, C, heads=C // 32, eps=1e-8)
    om = O.GLUMBConv(C, HID, use_bias=(True, True, False), norm=(None, None, None), act=("silu", "silu", None))
    with torch.no_grad():
        for m in (oa, om):
            for n_, p_ in m.named_parameters():
                p_.copy_(tn(p_) if p_.dim() > 1 else torch.zeros_like(p_))
    oa.fp32_attention = True
    ha = S.ChunkCausalAttention(C, C, heads=C // 32, eps=1e-8).bfloat16()
    hm = S.GLUMBConv(C, HID, use_bias=(True, True, False), norm=(None, None, None), act=("silu", "silu", None)).bfloat16()
    ha.load_state_dict({k: v.bfloat16() for k, v in oa.state_dict().items()})
    hm.load_state_dict({k: v.bfloat16() for k, v in om.state_dict().items()})
    ha, hm = ha.to(dev), hm.to(dev)
    x = torch.randn(1, N, C, generator=g)
    xd = x.bfloat16().to(dev)
    every_frame = list(range(T))
    res = {"workload": "chunk-causal linear attention module (qkv + attention + proj), bf16 io / fp32 state, C=2240, 70 heads x 32, "
                       "21 frames x 30x52 tokens (N=32760), B=1, followed by the GLUMBConv Mix-FFN (hidden 5600) with the "
                       "depthwise 3x3 per frame"}
    with torch.no_grad():
        res["gpu_attention_ms_21_chunks"] = round(event_time_us(
            lambda: ha(xd, HW=(T, H, W), chunk_index=every_frame), 10, 3) / 1e3, 4)
        res["gpu_attention_ms_chunks_0_11"] = round(event_time_us(
            lambda: ha(xd, HW=(T, H, W), chunk_index=[0, 11]), 10, 3) / 1e3, 4)
        res["gpu_mix_ffn_ms"] = round(event_time_us(lambda: hm(xd, HW=(T, H, W)), 10, 3) / 1e3, 4)
        oa(x, HW=(T, H, W), chunk_index=[0, 11])
        t0 = time.perf_counter()
        for _ in range(2):
            oa(x, HW=(T, H, W), chunk_index=[0, 11])
        t_att = (time.perf_counter() - t0) / 2 * 1e3
        om(x, HW=(T, H, W))
        t0 = time.perf_counter()
        for _ in range(2):
            om(x, HW=(T, H, W))
        t_ffn = (time.perf_counter() - t0) / 2 * 1e3
    res["cpu_baseline"] = {"value": round(t_att + t_ffn, 1), "attention_ms": round(t_att, 1), "mix_ffn_ms": round(t_ffn, 1),
                           "unit": "ms per pass of the two modules", "cores": torch.get_num_threads(), "kind": "port",
                           "sample": "the whole workload (chunk_index [0, 11]) in fp32, 2 timed iterations after 1 warm-up; "
                                     f"cpu='{_cpu_model()}'"}
    return res


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=10)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-kernels", action="store_true", help="skip the per-kernel roofline section")
    ap.add_argument("--kernels-only", action="store_true", help="only the per-kernel section (profiling runs)")
    ap.add_argument("--cfg3-only", action="store_true",
                    help="with --kernels-only: skip the video-shape and 112-wide-head launches (counter runs: every "
                         "kernel instance then runs at the cfg3 shape only)")
    ap.add_argument("--step-only", action="store_true",
                    help="only the timed cfg3 chain, printed as a short JSON line (profiling runs: every kernel row of a "
                         "trace is then the cfg3 shape inside the chained step)")
    ap.add_argument("--stock-conv", action="store_true",
                    help="also time the stock convolution beside the temporal-conv GEMM (minutes of library tuning on a fresh machine)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU: this build has no multi-GPU path (run with --gpus 1)", file=sys.stderr)
        sys.exit(2)
    if not torch.cuda.is_available():
        print("bench.py needs an MI355X (no GPU visible)", file=sys.stderr)
        sys.exit(2)
    import sana_amd as S

    dev = torch.device("cuda:0")
    if args.kernels_only:
        with torch.no_grad():
            kernels, copy_gbs = kernel_rooflines(dev, stock_conv=args.stock_conv, cfg3_only=args.cfg3_only)
        print(json.dumps({"kernels": kernels, "copy_GBps_this_box": copy_gbs}))
        return
    B, HW = 1, (128, 128)
    N = HW[0] * HW[1]
    blocks = make_blocks(dev)
    cond = S.StepConditioning(blocks)
    x, y, t = (a.bfloat16().to(dev) for a in make_inputs(B, N))

    def step():
        return chain_step(blocks, cond, x, y, t, HW)

    with torch.no_grad():
        for _ in range(args.warmup):
            step()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(args.steps):
            out = step()
        torch.cuda.synchronize()
        wall = time.perf_counter() - t0
        assert torch.isfinite(out.float()).all()
        ms_per_step = wall * 1e3 / args.steps
        block_ms = ms_per_step / DEPTH
        if args.step_only:
            print(json.dumps({"metric": "cfg3 chained step only", "value": round(block_ms, 4), "unit": "ms per block",
                              "ms_per_step": round(ms_per_step, 3), "steps": args.steps, "warmup": args.warmup}))
            return

        kernels, copy_gbs = ([], None) if args.no_kernels else kernel_rooflines(dev, stock_conv=args.stock_conv)
        ips_bf16 = images_per_s(dev, blocks, 5, 2)
        one_image_ms = 1e3 / images_per_s(dev, blocks, 20, 5, B=1)   # 20 blocks on one image: latency, not throughput
        one_image_ms_graph = 1e3 / images_per_s(dev, blocks, 20, 5, B=1, graphed=True)
        del cond, blocks
        blocks = make_blocks(dev, w8=True)
        ips_w8 = images_per_s(dev, blocks, 5, 2)
        one_image_ms_w8 = 1e3 / images_per_s(dev, blocks, 20, 5, B=1)
        video_ms = video_block_ms(dev)
    del blocks
    torch.cuda.empty_cache()

    dom = next((r for r in kernels if r["kernel"] == "gemm_inverted"), None)
    roofline = None
    if dom:
        roofline = {"kernel": "gemm4_kernel<bf16, bias+silu> (inverted 1x1 conv, M=16384 N=11200 K=2240)",
                    "bound": "mfma", "achieved": dom["achieved"], "peak": dom["peak"], "unit": "TFLOP/s",
                    "frac": dom["frac"], "traffic": dominant_kernel_traffic_bytes()}
    line = {
        "metric": "Sana-1.6B SanaMSBlock forward latency @16384 tokens (4096px latent)",
        "value": round(block_ms, 4), "unit": "ms", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 3), "higher_is_better": False, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16", "data": "synthetic",
        "config": {"workload": "cfg3: Sana-1.6B, 20 SanaMSBlocks chained = one denoising step, B=1, N=128x128=16384, "
                               "C=2240, 70x32 heads, Mix-FFN hidden 5600, 300 text tokens, random init"},
        "images_per_s_1024px": {"bf16": round(ips_bf16, 2), "w8a16": round(ips_w8, 2),
                                "one_image_step_ms_bf16": round(one_image_ms, 3),
                                "one_image_step_ms_bf16_hip_graph": round(one_image_ms_graph, 3),
                                "one_image_step_ms_w8a16": round(one_image_ms_w8, 3),
                                "note": "B=16, N=1024: B / time of the 20 chained blocks; DiT blocks of one denoising step only "
                                        "(no text encoder, VAE, embedders, step count or CFG doubling); "
                                        "one_image_step_ms: the same 20 blocks at B=1 (hip_graph: replayed from one captured HIP graph)"},
        "video_block_ms": {"value": round(video_ms, 3),
                           "note": "one SanaVideoMSBlock forward, bf16: N=21x30x52=32760 tokens, C=2240, 20 heads of 112, "
                                   "q/k RMSNorm + rotary embedding, chunk_index [0, 11], ChunkGLUMBConvTemp, 300 text tokens"},
        "roofline": roofline,
        "kernels": kernels,
        "copy_GBps_this_box": copy_gbs,
        "peaks": {"hbm_GBps": HBM_PEAK_GBS, "mfma_bf16_TFLOPs": MFMA_BF16_PEAK_TFLOPS},
        "cpu_baseline": None if args.no_cpu_baseline else cpu_baseline(),
        "configs": None if args.no_cpu_baseline else small_configs(dev),
    }
    if line["configs"] is not None:
        line["configs"]["cfg4"] = config4(dev, ips_w8, ips_bf16)
        line["configs"]["cfg5"] = config5(dev)
    print(json.dumps(line))


if __name__ == "__main__":
    main()
