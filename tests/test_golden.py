"""Known-answer vectors (``tests/golden/kat.npz``, frozen fp64 answers of the plain-C quadratic-form /
9-tap restatement on seeded bf16-representable inputs): the stock-PyTorch oracle must reproduce them on
the CPU, the HIP kernels on the GPU.  ``tests/golden/make_vectors.py`` regenerates the file."""
import os

import numpy as np
import pytest
import torch
import torch.nn.functional as F

from oracle import sana_oracle as O

KAT = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "kat.npz"))


def T(name):
    return torch.from_numpy(KAT[name])


def rel_l2(a, b):
    return ((a.double() - b.double()).norm() / b.double().norm()).item()


# ----------------------------------------------------------------------------- CPU: oracle vs fixture

@pytest.mark.parametrize("tag", ["la32", "la112"])
def test_oracle_linear_attention_reproduces_fixture(tag):
    q, k, v = T(f"{tag}_q"), T(f"{tag}_k"), T(f"{tag}_v")            # [BH, N, d] fp64
    out, state = O.relu_linear_attention(q.transpose(1, 2)[None], k[None], v.transpose(1, 2)[None], 1e-8,
                                         return_state=True)           # q, v (B, h, d, N); k (B, h, N, d)
    assert rel_l2(out[0].transpose(1, 2), T(f"{tag}_out")) < 1e-12
    assert rel_l2(state[0], T(f"{tag}_state")) < 1e-12


def test_oracle_chunk_causal_reproduces_fixture():
    q, k, v, chunk_of = T("cc_q"), T("cc_k"), T("cc_v"), KAT["cc_chunk_of"]
    eps = 1e-8
    # the attention core the way ChunkCausalAttention.forward drives it: per chunk, on the running state
    outs, run = [], 0
    for c in range(int(chunk_of.max()) + 1):
        idx = np.nonzero(chunk_of == c)[0]
        a, b = int(idx[0]), int(idx[-1]) + 1
        _, st = O.relu_linear_attention(q[:, a:b].transpose(1, 2)[None], k[:, a:b][None],
                                        v[:, a:b].transpose(1, 2)[None], eps, return_state=True)
        run = run + st
        o = run @ torch.relu(q[:, a:b].transpose(1, 2)[None])
        outs.append(o[:, :, :-1] / (o[:, :, -1:] + eps))
    out = torch.cat(outs, -1)[0].transpose(1, 2)
    assert rel_l2(out, T("cc_out")) < 1e-12


def test_oracle_depthwise_gate_reproduces_fixture():
    u, w, b = T("dw_u"), T("dw_w"), T("dw_b")                          # [BT,H,W,2C], [2C,3,3], [2C]
    C2 = u.shape[-1]
    m = O.GLUMBConv(4, C2 // 2, use_bias=(True, True, False)).double()
    with torch.no_grad():
        m.depth_conv.conv.weight.copy_(w[:, None])
        m.depth_conv.conv.bias.copy_(b)
        x = m.depth_conv(u.permute(0, 3, 1, 2))
        a, g = torch.chunk(x, 2, dim=1)
        out = (a * m.glu_act(g)).permute(0, 2, 3, 1)
    assert rel_l2(out, T("dw_out")) < 1e-12


def _module_fed_with(cls, q, k, v):
    """An oracle attention module whose qkv projection reproduces the fixture's q, k, v exactly (N <= C, so a
    weight with x @ W^T = [q | k | v] exists) and whose output projection is the identity."""
    BH, N, d = q.shape
    C = BH * d
    tok = lambda t: t.transpose(0, 1).reshape(N, C)
    target = torch.cat([tok(q), tok(k), tok(v)], dim=1)                 # [N, 3C]
    x = torch.randn(N, C, generator=torch.Generator().manual_seed(1), dtype=torch.float64)
    W = torch.linalg.lstsq(x, target).solution.T                        # [3C, C]
    assert (x @ W.T - target).abs().max().item() < 1e-10
    m = cls(C, C, dim=d, eps=1e-8).double()
    with torch.no_grad():
        m.qkv.weight.copy_(W)
        m.proj.weight.copy_(torch.eye(C, dtype=torch.float64))
        m.proj.bias.zero_()
    return m, x[None], tok


@pytest.mark.parametrize("tag", ["rope32", "rope112"])
def test_oracle_rotary_family_reproduces_fixture(tag):
    """LiteLAReLURope, ChunkCausalAttention and the streamed CachedCausalAttention against the frozen brute-force
    answers (numerator rotated, denominator not: sana_blocks.py:378-381, 481-489, 544-562)."""
    q, k, v = T(f"{tag}_q"), T(f"{tag}_k"), T(f"{tag}_v")
    N = q.shape[1]
    rot = torch.complex(T(f"{tag}_cos"), T(f"{tag}_sin"))[None, None]
    m, x, tok = _module_fed_with(O.LiteLAReLURope, q, k, v)
    assert rel_l2(m(x, rotary_emb=rot)[0], tok(T(f"{tag}_out"))) < 1e-9
    cc, x, tok = _module_fed_with(O.ChunkCausalAttention, q, k, v)
    ref_cc = tok(T(f"{tag}_cc_out"))
    assert rel_l2(cc(x, HW=(3, 3, 4), rotary_emb=rot, chunk_index=[0, 1, 2])[0], ref_cc) < 1e-9
    cm, x, tok = _module_fed_with(O.CachedCausalAttention, q, k, v)
    acc, outs = [None, None], []
    for c in range(3):
        sl = slice(12 * c, 12 * c + 12)
        o, cache = cm(x[:, sl], rotary_emb=rot[:, :, sl], save_kv_cache=True, kv_cache=[acc[0], acc[1]])
        acc = [cache[i] if acc[i] is None else acc[i] + cache[i] for i in range(2)]
        outs.append(o)
    assert rel_l2(torch.cat(outs, 1)[0], ref_cc) < 1e-9


# ----------------------------------------------------------------------------- GPU: kernels vs fixture

@pytest.mark.gpu
@pytest.mark.parametrize("tag,d", [("la32", 32), ("la112", 112)])
def test_kernels_linear_attention_reproduce_fixture(cuda, tag, d):
    from sana_amd import ops
    q, k, v = (T(f"{tag}_{n}") for n in "qkv")
    BH, N, _ = q.shape
    tm = lambda t: t.transpose(0, 1).reshape(1, N, BH * d).bfloat16().to(cuda)   # token-major [1, N, h*d]
    state = ops.linattn_state(tm(k), tm(v), head_dim=d)
    assert rel_l2(state[0, :, 0].cpu(), T(f"{tag}_state")) <= 1e-5
    out = ops.linattn_apply(tm(q), state, 1e-8, out_dtype=torch.float32)
    ref = T(f"{tag}_out").transpose(0, 1).reshape(1, N, BH * d)
    assert rel_l2(out.cpu(), ref) <= 1e-5
    out16 = ops.linattn_apply(tm(q), state, 1e-8)
    assert (out16.cpu().double() - ref).abs().max().item() <= 2e-2 and rel_l2(out16.cpu(), ref) <= 1e-2


@pytest.mark.gpu
def test_kernels_chunk_causal_reproduce_fixture(cuda):
    from sana_amd import ops
    q, k, v, chunk_of = T("cc_q"), T("cc_k"), T("cc_v"), KAT["cc_chunk_of"]
    BH, N, d = q.shape
    tm = lambda t: t.transpose(0, 1).reshape(1, N, BH * d).bfloat16().to(cuda)
    starts = [int(np.nonzero(chunk_of == c)[0][0]) for c in range(int(chunk_of.max()) + 1)]
    out = ops.relu_linear_attention(tm(q), tm(k), tm(v), 1e-8, chunk_tokens=starts, out_dtype=torch.float32)
    assert rel_l2(out.cpu(), T("cc_out").transpose(0, 1).reshape(1, N, BH * d)) <= 1e-5


@pytest.mark.gpu
def test_kernel_depthwise_gate_reproduces_fixture(cuda):
    from sana_amd import ops
    u, w, b = T("dw_u"), T("dw_w"), T("dw_b")
    ref = T("dw_out")
    y32 = ops.dwconv3x3_silu_gate(u.float().to(cuda), w.float().contiguous().to(cuda), b.float().to(cuda), False)
    assert rel_l2(y32.cpu(), ref) <= 1e-5
    y16 = ops.dwconv3x3_silu_gate(u.bfloat16().to(cuda), w.bfloat16().contiguous().to(cuda), b.bfloat16().to(cuda), True)
    assert (y16.cpu().double() - ref).abs().max().item() <= 2e-2 and rel_l2(y16.cpu(), ref) <= 1e-2


@pytest.mark.gpu
@pytest.mark.parametrize("tag,d", [("rope32", 32), ("rope112", 112)])
def test_kernels_rotary_family_reproduce_fixture(cuda, tag, d):
    """sana_hip_linattn_state_pre / sana_hip_linattn_apply_pre with a rope table, whole sequence and three causal
    chunks.  The kernels round the rotated operands to bf16 before the fp32-accumulating MFMA (the reference's
    `.type_as(hidden_states)` after its fp64 rotation), the fixture does not: bf16 tolerance on the output."""
    from sana_amd import ops
    q, k, v = (T(f"{tag}_{n}") for n in "qkv")
    BH, N, _ = q.shape
    tm = lambda t: t.transpose(0, 1).reshape(1, N, BH * d).bfloat16().to(cuda)
    table = torch.stack([T(f"{tag}_cos"), T(f"{tag}_sin")], dim=-1).float().contiguous().to(cuda)   # [N, d/2, 2]
    pre = ops.QkPre(rope=table)
    for key, chunks in ((f"{tag}_out", None), (f"{tag}_cc_out", [0, 12, 24])):
        ref = T(key).transpose(0, 1).reshape(1, N, BH * d)
        state = ops.linattn_state(tm(k), tm(v), chunks, causal=chunks is not None, pre=pre, head_dim=d)
        for out_dtype in (torch.float32, torch.bfloat16):
            out = ops.linattn_apply(tm(q), state, 1e-8, chunks, out_dtype=out_dtype, pre=pre).cpu()
            mx, rl = (out.double() - ref).abs().max().item(), rel_l2(out, ref)
            assert mx <= 2e-2 and rl <= 1e-2, f"{key} {out_dtype}: max-abs {mx:.3e} rel-L2 {rl:.3e}"
        # the unrotated k-sum row of the state is exact in fp32: sum of relu(k) over the tokens seen so far
        ksum = torch.relu(k).transpose(0, 1).reshape(N, BH, d)
        want = ksum.sum(0) if chunks is None else ksum[:12].sum(0)
        assert rel_l2(state[0, :, 0, d].cpu(), want) <= 1e-6


# ----------------------------------------------------------------------------- qkv projection + state, exact integers

def test_oracle_qkv_projection_and_state_reproduce_fixture():
    """The oracle's LiteLA pieces on the integer fixture: linear -> q, and v . relu(k)^T with the row of ones."""
    x, w = T("qkvs_x"), T("qkvs_w")
    qkv = F.linear(x, w)                                               # [1, N, 3C]
    assert torch.equal(qkv[..., :64], T("qkvs_q"))
    k, v = (qkv[0, :, 64 * i:64 * (i + 1)].reshape(-1, 2, 32).permute(1, 0, 2) for i in (1, 2))   # [h, N, d]
    _, state = O.relu_linear_attention(k.transpose(1, 2)[None], k[None], v.transpose(1, 2)[None], 1e-8, return_state=True)
    assert torch.equal(state[0], T("qkvs_state"))


@pytest.mark.gpu
def test_kernel_qkv_projection_with_state_reproduces_fixture_exactly(cuda):
    """sana_hip_gemm_qkv_state on the integer fixture (two token tiles, two heads, one k / v column tile with two
    dummy heads): q and the state bit for bit -- nothing on the way rounds -- and the unfused pair of launches too."""
    from sana_amd import ops
    x, w = T("qkvs_x").bfloat16().to(cuda), T("qkvs_w").bfloat16().to(cuda)
    wt, _ = ops.tile_qkv_weight(w, None, 2)
    q, state = ops.gemm_qkv_state(x, wt, None, 2)
    assert torch.equal(q.double().cpu(), T("qkvs_q"))
    assert torch.equal(state[0, :, 0].double().cpu(), T("qkvs_state"))
    qkv = ops.gemm_bf16(x.view(-1, 64), w).view(1, -1, 3, 64)
    assert torch.equal(ops.linattn_state(qkv[:, :, 1], qkv[:, :, 2])[0, :, 0].double().cpu(), T("qkvs_state"))
