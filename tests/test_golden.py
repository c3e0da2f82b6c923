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
