"""GPU parity of the head_dim-112 linear-attention kernels (the `linear_head_dim: 112` video configurations,
bf16 io) through the C ABI against the oracle, same tolerances as the head_dim-32 kernels."""
import pytest
import torch

from oracle import sana_oracle as O
from sana_amd import ops

pytestmark = pytest.mark.gpu
D = 112


def _qkv(B, N, C, seed, dtype=torch.bfloat16):
    g = torch.Generator().manual_seed(seed)
    return torch.randn(B, N, 3, C, generator=g).to(dtype)


def _heads(x, B, N, h):
    return x.double().view(B, N, h, D).permute(0, 2, 3, 1)      # (B, h, d, N)


def _oracle(qkv, eps):
    B, N, _, C = qkv.shape
    h = C // D
    q, k, v = (_heads(qkv[:, :, i], B, N, h) for i in range(3))
    out, state = O.relu_linear_attention(q, k.transpose(-1, -2), v, eps, return_state=True)
    return out.permute(0, 3, 1, 2).reshape(B, N, C), state


def rel_l2(a, b):
    return ((a.double() - b.double()).norm() / b.double().norm()).item()


CASES = [
    # B, N, C
    (1, 4096, 2240),      # 20 heads of 112: the 2B video width
    (2, 777, 336),        # ragged token count
    (1, 50, 112),         # single head, partial tiles only
    (1, 1, 224),          # one token
    (3, 129, 112),
    (1, 21 * 1560, 224),  # cfg5 token count (long splits)
    (13, 300, 2240),      # 260 (batch, head) pairs: more than compute units, one token range each
    (2, 2100, 1120),      # ranges of 192 tokens that end inside tiles
]


@pytest.mark.parametrize("B,N,C", CASES)
def test_state_and_output_match_oracle(cuda, B, N, C):
    eps = 1e-8
    qkv = _qkv(B, N, C, seed=N + C)
    ref_out, ref_state = _oracle(qkv, eps)
    d = qkv.to(cuda)
    q, k, v = d[:, :, 0], d[:, :, 1], d[:, :, 2]
    state = ops.linattn_state(k, v, head_dim=D)
    assert state.shape == (B, C // D, 1, D + 1, D) and state.dtype == torch.float32
    assert rel_l2(state.cpu()[:, :, 0], ref_state) <= 1e-5
    # every entry, not only the norm: a misplaced tile would hide in a norm
    assert (state.cpu()[:, :, 0].double() - ref_state).abs().max().item() <= 1e-4 * ref_state.abs().max().item()
    out32 = ops.linattn_apply(q, state, eps, out_dtype=torch.float32)
    assert rel_l2(out32.cpu(), ref_out) <= 1e-5
    out = ops.linattn_apply(q, state, eps)
    assert out.dtype == torch.bfloat16
    assert (out.cpu().double() - ref_out).abs().max().item() <= 2e-2
    assert rel_l2(out.cpu(), ref_out) <= 1e-2
    # the bf16-output kernel applies the state as two bf16 terms (16 mantissa bits): one unit in the last place
    # of the correctly rounded fp32 result, plus 2^-16 of the output scale where the numerator cancels
    floor = 2.0 ** -16 * out32.abs().max().item()
    bad = ((out.float() - out32).abs() > 2.0 ** -7 * out32.abs() + floor).sum().item()
    assert bad == 0


def test_f16_state(cuda):
    qkv = _qkv(2, 300, 224, seed=5, dtype=torch.float16)
    _, ref_state = _oracle(qkv, 1e-8)
    d = qkv.to(cuda)
    state = ops.linattn_state(d[:, :, 1], d[:, :, 2], head_dim=D)
    assert rel_l2(state.cpu()[:, :, 0], ref_state) <= 1e-5


def test_deterministic_and_additive(cuda):
    B, N, C = 1, 8192, 2240
    qkv = _qkv(B, N, C, 1).to(cuda)
    k, v = qkv[:, :, 1], qkv[:, :, 2]
    s1 = ops.linattn_state(k, v, head_dim=D).clone()
    s2 = ops.linattn_state(k, v, head_dim=D)
    assert torch.equal(s1, s2)
    s_a = ops.linattn_state(k[:, :3000], v[:, :3000], head_dim=D)
    s_b = ops.linattn_state(k[:, 3000:], v[:, 3000:], head_dim=D)
    assert rel_l2(s_a + s_b, s1) < 1e-6
    ksum = torch.relu(k.float()).sum(1).view(B, C // D, D)
    assert rel_l2(s1[:, :, 0, D], ksum) < 1e-5
    # constant v = c  =>  out = c * den / (den + eps) ~= c
    qkv_c = qkv.clone()
    qkv_c[:, :, 2] = 1.5
    out = ops.relu_linear_attention(qkv_c[:, :, 0], qkv_c[:, :, 1], qkv_c[:, :, 2], 1e-8, out_dtype=torch.float32,
                                    head_dim=D)
    assert (out - 1.5).abs().max().item() < 1e-4


@pytest.mark.parametrize("frames,hw,chunk_frames", [(4, 6, [0, 1, 2, 3]), (5, 37, [0, 2]), (21, 1560, [0, 11]),
                                                    (40, 30, list(range(40))),        # 40 chunks shorter than a tile
                                                    (33, 100, list(range(0, 33, 2)))])  # 17 chunks, several per range
def test_chunk_causal_matches_oracle(cuda, frames, hw, chunk_frames):
    B, C, eps = 1, 224, 1e-8
    N = frames * hw
    h = C // D
    qkv = _qkv(B, N, C, seed=frames * 7)
    bounds = [f * hw for f in chunk_frames] + [N]
    q, k, v = (_heads(qkv[:, :, i], B, N, h) for i in range(3))
    outs, run = [], 0
    for a, b in zip(bounds[:-1], bounds[1:]):
        _, st = O.relu_linear_attention(q[..., a:b], k[..., a:b].transpose(-1, -2), v[..., a:b], eps, return_state=True)
        run = run + st
        o = run @ torch.relu(q[..., a:b])
        outs.append(o[:, :, :-1] / (o[:, :, -1:] + eps))
    ref = torch.cat(outs, -1).permute(0, 3, 1, 2).reshape(B, N, C)
    d = qkv.to(cuda)
    out = ops.relu_linear_attention(d[:, :, 0], d[:, :, 1], d[:, :, 2], eps, chunk_tokens=bounds[:-1],
                                    out_dtype=torch.float32, head_dim=D)
    assert rel_l2(out.cpu(), ref) <= 1e-5


def test_chunk_scan_entry_point(cuda):
    st = torch.randn(2, 3, 5, D + 1, D, device=cuda)
    ref = st.cumsum(2)
    ops.linattn_chunk_scan_(st)
    torch.testing.assert_close(st, ref, rtol=1e-6, atol=1e-6)


@pytest.mark.parametrize("norm,rot", [(True, False), (False, True), (True, True)])
@pytest.mark.parametrize("B,N,C", [(2, 333, 224), (1, 4096, 2240)])
def test_norm_and_rope_on_load(cuda, B, N, C, norm, rot):
    """q/k RMSNorm over all channels before the ReLU and the complex rotation after it, applied inside the kernels,
    against the oracle's RMSNorm and rotary_complex in fp64 on the bf16-rounded intermediate values."""
    eps, h = 1e-8, C // D
    qkv = _qkv(B, N, C, seed=3 * N + C)
    g = torch.Generator().manual_seed(11)
    wq = (1.0 + 0.3 * torch.randn(C, generator=g)).bfloat16()
    wk = (1.0 + 0.3 * torch.randn(C, generator=g)).bfloat16()
    theta = torch.rand(N, D // 2, generator=g, dtype=torch.float64) * 6.283
    freqs = torch.polar(torch.ones_like(theta), theta)[None, None]
    q, k, v = qkv[:, :, 0], qkv[:, :, 1], qkv[:, :, 2]
    if norm:
        nq, nk = O.RMSNorm(C, eps=1e-5), O.RMSNorm(C, eps=1e-5)
        with torch.no_grad():
            nq.weight.copy_(wq.float())
            nk.weight.copy_(wk.float())
            q, k = nq.bfloat16()(q), nk.bfloat16()(k)        # bf16 out, fp32 inside: what the reference computes
    qh, kh, vh = (_heads(t, B, N, h) for t in (q, k, v))
    qr, kr = torch.relu(qh), torch.relu(kh)
    if rot:
        # the reference rotates in fp64 and casts back to the io dtype (bf16)
        q_rot = O.rotary_complex(qr.bfloat16(), freqs).double()
        k_rot = O.rotary_complex(kr.bfloat16(), freqs).double()
    else:
        q_rot, k_rot = qr, kr
    vk = vh @ k_rot.transpose(-1, -2)
    num = vk @ q_rot
    den = kr.sum(-1, keepdim=True).transpose(-1, -2) @ qr
    ref = (num / (den + eps)).permute(0, 3, 1, 2).reshape(B, N, C)

    d = qkv.to(cuda)
    dq, dk, dv = d[:, :, 0], d[:, :, 1], d[:, :, 2]
    rq = rk = None
    if norm:
        rq, rk = ops.qk_rms(dq, dk, 1e-5)
    table = ops.rope_table(freqs, N, cuda, head_dim=D) if rot else None
    pre_k = ops.QkPre(rk, wk.to(cuda) if norm else None, table)
    pre_q = ops.QkPre(rq, wq.to(cuda) if norm else None, table)
    state = ops.linattn_state(dk, dv, pre=pre_k, head_dim=D)
    out = ops.linattn_apply(dq, state, eps, pre=pre_q)
    assert (out.cpu().double() - ref).abs().max().item() <= 2e-2
    assert rel_l2(out.cpu(), ref) <= 1e-2
    out32 = ops.linattn_apply(dq, state, eps, pre=pre_q, out_dtype=torch.float32)
    assert rel_l2(out32.cpu(), ref) <= 2e-3     # bf16 roundings of the normalised / rotated operands remain
