"""GPU parity of the linear-attention kernels (through the C ABI) against the oracle."""
import pytest
import torch

from oracle import sana_oracle as O
from sana_amd import ops

pytestmark = pytest.mark.gpu


def _qkv(B, N, C, dtype, seed):
    g = torch.Generator().manual_seed(seed)
    return torch.randn(B, N, 3, C, generator=g).to(dtype)


def _oracle(qkv, eps, chunk_of=None):
    """fp64 oracle on the values the kernel sees (inputs already rounded to the io dtype)."""
    B, N, _, C = qkv.shape
    h = C // 32
    q, k, v = (qkv[:, :, i].double().view(B, N, h, 32).permute(0, 2, 3, 1) for i in range(3))
    out, state = O.relu_linear_attention(q, k.transpose(-1, -2), v, eps, return_state=True)
    return out.permute(0, 3, 1, 2).reshape(B, N, C), state


def rel_l2(a, b):
    return ((a.double() - b.double()).norm() / b.double().norm()).item()


CASES = [
    # B, N, C, dtype
    (1, 1024, 1152, torch.float32),    # cfg1: Sana-600M op alone
    (4, 1024, 1152, torch.bfloat16),   # cfg2 attention shape
    (1, 16384, 2240, torch.bfloat16),  # cfg3 attention shape (split over tokens)
    (2, 777, 96, torch.bfloat16),      # ragged token count, odd number of heads
    (1, 50, 32, torch.bfloat16),       # single head, one partial tile
    (2, 300, 160, torch.float16),
    (1, 1, 64, torch.bfloat16),        # one token
    (3, 129, 64, torch.float32),
]


@pytest.mark.parametrize("B,N,C,dtype", CASES)
def test_state_and_output_match_oracle(cuda, B, N, C, dtype):
    eps = 1e-15 if dtype == torch.float32 else 1e-8
    qkv = _qkv(B, N, C, dtype, seed=N + C)
    ref_out, ref_state = _oracle(qkv, eps)
    d = qkv.to(cuda)
    q, k, v = d[:, :, 0], d[:, :, 1], d[:, :, 2]   # strided views of the fused buffer, as LiteLA.forward sees them
    state = ops.linattn_state(k, v)
    assert state.shape == (B, C // 32, 1, 33, 32) and state.dtype == torch.float32
    # fp32 attention state: rel-L2 <= 1e-5 (north-star tolerance)
    assert rel_l2(state.cpu()[:, :, 0], ref_state) <= 1e-5
    out32 = ops.linattn_apply(q, state, eps, out_dtype=torch.float32)
    assert rel_l2(out32.cpu(), ref_out) <= 1e-5
    out = ops.linattn_apply(q, state, eps)
    assert out.dtype == dtype
    if dtype != torch.float32:
        # io-dtype output: max-abs 2e-2, rel-L2 1e-2 (north-star tolerance for bf16)
        assert (out.cpu().double() - ref_out).abs().max().item() <= 2e-2
        assert rel_l2(out.cpu(), ref_out) <= 1e-2
        # and it is the correctly rounded fp32 result up to one unit in the last place
        ulp, floor = (2.0 ** -7, 1e-30) if dtype == torch.bfloat16 else (2.0 ** -10, 2.0 ** -24)
        bad = ((out.float() - out32).abs() > ulp * out32.abs() + floor).sum().item()
        assert bad == 0


def test_bitwise_deterministic(cuda):
    qkv = _qkv(1, 4096, 2240, torch.bfloat16, 1).to(cuda)
    s1 = ops.linattn_state(qkv[:, :, 1], qkv[:, :, 2]).clone()
    s2 = ops.linattn_state(qkv[:, :, 1], qkv[:, :, 2])
    assert torch.equal(s1, s2)


def test_properties_at_full_size(cuda):
    """Size-independent properties at the 1.6B / 16384-token shape."""
    B, N, C = 1, 16384, 2240
    qkv = _qkv(B, N, C, torch.bfloat16, 7).to(cuda)
    q, k, v = qkv[:, :, 0], qkv[:, :, 1], qkv[:, :, 2]
    s_all = ops.linattn_state(k, v)
    # additivity of the state over token subsets
    s_a = ops.linattn_state(k[:, :5000], v[:, :5000])
    s_b = ops.linattn_state(k[:, 5000:], v[:, 5000:])
    assert rel_l2(s_a + s_b, s_all) < 1e-6
    # last row = sum of relu(k)
    ksum = torch.relu(k.float()).sum(1).view(B, C // 32, 32)
    assert rel_l2(s_all[:, :, 0, 32], ksum) < 1e-5
    # constant v = c  =>  out = c * den / (den + eps)  ~= c
    qkv_c = qkv.clone()
    qkv_c[:, :, 2] = 1.5
    out = ops.relu_linear_attention(qkv_c[:, :, 0], qkv_c[:, :, 1], qkv_c[:, :, 2], 1e-8, out_dtype=torch.float32)
    assert (out - 1.5).abs().max().item() < 1e-4
    # key/value permutation invariance (fp32 summation order changes only)
    perm = torch.randperm(N, device=cuda)
    s_p = ops.linattn_state(k[:, perm].contiguous(), v[:, perm].contiguous())
    assert rel_l2(s_p, s_all) < 1e-6
    # an all-negative query token gives exactly zero
    q2 = q.clone()
    q2[:, 123] = -q2[:, 123].abs() - 0.5
    out = ops.linattn_apply(q2, s_all, 1e-8)
    assert (out[:, 123] == 0).all()


def test_eps_is_runtime(cuda):
    qkv = _qkv(1, 64, 64, torch.bfloat16, 3).to(cuda)
    st = ops.linattn_state(qkv[:, :, 1], qkv[:, :, 2])
    a = ops.linattn_apply(qkv[:, :, 0], st, 1e-15, out_dtype=torch.float32)
    b = ops.linattn_apply(qkv[:, :, 0], st, 100.0, out_dtype=torch.float32)
    assert (a - b).abs().max().item() > 1e-3


@pytest.mark.parametrize("frames,hw,chunk_frames,dtype", [
    (4, 6, [0, 1, 2, 3], torch.bfloat16),
    (5, 37, [0, 2], torch.bfloat16),
    (3, 40, [0, 1], torch.float32),
    (21, 1560, [0, 11], torch.bfloat16),                      # cfg5 token count, two chunks
])
def test_chunk_causal_matches_oracle(cuda, frames, hw, chunk_frames, dtype):
    B, C, eps = 1, 96, 1e-8
    N = frames * hw
    qkv = _qkv(B, N, C, dtype, seed=frames * 7)
    h = C // 32
    # oracle: inclusive prefix of per-chunk states, as ChunkCausalAttention with a unit rotary
    bounds = [f * hw for f in chunk_frames] + [N]
    q, k, v = (qkv[:, :, i].double().view(B, N, h, 32).permute(0, 2, 3, 1) for i in range(3))
    outs, run = [], 0
    for a, b in zip(bounds[:-1], bounds[1:]):
        _, st = O.relu_linear_attention(q[..., a:b], k[..., a:b].transpose(-1, -2), v[..., a:b], eps, return_state=True)
        run = run + st
        o = run @ torch.relu(q[..., a:b])
        outs.append(o[:, :, :-1] / (o[:, :, -1:] + eps))
    ref = torch.cat(outs, -1).permute(0, 3, 1, 2).reshape(B, N, C)
    d = qkv.to(cuda)
    out = ops.relu_linear_attention(d[:, :, 0], d[:, :, 1], d[:, :, 2], eps, chunk_tokens=bounds[:-1],
                                    out_dtype=torch.float32)
    assert rel_l2(out.cpu(), ref) <= 1e-5


def test_chunk_scan_entry_point(cuda):
    st = torch.randn(2, 3, 5, 33, 32, device=cuda)
    ref = st.cumsum(2)
    ops.linattn_chunk_scan_(st)
    torch.testing.assert_close(st, ref, rtol=1e-6, atol=1e-6)
