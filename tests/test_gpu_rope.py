"""GPU parity of the attention variants with q/k RMSNorm and rotary embedding applied inside the
kernels (LiteLAReLURope, ChunkCausalAttention with rotary_emb, CachedCausalAttention) against the
oracle's restatement of the reference modules, same state_dict, same seeded inputs."""
import copy

import pytest
import torch

import sana_amd as S
from oracle import sana_oracle as O
from sana_amd import ops

pytestmark = pytest.mark.gpu


def rel_l2(a, b):
    return ((a.double() - b.double()).norm() / b.double().norm()).item()


def check(out, ref, what=""):
    """north-star tolerance for bf16 attention outputs: max-abs 2e-2, rel-L2 1e-2 (against fp64)."""
    mx = (out.double().cpu() - ref.double()).abs().max().item()
    rl = rel_l2(out.cpu(), ref)
    assert mx <= 2e-2 and rl <= 1e-2, f"{what}: max-abs {mx:.3e} rel-L2 {rl:.3e}"


def freqs(N, seed=0, head_dim=32):
    """Unit complex rotary factors [1, 1, N, head_dim/2], as the reference passes rotary_emb."""
    theta = torch.rand(N, head_dim // 2, generator=torch.Generator().manual_seed(seed), dtype=torch.float64) * 6.283
    return torch.polar(torch.ones_like(theta), theta)[None, None]


def make(cls_name, C, qk_norm, seed, head_dim=32):
    heads = C // head_dim
    om = getattr(O, cls_name)(C, C, heads=heads, eps=1e-8, qk_norm=qk_norm)
    g = torch.Generator().manual_seed(seed)
    with torch.no_grad():
        for n, p in om.named_parameters():
            if "norm" in n:
                p.copy_(1.0 + 0.3 * torch.randn(p.shape, generator=g))
            elif n.endswith("bias"):
                p.copy_(torch.randn(p.shape, generator=g) * 0.05)
            else:
                p.copy_(torch.randn(p.shape, generator=g) * (2.0 / C) ** 0.5)
    om = om.bfloat16()
    hm = getattr(S, cls_name)(C, C, heads=heads, eps=1e-8, qk_norm=qk_norm).bfloat16()
    hm.load_state_dict(om.state_dict(), strict=True)
    return om, hm


def ref64(module, x, **kw):
    m = copy.deepcopy(module).double()
    return m(x.double(), **kw)


@pytest.mark.parametrize("B,N,C", [(2, 1024, 1152), (1, 16384, 2240)])
def test_qk_rms_statistic(cuda, B, N, C):
    g = torch.Generator().manual_seed(N + C)
    qkv = (torch.randn(B, N, 3, C, generator=g) * 1.7).bfloat16().to(cuda)
    rq, rk = ops.qk_rms(qkv[:, :, 0], qkv[:, :, 1], 1e-5)
    for r, x in ((rq, qkv[:, :, 0]), (rk, qkv[:, :, 1])):
        ref = torch.rsqrt(x.double().pow(2).mean(-1) + 1e-5)
        assert r.shape == (B, N) and r.dtype == torch.float32
        assert ((r.double() - ref).abs() / ref).max().item() <= 2e-6


@pytest.mark.parametrize("qk_norm", [False, True])
@pytest.mark.parametrize("rot", [False, True])
@pytest.mark.parametrize("B,N,C", [(2, 640, 1152), (1, 77, 96), (1, 4096, 2240)])
def test_litela_relu_rope(cuda, B, N, C, qk_norm, rot):
    om, hm = make("LiteLAReLURope", C, qk_norm, seed=N)
    hm = hm.to(cuda)
    x = torch.randn(B, N, C, generator=torch.Generator().manual_seed(1)).bfloat16()
    f = freqs(N) if rot else None
    with torch.no_grad():
        ref = ref64(om, x, rotary_emb=f)
        out = hm(x.to(cuda), rotary_emb=None if f is None else f.to(cuda))
    assert out.dtype == torch.bfloat16 and out.shape == (B, N, C)
    check(out, ref, f"LiteLAReLURope norm={qk_norm} rope={rot}")


@pytest.mark.parametrize("qk_norm", [False, True])
@pytest.mark.parametrize("B,N,C", [(2, 640, 224), (1, 4096, 2240)])
def test_litela_relu_rope_head_dim_112(cuda, B, N, C, qk_norm):
    """The video configurations' linear_head_dim = 112 (2240 = 20 heads of 112)."""
    om, hm = make("LiteLAReLURope", C, qk_norm, seed=N, head_dim=112)
    hm = hm.to(cuda)
    assert hm.dim == 112
    x = torch.randn(B, N, C, generator=torch.Generator().manual_seed(1)).bfloat16()
    f = freqs(N, head_dim=112)
    with torch.no_grad():
        ref = ref64(om, x, rotary_emb=f)
        out = hm(x.to(cuda), rotary_emb=f.to(cuda))
    check(out, ref, f"LiteLAReLURope d=112 norm={qk_norm}")


def test_cached_stream_head_dim_112(cuda):
    """Streaming chunks with 112-wide heads: each step against the oracle's cached module, and the saved state
    has the reference's kv_cache shapes."""
    B, hw, C = 1, 48, 224
    om, hm = make("CachedCausalAttention", C, True, seed=6, head_dim=112)
    hm = hm.to(cuda)
    o64 = copy.deepcopy(om).double()
    starts = [0, 2, 3, 5]
    N = starts[-1] * hw
    x = torch.randn(B, N, C, generator=torch.Generator().manual_seed(7)).bfloat16()
    fr = freqs(N, 8, head_dim=112)
    acc, acc_ref = None, None
    with torch.no_grad():
        for a, b in zip(starts[:-1], starts[1:]):
            xs, fs = x[:, a * hw:b * hw], fr[:, :, a * hw:b * hw]
            cache = [None, None] if acc is None else [acc[0], acc[1]]
            out, cache = hm(xs.to(cuda), rotary_emb=fs.to(cuda), save_kv_cache=True, kv_cache=cache)
            assert cache[0].shape == (B, 2, 112, 112) and cache[1].shape == (B, 2, 1, 112)
            acc = S.accumulate_kv_cache(acc, cache)
            cache_ref = [None, None] if acc_ref is None else [acc_ref[0], acc_ref[1]]
            ref, cache_ref = o64(xs.double(), rotary_emb=fs, save_kv_cache=True, kv_cache=cache_ref)
            acc_ref = cache_ref if acc_ref is None else [acc_ref[0] + cache_ref[0], acc_ref[1] + cache_ref[1]]
            check(out, ref, f"cached chunk {a}:{b} d=112")


def test_rotation_is_numerator_only_and_unit_rotation_is_identity(cuda):
    """theta = 0 must reproduce the call without rotary_emb bit for bit; a rotation by pi flips the sign of
    every rotated q and k, which cancels in the numerator (vk . q_rot) and never touches the denominator."""
    B, N, C = 1, 512, 256
    om, hm = make("LiteLAReLURope", C, False, seed=9)
    hm = hm.to(cuda)
    x = torch.randn(B, N, C, generator=torch.Generator().manual_seed(2)).bfloat16().to(cuda)
    one = torch.ones(1, 1, N, 16, dtype=torch.complex128)
    with torch.no_grad():
        base = hm(x)
        assert torch.equal(hm(x, rotary_emb=one.to(cuda)), base)
        assert torch.equal(hm(x, rotary_emb=(-one).to(cuda)), base)


@pytest.mark.parametrize("qk_norm", [False, True])
@pytest.mark.parametrize("frames,hw,chunk_index", [(24, (5, 6), list(range(24))),      # every chunk shorter than a tile
                                                   (9, (20, 23), [0, 1, 2, 5, 8])])   # chunks of 460 .. 1380 tokens
def test_chunk_causal_with_rope_head_dim_112_many_chunks(cuda, qk_norm, frames, hw, chunk_index):
    """The 112-wide-head kernels walk token ranges across chunk boundaries: records per (range, chunk), the unrotated
    key sums folded when a chunk ends (at every tile in the first case), the state operands rebuilt per chunk."""
    B, C = 2, 448
    N = frames * hw[0] * hw[1]
    om, hm = make("ChunkCausalAttention", C, qk_norm, seed=9, head_dim=112)
    hm = hm.to(cuda)
    x = torch.randn(B, N, C, generator=torch.Generator().manual_seed(N)).bfloat16()
    fr = freqs(N, 2, head_dim=112)
    with torch.no_grad():
        ref = ref64(om, x, HW=(frames, *hw), rotary_emb=fr, chunk_index=chunk_index)
        out = hm(x.to(cuda), HW=(frames, *hw), rotary_emb=fr.to(cuda), chunk_index=chunk_index)
    check(out, ref, "ChunkCausalAttention d=112 + rope, many chunks")


@pytest.mark.parametrize("qk_norm", [False, True])
@pytest.mark.parametrize("C,head_dim", [(160, 32), (224, 112)])
def test_chunk_causal_with_rope(cuda, qk_norm, C, head_dim):
    B, (f, h, w) = 1, (5, 6, 8)
    N = f * h * w
    om, hm = make("ChunkCausalAttention", C, qk_norm, seed=4, head_dim=head_dim)
    hm = hm.to(cuda)
    x = torch.randn(B, N, C, generator=torch.Generator().manual_seed(3)).bfloat16()
    fr = freqs(N, 5, head_dim=head_dim)
    with torch.no_grad():
        ref = ref64(om, x, HW=(f, h, w), rotary_emb=fr, chunk_index=[0, 1, 3])
        out = hm(x.to(cuda), HW=(f, h, w), rotary_emb=fr.to(cuda), chunk_index=[0, 1, 3])
    check(out, ref, "ChunkCausalAttention + rope")


def test_cached_stream_equals_chunk_causal(cuda):
    """Feeding chunks one at a time through CachedCausalAttention, with the caller accumulating the
    saved states, reproduces the chunk-causal module on the whole sequence; and each step matches
    the oracle's cached module given the same accumulated past."""
    B, (f, h, w), C = 2, (6, 4, 8), 128
    hw = h * w
    N = f * hw
    om, hm = make("CachedCausalAttention", C, True, seed=6)
    whole = S.ChunkCausalAttention(C, C, heads=C // 32, eps=1e-8, qk_norm=True).bfloat16()
    whole.load_state_dict(om.state_dict(), strict=True)
    hm, whole = hm.to(cuda), whole.to(cuda)
    x = torch.randn(B, N, C, generator=torch.Generator().manual_seed(7)).bfloat16()
    fr = freqs(N, 8)
    starts = [0, 2, 3, 6]
    with torch.no_grad():
        full = whole(x.to(cuda), HW=(f, h, w), rotary_emb=fr.to(cuda), chunk_index=starts[:-1])
        acc, acc_ref = None, None
        o64 = copy.deepcopy(om).double()
        for a, b in zip(starts[:-1], starts[1:]):
            xs, fs = x[:, a * hw:b * hw], fr[:, :, a * hw:b * hw]
            cache = [None, None] if acc is None else [acc[0], acc[1]]
            out, cache = hm(xs.to(cuda), rotary_emb=fs.to(cuda), save_kv_cache=True, kv_cache=cache)
            assert cache[0].shape == (B, C // 32, 32, 32) and cache[1].shape == (B, C // 32, 1, 32)
            acc = S.accumulate_kv_cache(acc, cache)
            # the streamed chunk equals the same tokens of the whole-sequence chunk-causal call
            assert (out.float() - full[:, a * hw:b * hw].float()).abs().max().item() <= 2e-2
            # and the oracle's cached module, given its own accumulated past
            cache_ref = [None, None] if acc_ref is None else [acc_ref[0], acc_ref[1]]
            ref, cache_ref = o64(xs.double(), rotary_emb=fs, save_kv_cache=True, kv_cache=cache_ref)
            acc_ref = cache_ref if acc_ref is None else [acc_ref[0] + cache_ref[0], acc_ref[1] + cache_ref[1]]
            check(out, ref, f"cached chunk {a}:{b}")
            assert rel_l2(cache[0].cpu(), cache_ref[0]) <= 1e-2 and rel_l2(cache[1].cpu(), cache_ref[1]) <= 1e-2


# ---------------------------------------------------------------- LiteLA.forward's own order: rotation BEFORE the ReLU


def real_tables(N, seed, head_dim=32, pair_equal=True):
    """(cos, sin) [N, head_dim] as LiteLA.forward receives them (sana_blocks.py:282-284); generic angles."""
    g = torch.Generator().manual_seed(seed)
    if pair_equal:
        theta = (torch.rand(N, head_dim // 2, generator=g) * 6.283).repeat_interleave(2, 1)
    else:
        theta = torch.rand(N, head_dim, generator=g) * 6.283
    return torch.cos(theta), torch.sin(theta)


@pytest.mark.parametrize("B,N,C,qk_norm", [(2, 1024, 1152, False), (2, 1024, 1152, True), (1, 16384, 2240, True),
                                           (3, 77, 96, True)])
def test_litela_pre_relu_rotary_runs_in_the_kernels(cuda, caplog, B, N, C, qk_norm):
    """LiteLA with image_rotary_emb: RMSNorm, the real-valued rotation before the ReLU and the ReLU happen on load in
    the two attention kernels (no stock-op pass over the qkv buffer is logged), within the attention tolerance of the
    oracle module in fp64 on the same bf16 weights and inputs."""
    import logging
    om, hm = make("LiteLA", C, qk_norm, seed=N + C)
    hm = hm.to(cuda)
    x = torch.randn(B, N, C, generator=torch.Generator().manual_seed(5)).bfloat16()
    cos, sin = real_tables(N, 7)
    with torch.no_grad():
        ref = ref64(om, x, rotary_emb=(cos.double(), sin.double()))
        S.modules._stock_paths_seen.clear()
        with caplog.at_level(logging.WARNING, logger="sana_amd"):
            out = hm(x.to(cuda), rotary_emb=(cos.to(cuda), sin.to(cuda)))
    assert not [r for r in caplog.records if "LiteLA" in r.getMessage()], [r.getMessage() for r in caplog.records]
    check(out, ref, f"LiteLA pre-ReLU rotary, qk_norm={qk_norm}")


def test_litela_pre_relu_rotary_state_and_output_against_explicit_rotation(cuda):
    """The kernels' rotate-first order against the same kernels WITHOUT transforms on explicitly rotated inputs
    (rotation in fp32 with the fmas of the kernel, rounded to bf16): the vk block of the state is bit-identical (same
    MFMA operands, same order), its ksum row and the output agree to fp32 summation order.  A rotation pins what the
    order means: rotating AFTER the ReLU (the LiteLAReLURope order) on the same inputs gives another state."""
    B, N, h = 2, 1000, 6
    C = 32 * h
    g = torch.Generator().manual_seed(3)
    q, k, v = ((torch.randn(B, N, C, generator=g) * 1.3).bfloat16().to(cuda) for _ in range(3))
    cos, sin = real_tables(N, 11)
    table = ops.rope_table_real(cos, sin, N, cuda)
    assert table is not None and tuple(table.shape) == (N, 16, 2)
    assert ops.rope_table_real(*real_tables(N, 11, pair_equal=False), N, cuda) is None

    def rotate(t):
        x = t.float().view(B, N, h, 16, 2)
        c, s = table[None, :, None, :, 0], table[None, :, None, :, 1]
        x0, x1 = x[..., 0], x[..., 1]
        r0 = torch.addcmul(-(x1 * s), x0, c)      # fma(x0, c, -(x1 * s))
        r1 = torch.addcmul(x1 * c, x0, s)         # fma(x0, s, x1 * c)
        return torch.stack([r0, r1], dim=-1).view(B, N, C).bfloat16()

    pre = ops.QkPre(rope=table, rope_first=True)
    st = ops.linattn_state(k, v, pre=pre)
    st_ref = ops.linattn_state(rotate(k), v)
    # fma contraction on the host may differ from the kernel's in the last fp32 bit of a rotated value, which can flip
    # its bf16 rounding: compare the states at the level of a few such flips
    assert rel_l2(st[:, :, :, :32], st_ref[:, :, :, :32]) <= 2e-4
    assert rel_l2(st[:, :, :, 32:], st_ref[:, :, :, 32:]) <= 2e-4
    out = ops.linattn_apply(q, st_ref, 1e-8, pre=pre)
    out_ref = ops.linattn_apply(rotate(q), st_ref, 1e-8)
    assert rel_l2(out, out_ref) <= 2e-3 and (out.float() - out_ref.float()).abs().max().item() <= 2e-2
    st_after = ops.linattn_state(k, v, pre=ops.QkPre(rope=table))           # ReLU first, then the rotation
    assert rel_l2(st_after[:, :, :, :32], st_ref[:, :, :, :32]) > 0.1


def test_litela_rotary_tables_without_pair_structure_take_the_stock_pass(cuda, caplog):
    """cos / sin tables whose two entries per channel pair differ are no rotation of the pair: the module applies them
    with stock ops on the qkv buffer (logged) and still matches the oracle."""
    import logging
    B, N, C = 2, 200, 96
    om, hm = make("LiteLA", C, True, seed=9)
    hm = hm.to(cuda)
    x = torch.randn(B, N, C, generator=torch.Generator().manual_seed(5)).bfloat16()
    cos, sin = real_tables(N, 7, pair_equal=False)
    with torch.no_grad():
        ref = ref64(om, x, rotary_emb=(cos.double(), sin.double()))
        S.modules._stock_paths_seen.clear()
        with caplog.at_level(logging.WARNING, logger="sana_amd"):
            out = hm(x.to(cuda), rotary_emb=(cos.to(cuda), sin.to(cuda)))
    assert any("LiteLA rotary embedding" in r.getMessage() for r in caplog.records)
    check(out, ref, "LiteLA generic real tables")


def test_chunk_causal_head_dim_112_replays_from_a_hip_graph(cuda):
    """The 112-wide-head kernels (rings of direct-to-LDS loads, counted waits, records per range and chunk) captured
    once: every replay, with eager launches and synchronisations between them, equals the eager result bit for bit,
    also after the input changes."""
    B, C, (f, h, w) = 1, 448, (6, 10, 13)
    N = f * h * w
    om, hm = make("ChunkCausalAttention", C, True, seed=12, head_dim=112)
    hm = hm.to(cuda)
    x = torch.randn(B, N, C, generator=torch.Generator().manual_seed(1)).bfloat16().to(cuda)
    fr = freqs(N, 3, head_dim=112).to(cuda)
    kw = dict(HW=(f, h, w), rotary_emb=fr, chunk_index=[0, 1, 4])
    with torch.no_grad():
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):           # warm-up off the default stream, as capture requires
            for _ in range(2):
                hm(x, **kw)
        torch.cuda.current_stream().wait_stream(side)
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            out = hm(x, **kw)
        for r in range(3):
            if r == 2:
                x.copy_(torch.randn(x.shape, generator=torch.Generator().manual_seed(9)).bfloat16())
            graph.replay()
            torch.cuda.synchronize()
            eager = hm(x, **kw)
            torch.cuda.synchronize()
            assert torch.equal(out, eager), f"replay {r}"
        check(out, ref64(om, x.cpu(), HW=(f, h, w), rotary_emb=fr.cpu(), chunk_index=[0, 1, 4]), "graph replay, d=112")
