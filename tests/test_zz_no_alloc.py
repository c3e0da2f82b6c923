"""``sana_hip_linattn_state_noalloc`` (phase 1 with the partial states in the library's fixed per-GPU scratch
array, for callers that cannot allocate) against ``sana_hip_linattn_state`` / ``sana_hip_linattn_state_pre`` with a
caller-provided workspace: same kernels, same split plan, so the states must agree bit for bit.  Called through
the C ABI with every buffer allocated beforehand; two calls in a row, the second on a smaller input (the array
keeps the first call's contents)."""
import numpy as np
import pytest
import torch

from sana_amd import _lib, ops

pytestmark = pytest.mark.gpu

BF16 = _lib.DT_BF16


def _qkv(B, N, C, seed, dev):
    g = torch.Generator().manual_seed(seed)
    return torch.randn(B, N, 3, C, generator=g).bfloat16().to(dev)


@pytest.fixture(scope="module", autouse=True)
def first_call_on_the_device(cuda):
    """The entry point's first call on a device resolves the scratch array's address (which makes the runtime load
    the code object that holds the array): set-up, done here once so the tests below can watch device memory."""
    qkv = _qkv(1, 64, 64, 9, cuda)
    state = torch.empty(1, 2, 1, 33, 32, device=cuda)
    ops.linattn_state(qkv[:, :, 1], qkv[:, :, 2], out=state, noalloc=True)
    torch.cuda.synchronize()


def _both(lib, qkv, d, chunk_starts, causal, rope, dev):
    """(state via the workspace entry point, state via the no-allocation entry point, bytes torch allocated and
    bytes of device memory that disappeared during the no-allocation call)."""
    B, N, _, C = qkv.shape
    h = C // d
    k, v = qkv[:, :, 1], qkv[:, :, 2]
    sb, sn = (k.stride(0) if B > 1 else 0), k.stride(1)
    if chunk_starts is None:
        tab, n_chunks, longest = None, 1, N
    else:
        bounds = list(chunk_starts) + [N]
        tab = torch.tensor(bounds, dtype=torch.int32, device=dev)
        n_chunks, longest = len(bounds) - 1, max(b - a for a, b in zip(bounds[:-1], bounds[1:]))
    tabp = None if tab is None else tab.data_ptr()
    ropep = None if rope is None else rope.data_ptr()
    need = lib.sana_hip_linattn_workspace_bytes(B, h, d, n_chunks, longest, BF16)
    ws = torch.empty(max(need, 16), dtype=torch.uint8, device=dev)
    ref = torch.full((B, h, n_chunks, d + 1, d), float("nan"), device=dev)
    out = torch.full((B, h, n_chunks, d + 1, d), float("nan"), device=dev)
    stream = torch.cuda.current_stream().cuda_stream
    shape = (B, N, h, d, sb, sn, tabp, n_chunks, longest, 1 if causal else 0, BF16)
    code = lib.sana_hip_linattn_state_pre(k.data_ptr(), v.data_ptr(), ref.data_ptr(), ws.data_ptr(), need, *shape,
                                          None, None, ropep, stream)
    assert code == 0, code
    torch.cuda.synchronize()
    t0, free0 = torch.cuda.memory_allocated(), torch.cuda.mem_get_info()[0]
    code = lib.sana_hip_linattn_state_noalloc(k.data_ptr(), v.data_ptr(), out.data_ptr(), *shape, None, None, ropep,
                                              stream)
    assert code == 0, code
    torch.cuda.synchronize()
    return ref, out, torch.cuda.memory_allocated() - t0, free0 - torch.cuda.mem_get_info()[0], need


def test_two_calls_in_a_row_match_the_workspace_entry_point(cuda):
    lib = _lib.load()
    # call 1: the 1.6B block at 16384 tokens (26 token splits per pair of heads: 7.3 MiB of partial states)
    big = _qkv(1, 16384, 2240, 0, cuda)
    ref, out, grew, lost, need = _both(lib, big, 32, None, False, None, cuda)
    print(f"call 1: B=1 N=16384 C=2240 d=32, partial states {need / 2**20:.1f} MiB", flush=True)
    assert need > 0 and torch.equal(ref, out) and not torch.isnan(out).any()
    assert grew == 0 and lost <= 0
    # and it is the right answer, not only the same one: row 32 of every state is sum_n relu(k_n)
    ksum = torch.relu(big[0, :, 1].float()).sum(0).view(70, 32)
    assert ((out[0, :, 0, 32] - ksum).abs() / ksum).max().item() < 1e-4
    # call 2, smaller: 3 causal chunks of a short sequence, fewer heads -- other slots, other split count
    small = _qkv(2, 1500, 96, 1, cuda)
    ref, out, grew, lost, need = _both(lib, small, 32, [0, 400, 1100], True, None, cuda)
    print(f"call 2: B=2 N=1500 C=96 d=32, 3 causal chunks, partial states {need / 2**20:.2f} MiB", flush=True)
    assert need > 0 and torch.equal(ref, out) and not torch.isnan(out).any()
    assert grew == 0 and lost <= 0
    # call 3, smaller again and with no split at all (the scratch array is not used): still the same
    tiny = _qkv(1, 200, 64, 2, cuda)
    ref, out, _, _, need = _both(lib, tiny, 32, None, False, None, cuda)
    assert need == 0 and torch.equal(ref, out)


def test_head_dim_112_with_rotary_table_then_a_smaller_call(cuda):
    lib = _lib.load()
    N = 4096
    theta = torch.rand(N, 56, generator=torch.Generator().manual_seed(3), dtype=torch.float64) * 6.283
    rope = torch.stack([torch.cos(theta), torch.sin(theta)], -1).float().contiguous().to(cuda)
    a = _qkv(1, N, 2240, 4, cuda)
    ref, out, grew, lost, need = _both(lib, a, 112, [0, 1024, 3072], True, rope, cuda)
    print(f"d=112 N={N} 3 causal chunks + rotary table, partial states {need / 2**20:.1f} MiB", flush=True)
    assert need > 0 and torch.equal(ref, out) and not torch.isnan(out).any() and grew == 0 and lost <= 0
    b = _qkv(1, 640, 224, 5, cuda)
    ref, out, _, _, need = _both(lib, b, 112, None, False, rope[:640].contiguous(), cuda)
    assert need > 0 and torch.equal(ref, out) and not torch.isnan(out).any()


def test_head_dim_112_video_shape_with_21_causal_chunks_fits(cuda):
    """One video of 21 x 1560 tokens, 20 heads of 112, a causal chunk per frame: 32 records per head, 30.9 MiB."""
    lib = _lib.load()
    per, n_chunks = 1560, 21
    a = _qkv(1, per * n_chunks, 2240, 8, cuda)
    ref, out, grew, lost, need = _both(lib, a, 112, [f * per for f in range(n_chunks)], True, None, cuda)
    print(f"d=112 N={per * n_chunks} 21 causal chunks, partial states {need / 2**20:.1f} MiB", flush=True)
    assert 30 * 2**20 < need <= ops.NOALLOC_SCRATCH_BYTES
    assert torch.equal(ref, out) and not torch.isnan(out).any() and grew == 0 and lost <= 0


def test_python_wrapper_and_the_size_limit(cuda):
    lib = _lib.load()
    qkv = _qkv(2, 3000, 256, 6, cuda)
    want = ops.linattn_state(qkv[:, :, 1], qkv[:, :, 2], [0, 1000], causal=True)
    got = torch.empty_like(want)
    assert ops.linattn_state(qkv[:, :, 1], qkv[:, :, 2], [0, 1000], causal=True, out=got, noalloc=True) is got
    assert torch.equal(want, got)
    # 4 videos x 20 heads of 112 x 21 chunks want 81 MiB of partial states: refused, nothing launched
    B, h, d, n_chunks, per = 4, 20, 112, 21, 1560
    need = lib.sana_hip_linattn_workspace_bytes(B, h, d, n_chunks, per, BF16)
    assert need > ops.NOALLOC_SCRATCH_BYTES
    sentinel = torch.full((64,), 7.0, device=cuda)
    tab = torch.arange(0, (n_chunks + 1) * per, per, dtype=torch.int32, device=cuda)
    code = lib.sana_hip_linattn_state_noalloc(sentinel.data_ptr(), sentinel.data_ptr(), sentinel.data_ptr(), B,
                                              n_chunks * per, h, d, n_chunks * per * h * d, h * d, tab.data_ptr(),
                                              n_chunks, per, 1, BF16, None, None, None, None)
    assert code == -7 and b"scratch" in lib.sana_hip_strerror(code)
    torch.cuda.synchronize()
    assert torch.equal(sentinel, torch.full((64,), 7.0, device=cuda))
