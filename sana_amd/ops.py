"""Tensor-level wrappers over the C ABI: shape/dtype/device checks, pointer and
stride extraction, launch on torch's current stream.  Forward only, no autograd.
Empty inputs (no batch entries or no tokens) are answered here, after the argument
checks, without a launch: empty outputs, and an all-zero state for no tokens.
"""
from __future__ import annotations

from typing import Optional, Sequence, Tuple

import torch

from . import _lib
from ._lib import DT_BF16, DT_F16, DT_F32, SanaHipError

_DT = {torch.float32: DT_F32, torch.bfloat16: DT_BF16, torch.float16: DT_F16}
IO16 = (torch.bfloat16, torch.float16)   # the 16-bit io dtypes of the GEMMs and of the block's fused seams
HEAD_DIM = 32
HEAD_DIMS = (32, 112)   # head dims with kernels: 32 (all dtypes), 112 (bf16; the video configurations)

# Scratch buffers (attention partial states, split-k planes): one per (device, stream), so calls on different
# streams never share scratch memory; calls on one stream are ordered by it.  A buffer that has become too small
# is RETIRED, never freed: a captured HIP graph (or work still queued) may hold its address, and the allocator
# would hand freed memory to the next tensor.  Sizes grow in powers of two, so everything retired on a stream is
# smaller than its current buffer.
_workspaces = {}     # (device index, raw stream handle) -> list of uint8 tensors, the last one current
_chunk_tables = {}   # (device index, tuple) -> int32 tensor
_CACHE_LIMIT = 256   # small derived device tensors (chunk tables, frame flags) kept per process


def _remember(cache: dict, key, make):
    t = cache.get(key)
    if t is None:
        t = make()
        if len(cache) < _CACHE_LIMIT:   # ever-changing chunkings must not grow the cache without bound; entries
            cache[key] = t              # are never dropped (a captured graph may hold their addresses)
    return t


def _stream() -> int:
    # the current device's current stream as a raw handle; torch.cuda.current_stream() builds a Stream
    # object through several Python layers, which costs more host time per call than the launch it precedes
    return torch._C._cuda_getCurrentRawStream(torch._C._cuda_getDevice())


def _dt(t: torch.Tensor) -> int:
    try:
        return _DT[t.dtype]
    except KeyError:
        raise SanaHipError(f"unsupported dtype {t.dtype}") from None


def _need_cuda(*ts: torch.Tensor) -> None:
    for t in ts:
        if t is not None and not t.is_cuda:
            raise SanaHipError("the HIP kernels need device tensors (no CPU path exists)")


def _workspace(device: torch.device, nbytes: int, stream: Optional[int] = None) -> Optional[torch.Tensor]:
    if nbytes == 0:
        return None
    key = (device.index, _stream() if stream is None else stream)
    bufs = _workspaces.get(key)
    if bufs is None:
        bufs = _workspaces[key] = []
    if not bufs or bufs[-1].numel() < nbytes:
        size = 1 << 20
        while size < nbytes:
            size <<= 1
        bufs.append(torch.empty(size, dtype=torch.uint8, device=device))   # earlier ones stay alive in the list
    return bufs[-1]


def chunk_table(chunk_tokens: Optional[Sequence[int]], N: int, device) -> Tuple[Optional[torch.Tensor], int, int]:
    """chunk_tokens: token offsets of chunk starts (first is 0).  Returns
    (int32 device tensor [n+1] or None, n_chunks, longest chunk)."""
    if chunk_tokens is None or len(chunk_tokens) <= 1:
        return None, 1, N
    starts = list(chunk_tokens) + [N]
    if starts[0] != 0 or any(b <= a for a, b in zip(starts[:-1], starts[1:])):
        raise SanaHipError(f"chunk starts must begin at 0 and increase strictly below N={N}: {chunk_tokens}")
    key = (torch.device(device).index, tuple(starts))
    tab = _remember(_chunk_tables, key, lambda: torch.tensor(starts, dtype=torch.int32, device=device))
    return tab, len(starts) - 1, max(b - a for a, b in zip(starts[:-1], starts[1:]))


def _token_major_view(t: torch.Tensor, what: str) -> Tuple[int, int]:
    """t: [B, N, C] with unit channel stride -> (stride_b, stride_n) in elements."""
    if t.dim() != 3 or t.stride(2) != 1:
        raise SanaHipError(f"{what} must be a [B, N, C] view with unit channel stride, got strides {t.stride()}")
    return (t.stride(0) if t.shape[0] > 1 else 0), t.stride(1)


class QkPre:
    """Transforms applied to q or k on load inside the attention kernels (bf16 io):
    RMSNorm over all channels (``rinv`` [B, N] fp32 from :func:`qk_rms` and the bf16
    ``weight`` [C]) before the ReLU, rotary embedding (``rope`` [N, head_dim/2, 2] fp32 from
    :func:`rope_table`) after it, on the numerator operands only.  ``rope_first=True`` is the order of
    ``LiteLA.forward`` instead (sana_blocks.py:282-286): the rotation comes BEFORE the ReLU and every
    operand -- numerator, ksum row, denominator -- sees the rotated values (head_dim 32, one chunk)."""

    __slots__ = ("rinv", "weight", "rope", "rope_first")

    def __init__(self, rinv=None, weight=None, rope=None, rope_first: bool = False):
        if (rinv is None) != (weight is None):
            raise SanaHipError("rinv and weight go together")
        if rope_first and rope is None:
            raise SanaHipError("rope_first needs a rope table")
        self.rinv, self.weight, self.rope, self.rope_first = rinv, weight, rope, bool(rope_first)

    def check(self, x: torch.Tensor, head_dim: int = HEAD_DIM) -> Tuple[Optional[int], Optional[int], Optional[int]]:
        B, N, C = x.shape
        _need_cuda(self.rinv, self.weight, self.rope)
        if x.dtype != torch.bfloat16:
            raise SanaHipError("qk-norm / rotary embedding inside the kernels is bf16 only")
        if self.rinv is not None:
            if self.rinv.dtype != torch.float32 or tuple(self.rinv.shape) != (B, N) or not self.rinv.is_contiguous():
                raise SanaHipError(f"rinv must be contiguous fp32 {(B, N)}")
            if self.weight.dtype != torch.bfloat16 or self.weight.numel() != C or not self.weight.is_contiguous():
                raise SanaHipError(f"norm weight must be contiguous bf16 [{C}]")
        if self.rope is not None:
            if self.rope.dtype != torch.float32 or tuple(self.rope.shape) != (N, head_dim // 2, 2) or \
                    not self.rope.is_contiguous():
                raise SanaHipError(f"rope must be contiguous fp32 {(N, head_dim // 2, 2)}")
        ptr = lambda t: None if t is None else t.data_ptr()
        return ptr(self.rinv), ptr(self.weight), ptr(self.rope)


def qk_rms(q: torch.Tensor, k: torch.Tensor, eps: float) -> Tuple[torch.Tensor, torch.Tensor]:
    """Per-token rsqrt(mean_c x^2 + eps) of q and of k: [B, N, C] bf16 views with equal strides -> two fp32 [B, N]."""
    _need_cuda(q, k)
    same = all(a == b or n == 1 for a, b, n in zip(q.stride(), k.stride(), q.shape))
    if q.shape != k.shape or q.dtype != k.dtype or not same:
        raise SanaHipError("q and k must share shape, dtype and strides")
    B, N, C = q.shape
    sb, sn = _token_major_view(q, "q")
    rq = torch.empty(B, N, dtype=torch.float32, device=q.device)
    rk = torch.empty(B, N, dtype=torch.float32, device=q.device)
    if B * N == 0:
        return rq, rk
    code = _lib.load().sana_hip_qk_rms(q.data_ptr(), k.data_ptr(), rq.data_ptr(), rk.data_ptr(), B, N, C, sb, sn,
                                       float(eps), _dt(q), _stream())
    _lib.check(code, "sana_hip_qk_rms")
    return rq, rk


def rope_table(freqs: torch.Tensor, N: int, device, head_dim: int = HEAD_DIM) -> torch.Tensor:
    """Complex rotary factors [..., N, d/2] (any leading singleton dims, as the reference passes
    ``rotary_emb`` [1, 1, N, d/2]) -> fp32 (cos, sin) table [N, d/2, 2] on ``device``."""
    if not torch.is_complex(freqs):
        raise SanaHipError("rotary_emb must be a complex tensor of unit factors")
    f = freqs.reshape(-1, freqs.shape[-1])
    if tuple(f.shape) != (N, head_dim // 2):
        raise SanaHipError(f"rotary_emb must broadcast over batch and heads: expected [.., {N}, {head_dim // 2}], "
                           f"got {tuple(freqs.shape)}")
    return torch.view_as_real(f.to(torch.complex64)).to(device=device, dtype=torch.float32).contiguous()


def rope_table_real(cos: torch.Tensor, sin: torch.Tensor, N: int, device, head_dim: int = HEAD_DIM) -> Optional[torch.Tensor]:
    """The real-valued rotary tables ``LiteLA.forward`` receives -- ``(cos, sin)``, each [N, d], applied to the channel
    pairs (2i, 2i+1) of a head (sana_blocks.py:1572-1582) -- as the kernels' fp32 (cos, sin) table [N, d/2, 2], or None
    when the two entries of some pair differ (the reference's builders repeat every angle for its pair; a table
    that does not is not a rotation of the pair and has no kernel form)."""
    if cos.shape != sin.shape or cos.dim() != 2 or tuple(cos.shape) != (N, head_dim):
        raise SanaHipError(f"rotary_emb must be (cos, sin) of shape {(N, head_dim)}, got {tuple(cos.shape)} / {tuple(sin.shape)}")
    c, sn = cos.to(torch.float32), sin.to(torch.float32)
    if not (torch.equal(c[:, 0::2], c[:, 1::2]) and torch.equal(sn[:, 0::2], sn[:, 1::2])):
        return None
    return torch.stack([c[:, 0::2], sn[:, 0::2]], dim=-1).to(device=device).contiguous()


def _head_dim(d: int) -> int:
    if d not in HEAD_DIMS:
        raise SanaHipError(f"head_dim {d} has no kernel (supported: {HEAD_DIMS})")
    return d


NOALLOC_SCRATCH_BYTES = 32 << 20   # SANA_HIP_NOALLOC_SCRATCH_BYTES of include/sana_hip.h


def linattn_state(k: torch.Tensor, v: torch.Tensor, chunk_tokens=None, causal: bool = False,
                  pre: Optional[QkPre] = None, head_dim: int = HEAD_DIM, out: Optional[torch.Tensor] = None,
                  noalloc: bool = False) -> torch.Tensor:
    """Phase 1.  k, v: [B, N, C] token-major views (C = h*d).  Returns the fp32
    state [B, h, n_chunks, d+1, d] (inclusive prefix over chunks when causal).
    ``out``: a state tensor to fill instead of a new one.  ``noalloc``: the partial states go to the library's
    fixed per-GPU scratch array instead of a torch workspace (``sana_hip_linattn_state_noalloc``: with ``out``
    given, nothing is allocated; problems beyond NOALLOC_SCRATCH_BYTES raise)."""
    d = _head_dim(head_dim)
    _need_cuda(k, v, out)
    same = all(a == b or n == 1 for a, b, n in zip(k.stride(), v.stride(), k.shape))
    if k.shape != v.shape or k.dtype != v.dtype or not same:
        raise SanaHipError("k and v must share shape, dtype and strides")
    B, N, C = k.shape
    if C % d:
        raise SanaHipError(f"C={C} is not a multiple of head_dim {d}")
    h = C // d
    sb, sn = _token_major_view(k, "k")
    tab, n_chunks, longest = chunk_table(chunk_tokens, N, k.device)
    lib = _lib.load()
    if out is None:
        state = torch.empty(B, h, n_chunks, d + 1, d, dtype=torch.float32, device=k.device)
    else:
        state = out
        if state.dtype != torch.float32 or not state.is_contiguous() or tuple(state.shape) != (B, h, n_chunks, d + 1, d):
            raise SanaHipError(f"out must be contiguous fp32 {(B, h, n_chunks, d + 1, d)}")
    if B * N == 0:
        if pre is not None:
            pre.check(k, d)
        return state.zero_()
    shape = (B, N, h, d, sb, sn, tab.data_ptr() if tab is not None else None, n_chunks, longest,
             1 if causal else 0, _dt(k))
    pre_args = pre.check(k, d) if pre is not None else (None, None, None)
    if pre is not None and pre.rope_first:
        if n_chunks != 1 or noalloc:
            raise SanaHipError("the rotate-before-ReLU order (LiteLA.forward) is not chunk-causal and has no no-alloc form")
        nbytes = lib.sana_hip_linattn_workspace_bytes(B, h, d, 1, N, _dt(k))
        ws = _workspace(k.device, nbytes)
        code = lib.sana_hip_litela_state(k.data_ptr(), v.data_ptr(), state.data_ptr(),
                                         ws.data_ptr() if ws is not None else None, nbytes, B, N, h, d, sb, sn, _dt(k),
                                         *pre_args, _stream())
        _lib.check(code, "sana_hip_litela_state")
        return state
    if noalloc:
        code = lib.sana_hip_linattn_state_noalloc(k.data_ptr(), v.data_ptr(), state.data_ptr(), *shape, *pre_args,
                                                  _stream())
        _lib.check(code, "sana_hip_linattn_state_noalloc")
        return state
    nbytes = lib.sana_hip_linattn_workspace_bytes(B, h, d, n_chunks, longest, _dt(k))
    ws = _workspace(k.device, nbytes)
    args = (k.data_ptr(), v.data_ptr(), state.data_ptr(), ws.data_ptr() if ws is not None else None, nbytes, *shape)
    if pre is None:
        code = lib.sana_hip_linattn_state(*args, _stream())
    else:
        code = lib.sana_hip_linattn_state_pre(*args, *pre_args, _stream())
    _lib.check(code, "sana_hip_linattn_state")
    return state


def linattn_chunk_scan_(state: torch.Tensor) -> torch.Tensor:
    """In-place inclusive prefix sum over the chunk axis of [B, h, n_chunks, d+1, d] fp32."""
    _need_cuda(state)
    if state.dtype != torch.float32 or not state.is_contiguous() or state.dim() != 5 or \
            state.shape[3] != state.shape[4] + 1:
        raise SanaHipError("state must be contiguous fp32 [B, h, n_chunks, d+1, d]")
    B, h, n_chunks = state.shape[:3]
    d = _head_dim(state.shape[4])
    code = _lib.load().sana_hip_linattn_chunk_scan(state.data_ptr(), B, h, d, n_chunks, _stream())
    _lib.check(code, "sana_hip_linattn_chunk_scan")
    return state


def linattn_apply(q: torch.Tensor, state: torch.Tensor, eps: float, chunk_tokens=None,
                  out_dtype: Optional[torch.dtype] = None, out: Optional[torch.Tensor] = None,
                  pre: Optional[QkPre] = None) -> torch.Tensor:
    """Phase 2.  q: [B, N, C] token-major view; state from :func:`linattn_state`.
    Returns [B, N, C] in ``out_dtype`` (q's dtype or fp32)."""
    _need_cuda(q, state)
    B, N, C = q.shape
    d = _head_dim(state.shape[-1])
    h = C // d
    qsb, qsn = _token_major_view(q, "q")
    tab, n_chunks, longest = chunk_table(chunk_tokens, N, q.device)
    if state.dtype != torch.float32 or not state.is_contiguous() or \
            tuple(state.shape) != (B, h, n_chunks, d + 1, d):
        raise SanaHipError(f"state must be contiguous fp32 {(B, h, n_chunks, d + 1, d)}, "
                           f"got {tuple(state.shape)}")
    out_dtype = out_dtype or q.dtype
    if out is None:
        out = torch.empty(B, N, C, dtype=out_dtype, device=q.device)
    elif out.shape != q.shape or out.dtype != out_dtype:
        raise SanaHipError("out has the wrong shape or dtype")
    osb, osn = _token_major_view(out, "out")
    if B * N == 0:
        if pre is not None:
            pre.check(q, d)
        return out
    args = (q.data_ptr(), state.data_ptr(), out.data_ptr(), B, N, h, d, qsb, qsn, osb, osn,
            tab.data_ptr() if tab is not None else None, n_chunks, longest, float(eps), _dt(q), _DT[out_dtype])
    if pre is not None and pre.rope_first:
        if n_chunks != 1:
            raise SanaHipError("the rotate-before-ReLU order (LiteLA.forward) is not chunk-causal")
        code = _lib.load().sana_hip_litela_apply(q.data_ptr(), state.data_ptr(), out.data_ptr(), B, N, h, d, qsb, qsn,
                                                osb, osn, float(eps), _dt(q), _DT[out_dtype], *pre.check(q, d), _stream())
        _lib.check(code, "sana_hip_litela_apply")
        return out
    if pre is None:
        code = _lib.load().sana_hip_linattn_apply(*args, _stream())
    else:
        code = _lib.load().sana_hip_linattn_apply_pre(*args, *pre.check(q, d), _stream())
    _lib.check(code, "sana_hip_linattn_apply")
    return out


def relu_linear_attention(q, k, v, eps: float, chunk_tokens=None, out_dtype=None,
                          head_dim: int = HEAD_DIM) -> torch.Tensor:
    """Both phases on token-major [B, N, C] views; chunk-causal when ``chunk_tokens`` has > 1 entry."""
    causal = chunk_tokens is not None and len(chunk_tokens) > 1
    state = linattn_state(k, v, chunk_tokens, causal=causal, head_dim=head_dim)
    return linattn_apply(q, state, eps, chunk_tokens, out_dtype)


# --------------------------------------------------------------------------- Mix-FFN pieces

def dwconv3x3_silu_gate(u: torch.Tensor, weight: torch.Tensor, bias: Optional[torch.Tensor],
                        round_like_reference: bool = True) -> torch.Tensor:
    """u: [BT, H, W, 2*Ch] contiguous channels-last; weight: [2*Ch, 1, 3, 3] or [2*Ch, 3, 3];
    bias: [2*Ch] or None.  Returns [BT, H, W, Ch]."""
    _need_cuda(u, weight, bias)
    if u.dim() != 4 or not u.is_contiguous():
        raise SanaHipError("u must be a contiguous [BT, H, W, 2*Ch] tensor")
    BT, H, W, C2 = u.shape
    if C2 % 2 or weight.numel() != C2 * 9 or not weight.is_contiguous() or weight.dtype != u.dtype:
        raise SanaHipError("weight must be contiguous [2*Ch, 1, 3, 3] in u's dtype")
    if bias is not None and (bias.numel() != C2 or bias.dtype != u.dtype or not bias.is_contiguous()):
        raise SanaHipError("bias must be contiguous [2*Ch] in u's dtype")
    y = torch.empty(BT, H, W, C2 // 2, dtype=u.dtype, device=u.device)
    if y.numel() == 0:
        return y
    code = _lib.load().sana_hip_dwconv3x3_silu_gate(
        u.data_ptr(), weight.data_ptr(), bias.data_ptr() if bias is not None else None, y.data_ptr(),
        BT, H, W, C2 // 2, 1 if round_like_reference else 0, _dt(u), _stream())
    _lib.check(code, "sana_hip_dwconv3x3_silu_gate")
    return y


_EPI = {None: _lib.EPI_NONE, "none": _lib.EPI_NONE, "bias": _lib.EPI_BIAS, "bias_silu": _lib.EPI_BIAS_SILU}


def _rows(t: torch.Tensor, what: str) -> Tuple[torch.Tensor, int]:
    """2-d row-major view (unit inner stride) -> (tensor, leading stride)."""
    if t.dim() != 2 or t.stride(1) != 1:
        raise SanaHipError(f"{what} must be 2-d with unit inner stride, got {tuple(t.shape)} / {t.stride()}")
    return t, t.stride(0)


SPLIT_K = True   # False: never hand the GEMMs a workspace (they then run unsplit; used by tests)


def _gemm_workspace(lib, device, M: int, N: int, K: int) -> Tuple[Optional[int], int]:
    """(pointer, bytes) of the split-k workspace this shape wants, or (None, 0): shapes with few output tiles
    run as a split-k GEMM through fp32 partial planes in the per-device workspace."""
    nbytes = lib.sana_hip_gemm_workspace_bytes(M, N, K) if SPLIT_K else 0
    ws = _workspace(device, nbytes)
    return (ws.data_ptr(), nbytes) if ws is not None else (None, 0)


def gemm_bf16(a: torch.Tensor, weight: torch.Tensor, bias: Optional[torch.Tensor] = None,
              epilogue: Optional[str] = None, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """a: [M, K]; weight: [N, K] (nn.Linear layout); both bf16, or both fp16 (``sana_hip_gemm_f16``: the same
    kernels on the fp16 MFMA).  Returns epilogue(a @ weight.T) [M, N] in that dtype."""
    _need_cuda(a, weight, bias)
    dt = a.dtype
    if dt not in IO16 or weight.dtype != dt:
        raise SanaHipError(f"the GEMM needs bf16 or fp16 operands of one dtype, got {a.dtype} and {weight.dtype}")
    a, lda = _rows(a, "a")
    weight, ldw = _rows(weight, "weight")
    M, K = a.shape
    N = weight.shape[0]
    if weight.shape[1] != K:
        raise SanaHipError(f"K mismatch: a {tuple(a.shape)} vs weight {tuple(weight.shape)}")
    epi = _EPI[epilogue]
    if bias is not None and epi == _lib.EPI_NONE:
        epi = _lib.EPI_BIAS
    if bias is not None and (bias.dtype != dt or bias.numel() != N or not bias.is_contiguous()):
        raise SanaHipError(f"bias must be contiguous {dt} [N]")
    if out is None:
        out = torch.empty(M, N, dtype=dt, device=a.device)
    out, ldc = _rows(out, "out")
    if tuple(out.shape) != (M, N) or out.dtype != dt:
        raise SanaHipError("out has the wrong shape or dtype")
    if M == 0:
        return out
    lib = _lib.load()
    ws, nbytes = _gemm_workspace(lib, a.device, M, N, K)
    fn = lib.sana_hip_gemm_f16 if dt == torch.float16 else lib.sana_hip_gemm_bf16
    code = fn(a.data_ptr(), weight.data_ptr(), bias.data_ptr() if bias is not None else None,
                                  out.data_ptr(), M, N, K, lda, ldw, ldc, epi, ws, nbytes, _stream())
    _lib.check(code, "sana_hip_gemm_bf16")
    return out


# From this many rows on, an int8 weight is expanded to bf16 once per call (a streaming pass over N*K bytes) and
# the bf16 GEMM runs; below it the GEMM converts inside its main loop.  Both give the same bits; the conversion
# costs the main loop about 14 % at every M, the expansion a fixed 10-20 us.
W8_EXPAND_MIN_ROWS = 4096


def dequant_w8(wq: torch.Tensor, scale: torch.Tensor) -> torch.Tensor:
    """int8 [N, K] and fp32 [N] -> bf16 [N, K] = (wq.float() * scale[:, None]).bfloat16(), one kernel."""
    _need_cuda(wq, scale)
    if wq.dtype != torch.int8 or scale.dtype != torch.float32 or not scale.is_contiguous():
        raise SanaHipError("dequant_w8 needs int8 weights and contiguous fp32 scales")
    wq, ldw = _rows(wq, "wq")
    N, K = wq.shape
    if scale.numel() != N:
        raise SanaHipError("one scale per weight row")
    out = torch.empty(N, K, dtype=torch.bfloat16, device=wq.device)
    code = _lib.load().sana_hip_dequant_w8(wq.data_ptr(), scale.data_ptr(), out.data_ptr(), N, K, ldw, K, _stream())
    _lib.check(code, "sana_hip_dequant_w8")
    return out


def qkv_state_rows(C: int, heads: int) -> torch.Tensor:
    """Row map of the fused qkv projection's weight layout (``sana_hip_qkv_state_rows``): int64 [rows], entry i = the
    row of the [3C, C] qkv weight that row i of the tiled weight holds, -1 for a zero row.  Host code."""
    import ctypes
    lib = _lib.load()
    n = lib.sana_hip_qkv_state_rows(C, heads, None, 0)
    if n <= 0:
        raise SanaHipError(f"the fused qkv projection needs C == 32 * heads, got C={C}, heads={heads}")
    buf = (ctypes.c_int32 * n)()
    if lib.sana_hip_qkv_state_rows(C, heads, ctypes.cast(buf, ctypes.c_void_p), n) != n:
        raise SanaHipError("sana_hip_qkv_state_rows failed")
    return torch.tensor(list(buf), dtype=torch.int64)


def tile_qkv_rows(t: torch.Tensor, heads: int) -> torch.Tensor:
    """A per-output-channel tensor of the qkv projection ([3C, ...]: weight, int8 weight, bias, scales) in the fused
    GEMM's row layout ([rows, ...], zero where the layout has no source row)."""
    C = t.shape[0] // 3
    rows = qkv_state_rows(C, heads).to(t.device)
    live = rows >= 0
    out = torch.zeros(rows.numel(), *t.shape[1:], dtype=t.dtype, device=t.device)
    out[live] = t[rows[live]]
    return out


def tile_qkv_weight(weight: torch.Tensor, bias: Optional[torch.Tensor], heads: int):
    """(W_tiled, bias_tiled) for ``gemm_qkv_state`` from the reference's [3C, C] qkv weight and [3C] bias (or None)."""
    return tile_qkv_rows(weight, heads), None if bias is None else tile_qkv_rows(bias, heads)


def qkv_state_supported(n_tokens: int, C: int, heads: int, batch: int = 2, has_bias: bool = True) -> bool:
    """Shapes sana_hip_gemm_qkv_state takes: whole 256-token tiles per batch entry -- or one batch entry and no bias,
    where the ragged last tile's missing rows are zeros that add nothing to the state."""
    return heads > 0 and C == 32 * heads and C >= 64 and n_tokens > 0 and \
        (n_tokens % 256 == 0 or (batch == 1 and not has_bias))


def gemm_qkv_state(x: torch.Tensor, w_tiled: torch.Tensor, bias_tiled: Optional[torch.Tensor], heads: int):
    """qkv projection with phase 1 of the linear attention in its epilogue.  x: [B, N, C] bf16 (N % 256 == 0, or B == 1
    and no bias),
    w_tiled / bias_tiled: ``tile_qkv_weight``'s.  Returns (q [B, N, C] bf16, state [B, heads, 1, 33, 32] fp32)."""
    _need_cuda(x, w_tiled, bias_tiled)
    if x.dim() != 3 or x.dtype != torch.bfloat16 or w_tiled.dtype != torch.bfloat16:
        raise SanaHipError("gemm_qkv_state needs a bf16 [B, N, C] input and a bf16 tiled weight")
    B, N, C = x.shape
    if not qkv_state_supported(N, C, heads, B, bias_tiled is not None):
        raise SanaHipError(f"gemm_qkv_state needs C == 32 * heads and N % 256 == 0 (or one batch entry and no bias), "
                           f"got B={B}, N={N}, C={C}, heads={heads}, bias {'given' if bias_tiled is not None else 'absent'}")
    lib = _lib.load()
    if tuple(w_tiled.shape) != (lib.sana_hip_qkv_state_rows(C, heads, None, 0), C):
        raise SanaHipError(f"tiled weight of shape {tuple(w_tiled.shape)} does not fit C={C}, heads={heads}")
    if bias_tiled is not None and (bias_tiled.dtype != torch.bfloat16 or bias_tiled.numel() != w_tiled.shape[0]
                                   or not bias_tiled.is_contiguous()):
        raise SanaHipError("bias_tiled must be contiguous bf16 [rows]")
    a, lda = _rows(x.reshape(B * N, C), "x")
    w, ldw = _rows(w_tiled, "w_tiled")
    q = torch.empty(B, N, C, dtype=torch.bfloat16, device=x.device)
    state = torch.empty(B, heads, 1, 33, 32, dtype=torch.float32, device=x.device)
    nbytes = lib.sana_hip_gemm_qkv_state_workspace_bytes(B, N, heads)
    ws = _workspace(x.device, nbytes)
    code = lib.sana_hip_gemm_qkv_state(a.data_ptr(), w.data_ptr(), None if bias_tiled is None else bias_tiled.data_ptr(),
                                       q.data_ptr(), state.data_ptr(), ws.data_ptr(), nbytes, B, N, C, heads,
                                       lda, ldw, C, _stream())
    _lib.check(code, "sana_hip_gemm_qkv_state")
    return q, state


def gemm_w8a16(a: torch.Tensor, wq: torch.Tensor, scale: torch.Tensor, bias: Optional[torch.Tensor] = None,
               epilogue: Optional[str] = None, out: Optional[torch.Tensor] = None,
               expand: Optional[bool] = None) -> torch.Tensor:
    """a: [M, K] bf16; wq: [N, K] int8; scale: [N] fp32.  Equals gemm_bf16 on (wq.float()*scale).bfloat16().
    ``expand``: True = expand the weight to bf16 first, False = convert inside the GEMM, None = by M."""
    _need_cuda(a, wq, scale, bias)
    if a.dtype != torch.bfloat16 or wq.dtype != torch.int8 or scale.dtype != torch.float32:
        raise SanaHipError("gemm_w8a16 needs bf16 activations, int8 weights and fp32 scales")
    if expand or (expand is None and a.shape[0] >= W8_EXPAND_MIN_ROWS):
        return gemm_bf16(a, dequant_w8(wq, scale), bias, epilogue, out)
    a, lda = _rows(a, "a")
    wq, ldw = _rows(wq, "wq")
    M, K = a.shape
    N = wq.shape[0]
    if wq.shape[1] != K or scale.numel() != N or not scale.is_contiguous():
        raise SanaHipError("shape mismatch between a, wq and scale")
    epi = _EPI[epilogue]
    if bias is not None and epi == _lib.EPI_NONE:
        epi = _lib.EPI_BIAS
    if bias is not None and (bias.dtype != torch.bfloat16 or bias.numel() != N or not bias.is_contiguous()):
        raise SanaHipError("bias must be contiguous bf16 [N]")
    if out is None:
        out = torch.empty(M, N, dtype=torch.bfloat16, device=a.device)
    out, ldc = _rows(out, "out")
    if tuple(out.shape) != (M, N) or out.dtype != torch.bfloat16:
        raise SanaHipError("out has the wrong shape or dtype")
    if M == 0:
        return out
    lib = _lib.load()
    ws, nbytes = _gemm_workspace(lib, a.device, M, N, K)
    code = lib.sana_hip_gemm_w8a16(a.data_ptr(), wq.data_ptr(), scale.data_ptr(),
                                   bias.data_ptr() if bias is not None else None, out.data_ptr(),
                                   M, N, K, lda, ldw, ldc, epi, ws, nbytes, _stream())
    _lib.check(code, "sana_hip_gemm_w8a16")
    return out


# --------------------------------------------------------------------------- fused seams of the block

def _mod_rows(t: torch.Tensor, B: int, C: int, what: str, dtype) -> Tuple[torch.Tensor, int]:
    """Per-batch row vectors [B, 1, C] / [B, C] with unit inner stride -> (tensor, batch stride)."""
    if t.dtype != dtype:     # the kernels read these rows as 16-bit values: another dtype would be misread
        raise SanaHipError(f"{what} must be {dtype} like the activations, got {t.dtype}")
    if t.dim() == 3 and t.shape[1] == 1:
        t = t[:, 0]
    if t.dim() != 2 or t.shape != (B, C) or t.stride(1) != 1:
        raise SanaHipError(f"{what} must be [B, C] (or [B, 1, C]) with unit inner stride, got {tuple(t.shape)}")
    return t, (t.stride(0) if B > 1 else 0)


def gemm_gate_residual(a: torch.Tensor, weight: torch.Tensor, bias: Optional[torch.Tensor], gate: torch.Tensor,
                       residual: torch.Tensor, weight_scale: Optional[torch.Tensor] = None,
                       expand: Optional[bool] = None) -> torch.Tensor:
    """residual + gate * (a @ weight.T + bias) with a: [B, N, K], residual: [B, N, C], gate: [B, 1, C].
    weight is bf16 [C, K], or int8 with ``weight_scale`` (W8A16; ``expand`` as in :func:`gemm_w8a16`)."""
    _need_cuda(a, weight, bias, gate, residual, weight_scale)
    B, Ntok, K = a.shape
    if weight_scale is not None and (expand or (expand is None and B * Ntok >= W8_EXPAND_MIN_ROWS)):
        weight, weight_scale = dequant_w8(weight.reshape(weight.shape[0], -1), weight_scale), None
    C = weight.shape[0]
    dt = a.dtype
    if dt not in IO16 or residual.dtype != dt or gate.dtype != dt:
        raise SanaHipError("gemm_gate_residual needs bf16 or fp16 activations, gate and residual of one dtype")
    if weight_scale is not None and dt != torch.bfloat16:
        raise SanaHipError("W8A16 needs bf16 activations")
    if weight_scale is None and weight.dtype != dt:
        raise SanaHipError(f"weight must be {dt} (or int8 together with weight_scale), got {weight.dtype}")
    if weight_scale is not None and (weight.dtype != torch.int8 or weight_scale.dtype != torch.float32
                                     or weight_scale.numel() != C or not weight_scale.is_contiguous()):
        raise SanaHipError("W8A16 needs an int8 weight and contiguous fp32 scales, one per output channel")
    if bias is not None and (bias.dtype != dt or bias.numel() != C or not bias.is_contiguous()):
        raise SanaHipError(f"bias must be contiguous {dt} [C]")
    if weight.reshape(C, -1).shape[1] != K:
        raise SanaHipError(f"K mismatch: a {tuple(a.shape)} vs weight {tuple(weight.shape)}")
    a2, lda = _rows(a.reshape(B * Ntok, K), "a")
    w2, ldw = _rows(weight.reshape(C, -1), "weight")
    r2, ldr = _rows(residual.reshape(B * Ntok, C), "residual")
    g2, gstride = _mod_rows(gate, B, C, "gate", dt)
    out = torch.empty(B * Ntok, C, dtype=dt, device=a.device)
    if B * Ntok == 0:
        return out.view(B, Ntok, C)
    lib = _lib.load()
    ws, nbytes = _gemm_workspace(lib, a.device, B * Ntok, C, K)
    if dt == torch.float16:
        code = lib.sana_hip_gemm_gate_residual_f16(
            a2.data_ptr(), w2.data_ptr(), bias.data_ptr() if bias is not None else None, g2.data_ptr(), r2.data_ptr(),
            out.data_ptr(), B * Ntok, C, K, lda, ldw, ldr, C, Ntok, gstride, ws, nbytes, _stream())
        _lib.check(code, "sana_hip_gemm_gate_residual_f16")
        return out.view(B, Ntok, C)
    code = lib.sana_hip_gemm_gate_residual(
        a2.data_ptr(), w2.data_ptr(), weight_scale.data_ptr() if weight_scale is not None else None,
        bias.data_ptr() if bias is not None else None, g2.data_ptr(), r2.data_ptr(), out.data_ptr(),
        B * Ntok, C, K, lda, ldw, ldr, C, Ntok, gstride, ws, nbytes, _stream())
    _lib.check(code, "sana_hip_gemm_gate_residual")
    return out.view(B, Ntok, C)


_frame_flags = {}    # (device index, n_frames, tuple of flagged frames) -> uint8 tensor


def frame_flags(n_frames: int, flagged: Sequence[int], device) -> Optional[torch.Tensor]:
    """uint8 [n_frames] with ones at ``flagged`` (cached per device), or None when nothing is flagged."""
    flagged = tuple(sorted(set(int(f) for f in flagged)))
    if not flagged:
        return None
    if flagged[0] < 0 or flagged[-1] >= n_frames:
        raise SanaHipError(f"flagged frames {flagged} outside 0..{n_frames - 1}")
    def make():
        host = torch.zeros(n_frames, dtype=torch.uint8)
        host[list(flagged)] = 1
        return host.to(device)

    return _remember(_frame_flags, (torch.device(device).index, n_frames, flagged), make)


def tconv_residual(xp: torch.Tensor, weight: torch.Tensor, n_rows: int, tap_rows: int,
                   out: Optional[torch.Tensor] = None, zero_last_tap: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Temporal conv over frames plus its residual, as one GEMM over a virtual im2col.

    xp: [rows, C] bf16 (unit channel stride), the frame in front of the first output frame followed by the
    frames themselves (``rows >= n_rows + tap_rows``; rows past the end read as zero: the right padding);
    weight: [C, taps*C] bf16 with ``weight[o, t*C + i] = t_conv.weight[o, i, t, 0]``.  Returns
    ``out[m] = xp[m + (taps//2)*tap_rows] + sum_t weight[:, t*C:(t+1)*C] @ xp[m + t*tap_rows]``, m < n_rows.
    ``zero_last_tap``: uint8 [ceil(n_rows / tap_rows)] from :func:`frame_flags`; a flagged frame's last tap reads
    zeros (a chunk ends behind it), so all chunks of a sequence are one launch."""
    _need_cuda(xp, weight, out, zero_last_tap)
    if xp.dtype != torch.bfloat16 or weight.dtype != torch.bfloat16:
        raise SanaHipError("tconv_residual is bf16 only")
    x2, ldx = _rows(xp, "xp")
    w2, ldw = _rows(weight, "weight")
    rows, C = x2.shape
    if w2.shape[0] != C or w2.shape[1] % C:
        raise SanaHipError(f"weight must be [C, taps*C] with C={C}, got {tuple(w2.shape)}")
    taps = w2.shape[1] // C
    if out is None:
        out = torch.empty(n_rows, C, dtype=torch.bfloat16, device=xp.device)
    o2, ldo = _rows(out, "out")
    if tuple(o2.shape) != (n_rows, C) or o2.dtype != torch.bfloat16:
        raise SanaHipError("out has the wrong shape or dtype")
    if n_rows == 0:
        return out
    if zero_last_tap is not None and (zero_last_tap.dtype != torch.uint8 or not zero_last_tap.is_contiguous()
                                      or zero_last_tap.numel() < (n_rows + tap_rows - 1) // tap_rows):
        raise SanaHipError("zero_last_tap must be a contiguous uint8 tensor with one entry per frame")
    code = _lib.load().sana_hip_tconv_residual(x2.data_ptr(), w2.data_ptr(), o2.data_ptr(), n_rows, C, taps,
                                               tap_rows, rows,
                                               zero_last_tap.data_ptr() if zero_last_tap is not None else None,
                                               ldx, ldw, ldo, _stream())
    _lib.check(code, "sana_hip_tconv_residual")
    return out


def layernorm_modulate(x: torch.Tensor, scale: torch.Tensor, shift: torch.Tensor, eps: float = 1e-6) -> torch.Tensor:
    """LN(x) * (1 + scale) + shift over the last dim; x: [B, N, C] bf16, scale/shift: [B, 1, C]."""
    _need_cuda(x, scale, shift)
    B, Ntok, C = x.shape
    x2, ldx = _rows(x.reshape(B * Ntok, C), "x")
    sc, s1 = _mod_rows(scale, B, C, "scale", x.dtype)
    sh, s2 = _mod_rows(shift, B, C, "shift", x.dtype)
    if s1 != s2:
        raise SanaHipError("scale and shift must share their batch stride")
    out = torch.empty(B * Ntok, C, dtype=x.dtype, device=x.device)
    if B * Ntok == 0:
        return out.view(B, Ntok, C)
    code = _lib.load().sana_hip_layernorm_modulate(x2.data_ptr(), sc.data_ptr(), sh.data_ptr(), out.data_ptr(),
                                                   B * Ntok, C, ldx, C, Ntok, s1, float(eps), _dt(x), _stream())
    _lib.check(code, "sana_hip_layernorm_modulate")
    return out.view(B, Ntok, C)


def add_layernorm_modulate(x: torch.Tensor, y: torch.Tensor, scale: torch.Tensor, shift: torch.Tensor,
                           eps: float = 1e-6) -> Tuple[torch.Tensor, torch.Tensor]:
    """(x + y, LN(x + y) * (1 + scale) + shift) in one pass; x, y: [B, N, C] bf16, scale/shift: [B, 1, C]."""
    _need_cuda(x, y, scale, shift)
    if x.shape != y.shape or x.dtype != y.dtype:
        raise SanaHipError("x and y must share shape and dtype")
    B, Ntok, C = x.shape
    x2, ldx = _rows(x.reshape(B * Ntok, C), "x")
    y2, ldy = _rows(y.reshape(B * Ntok, C), "y")
    sc, s1 = _mod_rows(scale, B, C, "scale", x.dtype)
    sh, s2 = _mod_rows(shift, B, C, "shift", x.dtype)
    if s1 != s2:
        raise SanaHipError("scale and shift must share their batch stride")
    total = torch.empty(B * Ntok, C, dtype=x.dtype, device=x.device)
    out = torch.empty(B * Ntok, C, dtype=x.dtype, device=x.device)
    if B * Ntok == 0:
        return total.view(B, Ntok, C), out.view(B, Ntok, C)
    code = _lib.load().sana_hip_add_layernorm_modulate(
        x2.data_ptr(), y2.data_ptr(), sc.data_ptr(), sh.data_ptr(), total.data_ptr(), out.data_ptr(), B * Ntok, C,
        ldx, ldy, C, C, Ntok, s1, float(eps), _dt(x), _stream())
    _lib.check(code, "sana_hip_add_layernorm_modulate")
    return total.view(B, Ntok, C), out.view(B, Ntok, C)

CROSS_ATTN_MAX_KEYS = 320     # keys of one (batch, head) that fit LDS together with their values


def cross_attention_supported(head_dim: int, n_keys: int) -> bool:
    """Shapes sana_hip_cross_attention takes: one head's keys and values held in LDS."""
    return 64 < head_dim <= 112 and head_dim % 8 == 0 and 0 < n_keys <= CROSS_ATTN_MAX_KEYS


def cross_attention(q: torch.Tensor, kv: torch.Tensor, num_heads: int, key_bias: Optional[torch.Tensor] = None,
                    scale: Optional[float] = None, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """softmax(q k^T * scale + key_bias) v per head, bf16.  q: [B, N, C] (q_linear's output), kv: [B, Nk, 2C]
    (kv_linear's output: keys then values), key_bias: fp32 [B, Nk] added to every head's and query's scores
    (0 / -10000 for a padding mask) or None.  Returns [B, N, C], token-major like q."""
    _need_cuda(q, kv, key_bias)
    if q.dim() != 3 or kv.dim() != 3 or q.dtype != torch.bfloat16 or kv.dtype != torch.bfloat16:
        raise SanaHipError("cross_attention needs bf16 q [B, N, C] and kv [B, Nk, 2C]")
    B, N, C = q.shape
    Nk = kv.shape[1]
    if kv.shape[0] != B or kv.shape[2] != 2 * C or C % num_heads:
        raise SanaHipError(f"kv {tuple(kv.shape)} does not match q {tuple(q.shape)} with {num_heads} heads")
    d = C // num_heads
    if not cross_attention_supported(d, Nk):
        raise SanaHipError(f"cross_attention holds one head's keys in LDS: head_dim {d} (72 .. 112), {Nk} keys (<= 320)")
    if q.stride(2) != 1 or kv.stride(2) != 1 or q.stride(0) != N * q.stride(1) or kv.stride(0) != Nk * kv.stride(1):
        raise SanaHipError("cross_attention needs q and kv rows with unit inner stride, batch entries back to back")
    if key_bias is not None:
        if key_bias.dtype != torch.float32 or key_bias.shape != (B, Nk) or key_bias.stride(1) != 1:
            raise SanaHipError("key_bias must be fp32 [B, Nk] with unit inner stride")
    if out is None:
        out = torch.empty(B, N, C, dtype=torch.bfloat16, device=q.device)
    elif out.shape != (B, N, C) or out.dtype != torch.bfloat16 or not out.is_contiguous():
        raise SanaHipError("out must be a contiguous bf16 [B, N, C] tensor")
    if B * N == 0:
        return out
    code = _lib.load().sana_hip_cross_attention(
        q.data_ptr(), kv.data_ptr(), None if key_bias is None else key_bias.data_ptr(), out.data_ptr(), B, N, Nk,
        num_heads, d, q.stride(1), kv.stride(1), C, 0 if key_bias is None else key_bias.stride(0),
        float(d ** -0.5 if scale is None else scale), _stream())
    _lib.check(code, "sana_hip_cross_attention")
    return out


def gate_residual(y: torch.Tensor, gate: torch.Tensor, residual: torch.Tensor) -> torch.Tensor:
    """residual + gate * y in one pass with the stock op pair's two roundings; y, residual: [B, N, C] bf16;
    gate: [B, 1, C], or one row per group of consecutive tokens, [B, G, 1, C]."""
    _need_cuda(y, gate, residual)
    if y.shape != residual.shape or y.dtype not in IO16 or residual.dtype != y.dtype or gate.dtype != y.dtype:
        raise SanaHipError("gate_residual needs bf16 or fp16 y, residual (of one shape) and gate of one dtype")
    B, Ntok, C = y.shape
    groups = gate.numel() // max(B * C, 1)
    if groups < 1 or gate.numel() != B * groups * C or Ntok % groups:
        raise SanaHipError(f"gate {tuple(gate.shape)} does not divide the {Ntok} tokens of {B} batch entries")
    y2, ldy = _rows(y.reshape(B * Ntok, C), "y")
    r2, ldr = _rows(residual.reshape(B * Ntok, C), "residual")
    g2, gstride = _mod_rows(gate.reshape(B * groups, 1, C), B * groups, C, "gate", y.dtype)
    out = torch.empty(B * Ntok, C, dtype=y.dtype, device=y.device)
    if B * Ntok == 0:
        return out.view(B, Ntok, C)
    code = _lib.load().sana_hip_gate_residual(y2.data_ptr(), g2.data_ptr(), r2.data_ptr(), out.data_ptr(), B * Ntok, C,
                                              ldy, ldr, C, Ntok // groups, gstride, _dt(y), _stream())
    _lib.check(code, "sana_hip_gate_residual")
    return out.view(B, Ntok, C)
