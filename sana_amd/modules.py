"""Drop-in modules for the SanaMSBlock hot path over the gfx950 kernels.

Same constructor arguments, forward signatures, attribute names and
``state_dict`` keys as the reference classes they stand in for:

  ``LiteLA``               diffusion/model/nets/sana_blocks.py:211-301
  ``ChunkCausalAttention`` diffusion/model/nets/sana_blocks.py:391-495 (no-RoPE form)
  ``GLUMBConv``            diffusion/model/nets/basic_modules.py:111-199
  ``SanaMSBlock``          diffusion/model/nets/sana_multi_scale.py:54-157

Forward only (inference).  The modules run on a GPU through ``libsana_hip.so``;
there is no CPU path: a configuration the kernels do not cover raises
``NotImplementedError`` at construction or call time.  Cross-attention is stock
PyTorch-ROCm ops by design.  A few options keep the HIP attention / depthwise
kernels but take a stock op for one stage (fp32 models: library GEMM for the
linears; the real-valued pre-ReLU rotary embedding of ``LiteLA``; the temporal
conv with a frame mask, C % 64 != 0 or a dtype other than bf16; the unfused
LayerNorm / modulate / gate / residual seams outside bf16 / fp16 inference).  Each of
those logs one line per process and reason on the ``sana_amd`` logger
(:func:`stock_path`), so nothing leaves the fast path silently.
"""
from __future__ import annotations

import collections
import logging
from typing import List, Optional, Sequence, Tuple

import torch
import torch.nn.functional as F
from torch import nn

from . import ops
from ._lib import SanaHipError

HEAD_DIM = ops.HEAD_DIM

log = logging.getLogger("sana_amd")
_stock_paths_seen = set()


def stock_path(where: str, why: str) -> None:
    """Record that ``where`` runs a stock PyTorch op instead of a kernel of this library because of ``why``:
    one warning per (where, why) and process."""
    key = (where, why)
    if key not in _stock_paths_seen:
        _stock_paths_seen.add(key)
        log.warning("sana_amd: %s runs on stock PyTorch ops: %s", where, why)



def _version(t: torch.Tensor):
    """The tensor's in-place version counter, or None for a tensor created under ``torch.inference_mode()``
    (such tensors do not track one and reading it raises; an in-place edit of one is then not noticed by the
    caches of derived data below, which key on it)."""
    return None if t.is_inference() else t._version


def _sources_unchanged(entry, tensors) -> bool:
    """``entry`` = (source tensors, their versions) of a derived-data cache: true when ``tensors`` are the very
    same objects (not merely tensors at the same address: the allocator hands a freed address to the next
    parameter) with unchanged version counters."""
    if entry is None or len(entry[0]) != len(tensors):
        return False
    return all(a is b for a, b in zip(entry[0], tensors)) and entry[1] == tuple(
        None if t is None else _version(t) for t in tensors)


def _source_entry(tensors):
    return (tuple(tensors), tuple(None if t is None else _version(t) for t in tensors))


def _no_grad_only(*tensors):
    if torch.is_grad_enabled() and any(t is not None and t.requires_grad for t in tensors):
        raise SanaHipError("the HIP path is forward-only: call it under torch.no_grad() / inference_mode()")


# ------------------------------------------------------------------ linear layers


class HipLinear(nn.Linear):
    """``nn.Linear`` whose bf16 / fp16 GPU forward is the hand-written MFMA GEMM.

    Keys ``weight`` / ``bias`` as in ``nn.Linear``.  After :meth:`quantize_w8_`
    the bf16 weight is dropped and replaced by ``weight_q`` (int8 [out, in]) and
    ``weight_scale`` (fp32 [out]); the forward then runs the W8A16 GEMM.
    fp32 models use the stock library GEMM.
    """

    def quantize_w8_(self) -> "HipLinear":
        wq, scale = quantize_w8(self.weight.data)
        self.register_buffer("weight_q", wq.contiguous())
        self.register_buffer("weight_scale", scale.contiguous())
        self.weight = None
        return self

    @property
    def is_quantized(self) -> bool:
        return getattr(self, "weight_q", None) is not None

    def forward(self, x: torch.Tensor, epilogue: Optional[str] = None, gate=None, residual=None) -> torch.Tensor:
        return hip_linear(x, self.weight, self.bias, epilogue,
                          getattr(self, "weight_q", None), getattr(self, "weight_scale", None), gate, residual)


def hip_linear(x, weight, bias, epilogue=None, weight_q=None, weight_scale=None, gate=None, residual=None, out=None):
    """y = epilogue(x @ W^T + b) over the last dim of x.  epilogue: None | "silu".
    With ``gate`` [B, 1, C] and ``residual`` [B, N, C]: residual + gate * y (one fused kernel in bf16).
    ``out``: a [rows, C_out] bf16 view to write into (bf16 GEMM without gate only)."""
    _no_grad_only(x, weight, bias)
    lead = x.shape[:-1]
    K = x.shape[-1]
    if gate is not None:
        if x.dtype in ops.IO16 and gate.dtype == x.dtype and residual.dtype == x.dtype and x.is_cuda \
                and x.dim() == 3 and epilogue is None and (weight_q is None or x.dtype == torch.bfloat16):
            w = weight_q if weight_q is not None else weight
            return ops.gemm_gate_residual(x, w, bias, gate, residual, weight_scale if weight_q is not None else None)
        stock_path("gated residual behind a linear", f"the fused epilogue needs bf16 / fp16 [B, N, C] device input, gate and "
                   f"residual and no activation; got x {x.dtype} {x.dim()}-d, gate {gate.dtype}, residual "
                   f"{residual.dtype}, epilogue {epilogue!r}")
        return residual + gate * hip_linear(x, weight, bias, epilogue, weight_q, weight_scale)
    if x.dtype in ops.IO16 and x.is_cuda and (weight_q is not None or weight.dtype == x.dtype):
        x2 = x.reshape(-1, K)
        if x2.stride(1) != 1 or x2.stride(0) % 8 or x2.data_ptr() % 16:
            x2 = x2.contiguous()
        epi = {None: "bias" if bias is not None else None, "silu": "bias_silu"}[epilogue]
        if epilogue == "silu" and bias is None:
            bias = torch.zeros(weight_q.shape[0] if weight_q is not None else weight.shape[0],
                               dtype=x.dtype, device=x.device)
        if weight_q is not None:
            if x.dtype != torch.bfloat16:
                raise SanaHipError("W8A16 needs bf16 activations")
            y = ops.gemm_w8a16(x2, weight_q, weight_scale, bias, epi, out=out)
        else:
            y = ops.gemm_bf16(x2, weight.reshape(weight.shape[0], -1), bias, epi, out=out)
        return y.view(*lead, y.shape[-1])
    if not x.is_cuda:
        raise SanaHipError("the HIP path needs device tensors (no CPU path exists)")
    if weight_q is not None:
        raise SanaHipError("W8A16 needs bf16 activations")
    # fp32 models (or activations and weights of different dtypes): plain library GEMM, activation as a stock op
    stock_path("linear / 1x1 conv", f"the hand-written GEMM takes bf16 or fp16 operands of one dtype, got input {x.dtype} "
               f"and weight {weight.dtype} (library GEMM instead)")
    y = F.linear(x, weight.reshape(weight.shape[0], -1), bias)
    return F.silu(y) if epilogue == "silu" else y


def quantize_w8(weight: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor]:
    """Symmetric per-output-channel int8 quantiser of the W8A16 configuration:
    s_o = absmax_i |W[o, i]| / 127 (fp32), Wq = clamp(round(W / s), -127, 127).
    Returns (int8 [out, in], fp32 [out]).  Not part of the reference (it has no
    W8A16 code); the dequantised weight is (Wq.float() * s).bfloat16()."""
    # fp64 intermediates make the result independent of the device's fp32 division
    w = weight.detach().double().flatten(1)
    scale = (w.abs().amax(dim=1) / 127.0).float()
    scale = torch.where(scale > 0, scale, torch.ones_like(scale))
    wq = torch.clamp(torch.round(w / scale.double()[:, None]), -127, 127).to(torch.int8)
    return wq, scale


# ------------------------------------------------------------------ linear attention


class RMSNorm(nn.Module):
    """diffusion/model/norms.py:182-231 (stock ops; only used with qk_norm=True)."""

    def __init__(self, dim: int, scale_factor: float = 1.0, eps: float = 1e-6):
        super().__init__()
        self.eps = eps
        self.weight = nn.Parameter(torch.ones(dim) * scale_factor)

    def forward(self, x):
        xf = x.float()
        return (self.weight * (xf * torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + self.eps))).type_as(x)


def _rotary_real_tokens_(t: torch.Tensor, cos_sin) -> None:
    """In-place real-valued RoPE on a token-major [B, N, C] view: the
    ``use_real_unbind_dim=-2`` form LiteLA.forward uses (sana_blocks.py:282-284,
    1572-1582).  cos, sin: [N, d] with d = head_dim; pairs are channels (2m, 2m+1)."""
    cos, sin = cos_sin
    B, N, C = t.shape
    d = cos.shape[-1]
    x = t.reshape(B, N, C // d, d)
    cos = cos.to(t.device)[None, :, None, :]
    sin = sin.to(t.device)[None, :, None, :]
    xr, xi = x.reshape(B, N, C // d, d // 2, 2).unbind(-1)
    x_rot = torch.stack([-xi, xr], dim=-1).reshape(B, N, C // d, d)
    t.copy_((x.float() * cos + x_rot.float() * sin).to(t.dtype).reshape(B, N, C))


# (cos, sin) tables derived from the callers' rotary_emb tensors, shared by all blocks of a model.  An entry keeps
# its source tensor alive, so neither the tensor's id nor its storage address can be handed to another tensor while
# the entry exists; the key names the memory the factors were read from and its version counter, so fresh views of
# the same factors (a pipeline slicing one table per chunk, once per block) hit, and equal-shaped temporaries with
# other contents miss.  Entries used while a HIP graph was being captured are never dropped: the graph holds the
# table's address.
_ROPE_TABLES: "collections.OrderedDict" = collections.OrderedDict()
_ROPE_TABLE_LIMIT = 16


def _rope_table_cached(rotary_emb: torch.Tensor, N: int, device, head_dim: int) -> torch.Tensor:
    key = (rotary_emb.untyped_storage().data_ptr(), rotary_emb.storage_offset(), tuple(rotary_emb.shape),
           tuple(rotary_emb.stride()), rotary_emb.dtype, rotary_emb.device, _version(rotary_emb), N,
           torch.device(device), head_dim)
    capturing = rotary_emb.is_cuda and torch.cuda.is_current_stream_capturing()
    entry = _ROPE_TABLES.get(key)
    if entry is None:
        entry = [rotary_emb, ops.rope_table(rotary_emb, N, device, head_dim=head_dim), capturing]
        _ROPE_TABLES[key] = entry
        if len(_ROPE_TABLES) > _ROPE_TABLE_LIMIT:
            for old in [k for k, e in _ROPE_TABLES.items() if not e[2]][:len(_ROPE_TABLES) - _ROPE_TABLE_LIMIT]:
                del _ROPE_TABLES[old]
    else:
        _ROPE_TABLES.move_to_end(key)
        entry[2] = entry[2] or capturing
    return entry[1]


def _rope_real_table_cached(rotary_emb, N: int, device, head_dim: int):
    """:func:`ops.rope_table_real` of a ``(cos, sin)`` pair through the same cache as the complex tables (an entry
    may be None: a table whose pair entries differ is checked once, not on every call)."""
    cos, sin = rotary_emb
    key = ("real",) + tuple((t.untyped_storage().data_ptr(), t.storage_offset(), tuple(t.shape), tuple(t.stride()),
                            t.dtype, t.device, _version(t)) for t in (cos, sin)) + (N, torch.device(device), head_dim)
    capturing = torch.cuda.is_available() and torch.cuda.is_current_stream_capturing()
    entry = _ROPE_TABLES.get(key)
    if entry is None:
        entry = [(cos, sin), ops.rope_table_real(cos, sin, N, device, head_dim), capturing]
        _ROPE_TABLES[key] = entry
        if len(_ROPE_TABLES) > _ROPE_TABLE_LIMIT:
            for old in [k for k, e in _ROPE_TABLES.items() if not e[2]][:len(_ROPE_TABLES) - _ROPE_TABLE_LIMIT]:
                del _ROPE_TABLES[old]
    else:
        _ROPE_TABLES.move_to_end(key)
        entry[2] = entry[2] or capturing
    return entry[1]


def _as_token_major(t: torch.Tensor, token_dim: int) -> torch.Tensor:
    """(B, h, d, N) [token_dim=3] or (B, h, N, d) [token_dim=2] -> [B, N, h*d] with
    unit channel stride, without a copy when the memory already is token-major."""
    B, h = t.shape[0], t.shape[1]
    tm = t.permute(0, 3, 1, 2) if token_dim == 3 else t.permute(0, 2, 1, 3)  # (B, N, h, d)
    N, d = tm.shape[1], tm.shape[3]
    if tm.stride(3) == 1 and tm.stride(2) == d and tm.stride(1) % 8 == 0 and tm.data_ptr() % 16 == 0:
        return tm.as_strided((B, N, h * d), (tm.stride(0), tm.stride(1), 1))
    return tm.reshape(B, N, h * d).contiguous()


class LiteLA(nn.Module):
    """ReLU linear attention (reference: sana_blocks.py:211-301).

    ``qkv`` / ``proj`` carry the parameters the reference inherits from timm's
    ``Attention`` base; ``q_norm`` / ``k_norm`` are Identity or RMSNorm over the
    full channel dim.  The attention core always accumulates in fp32 (the
    reference's ``fp32_attention`` mode); the attribute is accepted and ignored.
    """

    PAD_VAL = 1

    def __init__(self, in_dim: int, out_dim: int, heads: Optional[int] = None, heads_ratio: float = 1.0,
                 dim: int = 32, eps: float = 1e-15, use_bias: bool = False, qk_norm: bool = False,
                 norm_eps: float = 1e-5):
        super().__init__()
        heads = heads or int(out_dim // dim * heads_ratio)
        if in_dim != out_dim:
            raise NotImplementedError("LiteLA: in_dim != out_dim is not used by any Sana block")
        self.in_dim, self.out_dim, self.heads = in_dim, out_dim, heads
        self.dim = out_dim // heads
        if self.dim not in ops.HEAD_DIMS:
            raise NotImplementedError(f"the gfx950 attention kernels are built for head_dim {ops.HEAD_DIMS}, "
                                      f"got {self.dim}")
        self.eps = eps
        self.num_heads = heads
        self.scale = self.dim ** -0.5
        self.qkv = HipLinear(in_dim, in_dim * 3, bias=use_bias)
        self.attn_drop = nn.Dropout(0.0)
        self.proj = HipLinear(in_dim, in_dim)
        self.proj_drop = nn.Dropout(0.0)
        self.kernel_func = nn.ReLU(inplace=False)
        if qk_norm:
            self.q_norm = RMSNorm(in_dim, 1.0, norm_eps)
            self.k_norm = RMSNorm(in_dim, 1.0, norm_eps)
        else:
            self.q_norm = nn.Identity()
            self.k_norm = nn.Identity()

    # -- second public entry point of the reference (used by the PAG processors,
    #    sana_blocks.py:588-620): q, v (B, h, d, N); k (B, h, N, d); returns fp32 (B, h, d, N)
    def attn_matmul(self, q: torch.Tensor, k: torch.Tensor, v: torch.Tensor) -> torch.Tensor:
        _no_grad_only(q, k, v)
        B, h, d, N = q.shape
        qt = _as_token_major(q, 3)
        kt = _as_token_major(k, 2)
        vt = _as_token_major(v, 3)
        if any(a != b and n > 1 for a, b, n in zip(kt.stride(), vt.stride(), kt.shape)):
            kt, vt = kt.contiguous(), vt.contiguous()
        out = ops.relu_linear_attention(qt, kt, vt, self.eps, out_dtype=torch.float32, head_dim=d)  # ReLU in-kernel
        return out.view(B, N, h, d).permute(0, 2, 3, 1)

    def _qkv_tokens(self, x: torch.Tensor, rotary_emb=None) -> torch.Tensor:
        """qkv GEMM, optional qk-norm and RoPE -> fused [B, N, 3, C] buffer."""
        B, N, C = x.shape
        qkv = self.qkv(x).view(B, N, 3, C)
        if not isinstance(self.q_norm, nn.Identity):
            stock_path("LiteLA q/k RMSNorm", "in-kernel norm is the bf16 path without image_rotary_emb; "
                       f"got {x.dtype}, rotary_emb {'given' if rotary_emb is not None else 'absent'}")
            qkv[:, :, 0].copy_(self.q_norm(qkv[:, :, 0]))
            qkv[:, :, 1].copy_(self.k_norm(qkv[:, :, 1]))
        if rotary_emb is not None:
            stock_path("LiteLA rotary embedding", "the real-valued pre-ReLU rotation of LiteLA.forward "
                       "(sana_blocks.py:282-284) runs inside the kernels for bf16, head_dim 32 and (cos, sin) tables whose "
                       "two entries per channel pair are equal; applied in place on the qkv buffer otherwise")
            _rotary_real_tokens_(qkv[:, :, 0], rotary_emb)
            _rotary_real_tokens_(qkv[:, :, 1], rotary_emb)
        return qkv

    def forward(self, x: torch.Tensor, mask=None, HW=None, rotary_emb=None, block_id=None,
                block_mask=None) -> torch.Tensor:
        return self.forward_gated(x, None, None, rotary_emb=rotary_emb)

    def forward_gated(self, x, gate, residual, rotary_emb=None, **kwargs) -> torch.Tensor:
        """forward(x), or residual + gate * forward(x) with the update fused into the proj GEMM."""
        _no_grad_only(x)
        if rotary_emb is None and x.dtype == torch.bfloat16 and self._state_in_qkv_gemm(x):
            # k and v never reach memory: their column tiles are contracted over the tokens in the qkv GEMM's epilogue
            wt, bt = self._tiled_qkv()
            if self.qkv.is_quantized:       # int8 weights: expanded to bf16 per call, as the plain GEMM does from 4096 rows
                wt = ops.dequant_w8(*wt)
            q, state = ops.gemm_qkv_state(x, wt, bt, self.heads)
            out = ops.linattn_apply(q, state, self.eps)
        elif rotary_emb is None and x.dtype == torch.bfloat16:   # qk-norm (if any) on load inside the kernels
            B, N, C = x.shape
            out = self._attend(self.qkv(x).view(B, N, 3, C), None)
        elif x.dtype == torch.bfloat16 and x.is_cuda and self.dim == 32 and \
                (table := _rope_real_table_cached(rotary_emb, x.shape[1], x.device, self.dim)) is not None:
            # LiteLA.forward's own order (sana_blocks.py:274-286): norm, rotation BEFORE the ReLU, everything rotated --
            # applied on load inside the two attention kernels, nothing written back to the qkv buffer
            B, N, C = x.shape
            qkv = self.qkv(x).view(B, N, 3, C)
            pre_q, pre_k = self._pre(qkv, None)
            pre_q = ops.QkPre(pre_q.rinv if pre_q else None, pre_q.weight if pre_q else None, table, rope_first=True)
            pre_k = ops.QkPre(pre_k.rinv if pre_k else None, pre_k.weight if pre_k else None, table, rope_first=True)
            state = ops.linattn_state(qkv[:, :, 1], qkv[:, :, 2], pre=pre_k, head_dim=self.dim)
            out = ops.linattn_apply(qkv[:, :, 0], state, self.eps, pre=pre_q)
        else:
            qkv = self._qkv_tokens(x, rotary_emb)
            out = ops.relu_linear_attention(qkv[:, :, 0], qkv[:, :, 1], qkv[:, :, 2], self.eps, head_dim=self.dim)
        return self._proj_gated(out, gate, residual)

    # rows from which the qkv projection and phase 1 of the attention run as one GEMM (below it the 192-wide tiles
    # of the plain GEMM fill the chip better than the fused kernel's 256-wide ones, and phase 1 is a few us)
    STATE_IN_QKV_GEMM_MIN_ROWS = 4096

    def _state_in_qkv_gemm(self, x) -> bool:
        B, N, C = x.shape
        return (x.is_cuda and self.dim == 32 and B * N >= self.STATE_IN_QKV_GEMM_MIN_ROWS
                and isinstance(self.q_norm, nn.Identity) and isinstance(self.k_norm, nn.Identity)
                and (self.qkv.is_quantized or self.qkv.weight.dtype == torch.bfloat16)
                and ops.qkv_state_supported(N, C, self.heads, B, self.qkv.bias is not None))

    def _tiled_qkv(self):
        """The qkv weight (and bias) in the fused GEMM's row layout: derived data, rebuilt when the parameters
        change, not part of the state_dict."""
        quant = self.qkv.is_quantized
        ps = (self.qkv.weight_q, self.qkv.weight_scale, self.qkv.bias) if quant else (self.qkv.weight, self.qkv.bias)
        cache = self.__dict__.get("_tiled_cache")
        if cache is None or not _sources_unchanged(cache[0], ps):
            with torch.no_grad():
                tiled = [None if p is None else ops.tile_qkv_rows(p.detach(), self.heads) for p in ps]
            # (weight, bias), the weight being the pair (int8 weight, scales) of a quantised projection
            cache = (_source_entry(ps), ((tiled[0], tiled[1]), tiled[2]) if quant else (tiled[0], tiled[1]))
            self.__dict__["_tiled_cache"] = cache
        return cache[1]

    def _proj_gated(self, out, gate, residual):
        """proj(out), or residual + gate * proj(out) in the GEMM epilogue; gate is [B, 1, C] or one row per
        group of consecutive tokens, [B, G, 1, C] (per-frame conditioning)."""
        if gate is None:
            return self.proj(out)
        B, N, C = out.shape
        groups = gate.numel() // (B * gate.shape[-1])
        if groups == 1:
            return self.proj(out, gate=gate.reshape(B, 1, -1), residual=residual)
        y = self.proj(out.view(B * groups, N // groups, C), gate=gate.reshape(B * groups, 1, -1),
                      residual=residual.reshape(B * groups, N // groups, -1))
        return y.view(B, N, -1)

    def _pre(self, qkv: torch.Tensor, rotary_emb):
        """(QkPre for q, QkPre for k) for a fused [B, N, 3, C] buffer, or (None, None)."""
        B, N = qkv.shape[:2]
        norm = not isinstance(self.q_norm, nn.Identity)
        if not norm and rotary_emb is None:
            return None, None
        if qkv.dtype != torch.bfloat16:
            raise NotImplementedError("qk-norm / rotary embedding inside the attention kernels is bf16 only")
        rope = None
        if rotary_emb is not None:
            rope = _rope_table_cached(rotary_emb, N, qkv.device, self.dim)
        if norm:
            if self.q_norm.eps != self.k_norm.eps:
                raise NotImplementedError("q_norm and k_norm with different eps")
            rq, rk = ops.qk_rms(qkv[:, :, 0], qkv[:, :, 1], self.q_norm.eps)
            wq = self.q_norm.weight.detach().to(torch.bfloat16).contiguous()
            wk = self.k_norm.weight.detach().to(torch.bfloat16).contiguous()
            return ops.QkPre(rq, wq, rope), ops.QkPre(rk, wk, rope)
        return ops.QkPre(rope=rope), ops.QkPre(rope=rope)

    def _attend(self, qkv, rotary_emb, chunk_tokens=None):
        pre_q, pre_k = self._pre(qkv, rotary_emb)
        causal = chunk_tokens is not None and len(chunk_tokens) > 1
        state = ops.linattn_state(qkv[:, :, 1], qkv[:, :, 2], chunk_tokens, causal=causal, pre=pre_k,
                                  head_dim=self.dim)
        return ops.linattn_apply(qkv[:, :, 0], state, self.eps, chunk_tokens, pre=pre_q)


    def quantize_w8_(self) -> "LiteLA":
        self.qkv.quantize_w8_()
        self.proj.quantize_w8_()
        return self

    def __repr__(self):
        return f"EPS{self.eps}-" + super().__repr__()


class LiteLAReLURope(LiteLA):
    """ReLU linear attention with the rotary embedding applied AFTER the ReLU and to the
    numerator only (reference: sana_blocks.py:304-388): ``vk = v @ rope(relu(k))^T``,
    ``out = vk @ rope(relu(q))``, ``z = 1 / (sum_n relu(k_n) . relu(q) + eps)``.
    ``rotary_emb`` is the complex factor tensor [1, 1, N, d/2] the reference passes
    (``None`` = the unit rotation).  RMSNorm of q / k, the ReLU and the rotation all happen
    on load inside the two attention kernels (bf16); nothing is written back to the qkv buffer."""

    def forward(self, x: torch.Tensor, mask=None, HW=None, rotary_emb=None, block_mask=None, **kwargs) -> torch.Tensor:
        return self.forward_gated(x, None, None, rotary_emb=rotary_emb)

    def forward_gated(self, x, gate, residual, rotary_emb=None, **kwargs) -> torch.Tensor:
        _no_grad_only(x)
        B, N, C = x.shape
        qkv = self.qkv(x).view(B, N, 3, C)
        return self._proj_gated(self._attend(qkv, rotary_emb), gate, residual)


class ChunkCausalAttention(LiteLAReLURope):
    """Chunk-causal ReLU linear attention (reference: sana_blocks.py:391-495):
    every chunk of whole frames attends to the running sum of the states of all
    earlier chunks plus its own.  ``HW = (frames, h, w)``; ``chunk_index`` lists
    the first frame of each chunk; ``rotary_emb`` as in :class:`LiteLAReLURope`."""

    def forward(self, x: torch.Tensor, mask=None, HW=None, rotary_emb=None, block_mask=None,
                chunk_index: Optional[List[int]] = None) -> torch.Tensor:
        return self.forward_gated(x, None, None, HW=HW, rotary_emb=rotary_emb, chunk_index=chunk_index)

    def forward_gated(self, x, gate, residual, HW=None, rotary_emb=None, chunk_index=None, **kwargs) -> torch.Tensor:
        _no_grad_only(x)
        if HW is None or len(HW) != 3:
            raise ValueError("ChunkCausalAttention needs HW = (frames, h, w)")
        f, hh, ww = HW
        B, N, C = x.shape
        if f * hh * ww != N:
            raise ValueError(f"HW={HW} does not match N={N}")
        starts = list(chunk_index) if chunk_index is not None else [0]
        qkv = self.qkv(x).view(B, N, 3, C)
        out = self._attend(qkv, rotary_emb, chunk_tokens=[s * hh * ww for s in starts])
        return self._proj_gated(out, gate, residual)


class CachedCausalAttention(LiteLAReLURope):
    """Streaming form of the chunk-causal attention (reference: sana_blocks.py:498-572): the call
    sees one chunk, computes that chunk's own state, optionally saves it UN-accumulated into
    ``kv_cache[0:2]`` (``vk`` [B, h, d, d] and ``k_sum`` [B, h, 1, d], here fp32), adds the
    accumulated past the caller supplies in the same two slots, and returns ``(out, kv_cache)``.
    The caller accumulates saved states across chunks (:func:`accumulate_kv_cache`, the host-side
    loop of diffusion/longsana/pipeline/sana_inference_pipeline.py:242-263)."""

    def forward(self, x: torch.Tensor, mask=None, HW=None, rotary_emb=None, block_mask=None,
                save_kv_cache: bool = False, kv_cache: Optional[list] = None, **kwargs):
        return self.forward_gated(x, None, None, rotary_emb=rotary_emb, save_kv_cache=save_kv_cache, kv_cache=kv_cache)

    def forward_gated(self, x, gate, residual, rotary_emb=None, save_kv_cache: bool = False,
                      kv_cache: Optional[list] = None, **kwargs):
        _no_grad_only(x)
        B, N, C = x.shape
        qkv = self.qkv(x).view(B, N, 3, C)
        pre_q, pre_k = self._pre(qkv, rotary_emb)
        d = self.dim
        state = ops.linattn_state(qkv[:, :, 1], qkv[:, :, 2], pre=pre_k, head_dim=d)  # [B, h, 1, d+1, d]: this chunk only
        if kv_cache is not None:
            past_vk, past_ks = kv_cache[0], kv_cache[1]
            if save_kv_cache:
                kv_cache[0] = state[:, :, 0, :d].clone()
                kv_cache[1] = state[:, :, 0, d:].clone()
            if past_vk is not None and past_ks is not None:
                state[:, :, 0, :d] += past_vk.to(state)
                state[:, :, 0, d:] += past_ks.to(state)
        out = self._proj_gated(ops.linattn_apply(qkv[:, :, 0], state, self.eps, pre=pre_q), gate, residual)
        if kv_cache is not None:
            return out, kv_cache
        return out


def accumulate_kv_cache(accumulated: Optional[list], saved: list) -> list:
    """Running sum of the attention states a :class:`CachedCausalAttention` saved, as the streaming
    pipeline keeps it between chunks (sana_inference_pipeline.py:242-263): slots 0 and 1 add up,
    any further slot (the temporal-conv tail) is replaced by the newest value."""
    if accumulated is None:
        return [None if t is None else t.clone() for t in saved]
    out = list(accumulated)
    for i, t in enumerate(saved):
        if t is None:
            continue
        out[i] = t.clone() if (i >= 2 or out[i] is None) else out[i] + t
    return out


# ------------------------------------------------------------------ Mix-FFN


class ConvLayer(nn.Module):
    """Parameter holder with the reference's attribute names (basic_modules.py:32-99):
    ``conv`` (nn.Conv2d), ``norm`` (None), ``act``.  GLUMBConv.forward reads the
    parameters and calls the kernels; this module's own forward is the stock op."""

    def __init__(self, in_dim, out_dim, kernel_size=3, groups=1, use_bias=False, act=None):
        super().__init__()
        self.conv = nn.Conv2d(in_dim, out_dim, kernel_size, 1, kernel_size // 2, 1, groups, use_bias)
        self.norm = None
        self.act = nn.SiLU(inplace=True) if act == "silu" else None

    def forward(self, x):
        x = self.conv(x)
        return self.act(x) if self.act else x


def _tuple3(x):
    xs = list(x) if isinstance(x, (list, tuple)) else [x]
    while len(xs) < 3:
        xs.insert(len(xs) - 1, xs[-1])
    return tuple(xs)


class GLUMBConv(nn.Module):
    """Mix-FFN (reference: basic_modules.py:111-199): 1x1 conv C->2H + SiLU,
    depthwise 3x3, gate a * SiLU(g), 1x1 conv H->C.  ``HW`` is (H, W) or
    (T, H, W) (3x3 per frame).  Channels-last throughout: the two 1x1 convs are
    MFMA GEMMs over tokens, the middle is one fused kernel."""

    def __init__(self, in_features: int, hidden_features: int, out_feature=None, kernel_size=3, stride=1,
                 padding=None, use_bias=False, norm=(None, None, None), act=("silu", "silu", None), dilation=1):
        super().__init__()
        out_feature = out_feature or in_features
        use_bias, norm, act = _tuple3(use_bias), _tuple3(norm), _tuple3(act)
        if kernel_size != 3 or stride != 1 or dilation < 1 or padding not in (None, dilation):
            raise NotImplementedError("GLUMBConv HIP path: kernel_size=3, stride=1, 'same' padding only")
        if any(n is not None for n in norm):
            raise NotImplementedError("GLUMBConv HIP path: norm must be (None, None, None)")
        if tuple(act) != ("silu", "silu", None):
            raise NotImplementedError("GLUMBConv HIP path: act must be ('silu', 'silu', None)")
        self.hidden_features = hidden_features
        self.out_feature = out_feature
        self.glu_act = nn.SiLU(inplace=False)
        self.inverted_conv = self._pointwise_layer(in_features, hidden_features * 2, use_bias[0], "silu")
        self.depth_conv = ConvLayer(hidden_features * 2, hidden_features * 2, 3, groups=hidden_features * 2,
                                    use_bias=use_bias[1], act=None)
        # dilation > 1 (`glumbconv_dilate`, diffusion/model/nets/sana.py:126-134) has no kernel: the depthwise stage
        # then runs as the stock convolution (logged), the two 1x1 convolutions stay on the MFMA GEMM
        self.dilation = dilation
        self.depth_conv.conv.dilation = (dilation, dilation)
        self.depth_conv.conv.padding = (dilation, dilation)
        self.point_conv = self._pointwise_layer(hidden_features, out_feature, use_bias[2], None)
        self.round_like_reference = True

    # the two token-wise linears: 1x1 convolutions here (keys ``*.conv.weight`` [out, in, 1, 1]),
    # nn.Linear in GLUMBConvLinear (keys ``*.linear.weight`` [out, in]); the same GEMM either way
    @staticmethod
    def _pointwise_layer(in_dim, out_dim, use_bias, act) -> nn.Module:
        return ConvLayer(in_dim, out_dim, 1, use_bias=use_bias, act=act)

    @staticmethod
    def _pointwise_params(layer: nn.Module) -> nn.Module:
        return layer.conv

    def forward(self, x: torch.Tensor, HW=None) -> torch.Tensor:
        return self.forward_gated(x, HW, None, None)

    def forward_gated(self, x, HW, gate, residual, out=None) -> torch.Tensor:
        """forward(x, HW), or residual + gate * forward(x, HW) fused into the point-conv GEMM.
        ``out``: [B*N, C_out] bf16 view that receives the result (bf16 device path without gate only)."""
        _no_grad_only(x)
        B, N, C = x.shape
        if HW is None:
            HW = self._default_hw(N)
        if len(HW) == 2:
            frames, (H, W) = B, HW
        else:
            T, H, W = HW
            frames = B * T
        if frames * H * W != B * N:
            raise ValueError(f"HW={HW} does not match N={N}")
        ic, pc = self._pointwise_params(self.inverted_conv), self._pointwise_params(self.point_conv)
        dc = self.depth_conv.conv
        u = hip_linear(x, ic.weight, ic.bias, "silu", getattr(ic, "weight_q", None), getattr(ic, "weight_scale", None))
        if self.dilation == 1:
            y = ops.dwconv3x3_silu_gate(u.view(frames, H, W, u.shape[-1]), dc.weight, dc.bias,
                                        round_like_reference=self.round_like_reference)
        else:
            stock_path("GLUMBConv depthwise conv", f"dilation {self.dilation} has no kernel (stock convolution, "
                       "chunk, SiLU and product on a channels-last view)")
            w4 = dc(u.view(frames, H, W, u.shape[-1]).permute(0, 3, 1, 2))          # NCHW view of NHWC memory
            a, g = torch.chunk(w4, 2, dim=1)
            y = (a * self.glu_act(g)).permute(0, 2, 3, 1).contiguous()
        return hip_linear(y.view(B, N, y.shape[-1]), pc.weight, pc.bias, None,
                          getattr(pc, "weight_q", None), getattr(pc, "weight_scale", None), gate, residual, out)

    @staticmethod
    def _default_hw(n_tokens: int):
        raise ValueError("GLUMBConv needs HW (the reference fails on HW=None too: basic_modules.py:193)")

    def quantize_w8_(self) -> "GLUMBConv":
        for conv in (self._pointwise_params(self.inverted_conv), self._pointwise_params(self.point_conv)):
            wq, scale = quantize_w8(conv.weight.data)
            conv.register_buffer("weight_q", wq.contiguous())
            conv.register_buffer("weight_scale", scale.contiguous())
            conv.weight = None
        return self


class GLUMBConvTemp(GLUMBConv):
    """Mix-FFN per frame plus a residual temporal conv (reference: basic_modules.py:200-264):
    ``x + t_conv(x)`` with ``t_conv`` a (t, 1) convolution over frames that mixes all channels,
    zero-initialised.  The per-frame part runs the HIP kernels; the temporal conv runs as one MFMA GEMM
    over the token-major frames (bf16, 3 taps, C % 64 == 0, no frame mask) or as the stock convolution
    on a channels-last view of the same buffer otherwise."""

    def __init__(self, in_features: int, hidden_features: int, out_feature=None, kernel_size=3, stride=1,
                 padding=None, use_bias=False, norm=(None, None, None), act=("silu", "silu", None), t_kernel_size=3):
        super().__init__(in_features, hidden_features, out_feature=out_feature, kernel_size=kernel_size,
                         stride=stride, padding=padding, use_bias=use_bias, norm=norm, act=act)
        out_feature = out_feature or in_features
        self.t_conv = nn.Conv2d(out_feature, out_feature, kernel_size=(t_kernel_size, 1), stride=1,
                                padding=(t_kernel_size // 2, 0), bias=False)
        nn.init.zeros_(self.t_conv.weight)

    def _spatial_bcthw(self, x: torch.Tensor, HW) -> torch.Tensor:
        """tokens [B, N, C] -> the Mix-FFN output as a (B, C, T, H*W) view of its token-major buffer."""
        if HW is None or len(HW) != 3:
            raise ValueError("HW must be a tuple of (T, H, W)")
        B, N, C = x.shape
        T, H, W = HW
        y = super().forward_gated(x, HW, None, None)          # [B, N, C_out], token-major
        return y.view(B, T, H * W, y.shape[-1]).permute(0, 3, 1, 2)

    @staticmethod
    def _tokens(x_bcthw: torch.Tensor) -> torch.Tensor:
        B, C, T, P = x_bcthw.shape
        return x_bcthw.permute(0, 2, 3, 1).reshape(B, T * P, C)

    # -- the temporal conv as one GEMM over a virtual im2col of the token-major frames (bf16, 3 taps,
    #    C % 64 == 0, no frame mask); anything else takes the stock convolution below
    def _tconv_gemm_ok(self, x: torch.Tensor, kwargs) -> bool:
        C = self.t_conv.out_channels
        return (x.is_cuda and x.dtype == torch.bfloat16 and self.t_conv.weight.dtype == torch.bfloat16
                and self.t_conv.kernel_size == (3, 1) and self.t_conv.in_channels == C and C % 64 == 0
                and kwargs.get("frame_valid_mask") is None and not torch.is_grad_enabled())

    def _tconv_stock_note(self, x: torch.Tensor, kwargs) -> None:
        C = self.t_conv.out_channels
        why = ("a frame_valid_mask is given" if kwargs.get("frame_valid_mask") is not None else
               f"dtype {x.dtype} (the GEMM is bf16)" if x.dtype != torch.bfloat16 or self.t_conv.weight.dtype != torch.bfloat16 else
               f"C = {C} is not a multiple of 64" if C % 64 else
               f"kernel {tuple(self.t_conv.kernel_size)} is not (3, 1)" if self.t_conv.kernel_size != (3, 1) else
               "autograd is enabled" if torch.is_grad_enabled() else "input is not on the GPU")
        stock_path(f"{type(self).__name__} temporal conv", why + " (stock convolution instead of the tap GEMM)")

    def _tconv_weight(self) -> torch.Tensor:
        """t_conv.weight [C, C, t, 1] -> [C, t*C] with k = tap * C + input channel (derived data, rebuilt when
        the parameter changes; not part of the state_dict)."""
        w = self.t_conv.weight
        cache = self.__dict__.get("_tconv_cache")
        if cache is None or not _sources_unchanged(cache[0], (w,)):
            with torch.no_grad():
                w2 = w[:, :, :, 0].permute(0, 2, 1).reshape(w.shape[0], -1).contiguous()
            cache = (_source_entry((w,)), w2)
            self.__dict__["_tconv_cache"] = cache
        return cache[1]

    def _spatial_into_frames(self, x: torch.Tensor, HW) -> torch.Tensor:
        """The per-frame Mix-FFN of x [B, T*P, C] written behind one spare frame: returns buf [B, (T+1)*P, C_out]
        with buf[:, P:] = Mix-FFN(x) (the point-conv GEMM stores there directly when B == 1) and buf[:, :P]
        left for the caller (the frame in front of frame 0)."""
        if HW is None or len(HW) != 3:
            raise ValueError("HW must be a tuple of (T, H, W)")
        B, N, _ = x.shape
        P = HW[1] * HW[2]
        buf = x.new_empty(B, N + P, self.t_conv.out_channels)
        if B == 1:
            GLUMBConv.forward_gated(self, x, HW, None, None, out=buf[0, P:])
        else:
            buf[:, P:].copy_(GLUMBConv.forward_gated(self, x, HW, None, None))
        return buf

    def _tconv_residual(self, buf: torch.Tensor, HW, bounds, left: Optional[torch.Tensor] = None) -> torch.Tensor:
        """buf: [B, (T+1)*P, C] from :meth:`_spatial_into_frames`; bounds: first frame of every chunk and T; left:
        the frame in front of frame 0 as tokens [B, P, C], or None for zeros.  A chunk sees the frame in front of
        it and zeros behind it.  Returns y + t_conv(y) [B, T*P, C] for y = buf[:, P:]."""
        B, _, C = buf.shape
        T, P = HW[0], HW[1] * HW[2]
        if left is None:
            buf[:, :P].zero_()
        else:
            buf[:, :P].copy_(left)
        out = buf.new_empty(B, T * P, C)
        w2 = self._tconv_weight()
        # one launch per batch entry for all chunks: the frame behind a chunk's last frame reads as zeros
        # (the last frame of the sequence has nothing behind it in the buffer anyway)
        ends = ops.frame_flags(T, [f1 - 1 for f1 in bounds[1:-1]], buf.device)
        for b in range(B):
            ops.tconv_residual(buf[b], w2, T * P, P, out=out[b], zero_last_tap=ends)
        return out

    def forward(self, x: torch.Tensor, HW=None, **kwargs) -> torch.Tensor:
        B = x.shape[0]
        if self._tconv_gemm_ok(x, kwargs):
            buf = self._spatial_into_frames(x, HW)
            return self._tconv_residual(buf, HW, [0, HW[0]])
        self._tconv_stock_note(x, kwargs)
        xr = self._spatial_bcthw(x, HW)
        frame_mask = kwargs.get("frame_valid_mask", None)
        if frame_mask is not None:
            frame_mask = frame_mask.reshape(B, HW[0]).to(xr)
            xr = xr * frame_mask[:, None, :, None]
        out = xr + self.t_conv(xr)
        if frame_mask is not None:
            out = out * frame_mask[:, None, :, None]
        return self._tokens(out)


class ChunkGLUMBConvTemp(GLUMBConvTemp):
    """Chunked temporal conv (reference: basic_modules.py:267-354, single GPU): every chunk of frames
    sees the tail of the previous chunk on its left and zeros on its right."""

    def forward(self, x: torch.Tensor, HW=None, chunk_index=None, **kwargs) -> torch.Tensor:
        if chunk_index is None:
            chunk_index = [0]
        B = x.shape[0]
        if self._tconv_gemm_ok(x, kwargs):
            buf = self._spatial_into_frames(x, HW)
            T = HW[0]
            return self._tconv_residual(buf, HW, sorted({0, *(int(i) for i in chunk_index if 0 < int(i) < T), T}))
        self._tconv_stock_note(x, kwargs)
        xr = self._spatial_bcthw(x, HW)
        T = HW[0]
        frame_mask = kwargs.get("frame_valid_mask")
        if frame_mask is not None:
            frame_mask = frame_mask.reshape(B, T).to(xr)
            xr = xr * frame_mask[:, None, :, None]
        pad = self.t_conv.kernel_size[0] // 2
        bounds = sorted({0, *(int(i) for i in chunk_index if 0 < int(i) < T), T})
        zeros = xr.new_zeros(B, xr.shape[1], pad, xr.shape[3])
        outs = []
        for a, b in zip(bounds[:-1], bounds[1:]):
            lo = max(a - pad, 0) if a > 0 else a
            seg = torch.cat([xr[:, :, lo:b], zeros], dim=2)
            outs.append(self.t_conv(seg)[:, :, a - lo:a - lo + (b - a)])
        out = xr + torch.cat(outs, dim=2)
        if frame_mask is not None:
            out = out * frame_mask[:, None, :, None]
        return self._tokens(out)


class CachedGLUMBConvTemp(GLUMBConvTemp):
    """Streaming temporal conv (reference: basic_modules.py:357-399): the left context is the last
    slot of ``kv_cache`` (the previous chunk's last frames, saved un-convolved when
    ``save_kv_cache``); returns ``(out, kv_cache)`` when a cache list is passed."""

    def forward(self, x: torch.Tensor, HW=None, save_kv_cache=False, kv_cache=None, **kwargs):
        if self._tconv_gemm_ok(x, kwargs):
            buf = self._spatial_into_frames(x, HW)
            T, P = HW[0], HW[1] * HW[2]
            left = None
            if kv_cache is not None:
                if kv_cache[-1] is not None:     # (B, C, frames, P): the last saved frame, as tokens
                    left = kv_cache[-1][:, :, -1].to(buf).transpose(1, 2)
                if save_kv_cache:                # saved un-convolved, in the reference's (B, C, 1, P) layout
                    kv_cache[-1] = buf[:, T * P:].transpose(1, 2).unsqueeze(2).detach().clone()
            out = self._tconv_residual(buf, HW, [0, T], left)
            return (out, kv_cache) if kv_cache is not None else out
        self._tconv_stock_note(x, kwargs)
        xr = self._spatial_bcthw(x, HW)
        pad = self.t_conv.kernel_size[0] // 2
        x_in, padded = xr, 0
        if kv_cache is not None:
            if kv_cache[-1] is not None:
                x_in = torch.cat([kv_cache[-1][:, :, -pad:].to(xr), xr], dim=2)
                padded = x_in.shape[2] - xr.shape[2]
            if save_kv_cache:
                kv_cache[-1] = xr[:, :, -pad:, :].detach().clone()
        out = self._tokens(xr + self.t_conv(x_in)[:, :, padded:])
        if kv_cache is not None:
            return out, kv_cache
        return out


class LinearLayer(nn.Module):
    """Parameter holder with the reference's attribute names (basic_modules_linear.py:32-58):
    ``linear`` (nn.Linear), ``norm`` (None), ``act``; its own forward is the stock op."""

    def __init__(self, in_dim, out_dim, use_bias=True, act=None):
        super().__init__()
        self.in_dim, self.out_dim, self.use_bias = in_dim, out_dim, use_bias
        self.linear = nn.Linear(in_dim, out_dim, bias=use_bias)
        self.norm = None
        self.act = nn.SiLU(inplace=True) if act == "silu" else None

    def forward(self, x):
        x = self.linear(x)
        return self.act(x) if self.act else x


class GLUMBConvLinear(GLUMBConv):
    """The Mix-FFN with its 1x1 convolutions held as ``nn.Linear`` (reference: basic_modules_linear.py:133-241,
    ``ffn_type="glumbconv_linear"``): keys ``inverted_conv.linear.{weight,bias}``, ``depth_conv.conv.*``,
    ``point_conv.linear.weight``.  Same kernels as GLUMBConv; ``HW=None`` means a square grid (:206-207)."""

    @staticmethod
    def _pointwise_layer(in_dim, out_dim, use_bias, act) -> nn.Module:
        return LinearLayer(in_dim, out_dim, use_bias=use_bias, act=act)

    @staticmethod
    def _pointwise_params(layer: nn.Module) -> nn.Module:
        return layer.linear

    @staticmethod
    def _default_hw(n_tokens: int):
        side = int(n_tokens ** 0.5)
        return side, side


class GLUMBConvLinearTemp(GLUMBConvLinear, GLUMBConvTemp):
    """GLUMBConvLinear per frame plus the residual temporal conv (reference: basic_modules_linear.py:243-311);
    constructor and forward of GLUMBConvTemp, parameters of GLUMBConvLinear."""


# ------------------------------------------------------------------ the block


def t2i_modulate(x, shift, scale):
    return x * (1 + scale) + shift


class MultiHeadCrossAttention(nn.Module):
    """Cross-attention to the text tokens (reference: sana_blocks.py:48-98, the scaled_dot_product_attention
    branch): bf16 inference runs the attention itself as the short-key softmax kernel; its linears are this library's
    GEMM from 4096 rows and library GEMM calls below; everything else (other dtypes, training, more than 320 text tokens, 4-d masks) is stock ops."""

    def __init__(self, d_model, num_heads, attn_drop=0.0, proj_drop=0.0, qk_norm=False, **block_kwargs):
        super().__init__()
        assert d_model % num_heads == 0, "d_model must be divisible by num_heads"
        self.d_model, self.num_heads, self.head_dim = d_model, num_heads, d_model // num_heads
        self.q_linear = nn.Linear(d_model, d_model)
        self.kv_linear = nn.Linear(d_model, d_model * 2)
        self.attn_drop = nn.Dropout(attn_drop)
        self.proj = nn.Linear(d_model, d_model)
        self.proj_drop = nn.Dropout(proj_drop)
        if qk_norm:
            self.q_norm = RMSNorm(d_model, 1.0, 1e-6)
            self.k_norm = RMSNorm(d_model, 1.0, 1e-6)
        else:
            self.q_norm = nn.Identity()
            self.k_norm = nn.Identity()

    # The stock fused-attention kernel is ~3.5x faster at head_dim 128 than at 112 (Sana-1.6B:
    # 2240 / 20 heads).  For inference the three linears are therefore applied with zero-padded
    # copies of their weights (head_dim -> 128): the extra q/k channels are exactly zero and the
    # extra v channels meet zero columns of the output projection, so the result is unchanged
    # while no activation is ever padded or sliced.  The copies are derived data, rebuilt when a
    # parameter changes, and are not part of the state_dict.
    def _padded(self, pad_to):
        ps = (self.q_linear.weight, self.q_linear.bias, self.kv_linear.weight, self.kv_linear.bias,
              self.proj.weight)
        cache = self.__dict__.get("_pad_cache")
        if cache is None or cache[2] != pad_to or not _sources_unchanged(cache[0], ps):
            H, d, C, e = self.num_heads, self.head_dim, self.d_model, pad_to - self.head_dim
            with torch.no_grad():
                wq = F.pad(ps[0].view(H, d, C), (0, 0, 0, e)).reshape(H * pad_to, C)
                bq = F.pad(ps[1].view(H, d), (0, e)).reshape(-1)
                wkv = F.pad(ps[2].view(2, H, d, C), (0, 0, 0, e)).reshape(2 * H * pad_to, C)
                bkv = F.pad(ps[3].view(2, H, d), (0, e)).reshape(-1)
                wo = F.pad(ps[4].view(C, H, d), (0, e)).reshape(C, H * pad_to)
            cache = (_source_entry(ps), (wq.contiguous(), bq.contiguous(), wkv.contiguous(), bkv.contiguous(),
                                         wo.contiguous()), pad_to)
            self.__dict__["_pad_cache"] = cache
        return cache[1]

    def _attend(self, x, cond, mask, kv=None):
        """The HIP path up to proj's input -- softmax(q k^T) v over the short text sequence as one kernel that reads
        q_linear's output and writes proj's input token-major (no head transposes, no padded head_dim) -- or None
        when the call is outside it.  ``kv``: kv_linear(cond) computed by the caller ([B, Nk, 2C] rows, see
        ``StepConditioning``)."""
        B, N, C = x.shape
        H, d = self.num_heads, self.head_dim
        if not (x.is_cuda and x.dtype == torch.bfloat16 and cond.dtype == torch.bfloat16 and not torch.is_grad_enabled()
                and cond.dim() == 3 and cond.shape[0] == B and ops.cross_attention_supported(d, cond.shape[1])
                and (mask is None or (mask.ndim == 2 and tuple(mask.shape) == (B, cond.shape[1])))
                and self.q_linear.weight.dtype == torch.bfloat16):
            return None
        # (below 4096 rows q_linear and kv_linear are library GEMM calls: at a few hundred to a few thousand rows
        # they are faster than this library's GEMM and cost less host time per call)
        if B * N >= self.RESIDUAL_GEMM_MIN_ROWS and self.q_linear.bias is not None and x.is_contiguous():
            q = ops.gemm_bf16(x.view(B * N, C), self.q_linear.weight, self.q_linear.bias, "bias").view(B, N, C)
        else:
            q = F.linear(x, self.q_linear.weight, self.q_linear.bias)
        if kv is None:
            kv = F.linear(cond, self.kv_linear.weight, self.kv_linear.bias)       # [B, Nk, 2C]
        if not isinstance(self.q_norm, nn.Identity):
            q = self.q_norm(q)
        if not isinstance(self.k_norm, nn.Identity):
            kv = torch.cat([self.k_norm(kv[:, :, :C]), kv[:, :, C:]], dim=-1)
        bias = None if mask is None else (1.0 - mask.to(torch.float32)) * -10000.0   # sana_blocks.py:89-90
        return ops.cross_attention(q, kv, H, bias)

    # rows from which proj + the block's residual add run as ONE GEMM of this library (its gated-residual epilogue
    # with a gate of ones: x + (o W^T + b), the same two roundings as the stock linear and add) instead of a
    # library GEMM and an elementwise pass; below it the library GEMM's shorter latency chain wins
    RESIDUAL_GEMM_MIN_ROWS = 4096

    def forward_residual(self, x, cond, mask=None, kv=None):
        """x + self(x, cond, mask) -- what the blocks compute (sana_multi_scale.py:154) -- with the add inside the
        projection GEMM's epilogue when the call is on the HIP path and large enough."""
        B, N, C = x.shape
        if B * N >= self.RESIDUAL_GEMM_MIN_ROWS and isinstance(self.proj_drop, nn.Dropout) and self.proj_drop.p == 0.0:
            o = self._attend(x, cond, mask, kv)
            if o is not None:
                ones = self.__dict__.get("_ones_gate")
                if ones is None or ones.device != x.device or ones.shape[-1] != C:
                    ones = self.__dict__["_ones_gate"] = torch.ones(1, 1, C, dtype=torch.bfloat16, device=x.device)
                return ops.gemm_gate_residual(o, self.proj.weight, self.proj.bias, ones.expand(B, 1, C), x)
        return x + self(x, cond, mask, kv)

    def forward(self, x, cond, mask=None, kv=None):
        B, N, C = x.shape
        H, d = self.num_heads, self.head_dim
        o = self._attend(x, cond, mask, kv)
        if o is not None:
            return self.proj_drop(F.linear(o, self.proj.weight, self.proj.bias))
        if x.is_cuda:
            stock_path("cross-attention",
                       f"the HIP path is bf16 inference with head_dim 72 .. 112, at most {ops.CROSS_ATTN_MAX_KEYS} text tokens "
                       f"and no mask or a [B, Nk] one; got {x.dtype}, head_dim {d}, cond {tuple(cond.shape)}, "
                       f"mask {None if mask is None else tuple(mask.shape)}, grad {'on' if torch.is_grad_enabled() else 'off'}")
        fast = (96 < d < 128 and x.is_cuda and not torch.is_grad_enabled()
                and isinstance(self.q_norm, nn.Identity) and isinstance(self.k_norm, nn.Identity))
        if fast:
            dp = 128
            wq, bq, wkv, bkv, wo = self._padded(dp)
            q = F.linear(x, wq, bq).view(B, -1, H, dp).transpose(1, 2)
            kv = F.linear(cond, wkv, bkv).view(B, -1, 2, H, dp)
            k, v = kv[:, :, 0].transpose(1, 2), kv[:, :, 1].transpose(1, 2)
        else:
            q = self.q_linear(x)
            kv = (self.kv_linear(cond) if kv is None else kv).view(B, -1, 2, C)   # the caller's kv_linear(cond), if given
            k, v = kv.unbind(2)
            q = self.q_norm(q).view(B, -1, H, d).transpose(1, 2)
            k = self.k_norm(k).view(B, -1, H, d).transpose(1, 2)
            v = v.view(B, -1, H, d).transpose(1, 2)
        if mask is not None and mask.ndim == 2:
            mask = (1 - mask.to(q.dtype)) * -10000.0
            mask = mask[:, None, None].repeat(1, H, 1, 1)
        x = F.scaled_dot_product_attention(q, k, v, attn_mask=mask, dropout_p=0.0, is_causal=False,
                                           scale=d ** -0.5)
        if fast:
            x = F.linear(x.transpose(1, 2).reshape(B, -1, H * dp), wo, self.proj.bias)
        else:
            x = self.proj(x.transpose(1, 2).reshape(B, -1, C))
        return self.proj_drop(x)


class SanaMSBlock(nn.Module):
    """Sana DiT block with adaLN-single conditioning (reference:
    sana_multi_scale.py:54-157) for ``attn_type="linear"``, ``ffn_type="glumbconv"``."""

    def __init__(self, hidden_size, num_heads, mlp_ratio=4.0, drop_path=0.0, qk_norm=False, attn_type="flash",
                 ffn_type="mlp", mlp_acts=("silu", "silu", None), linear_head_dim=32, cross_norm=False,
                 cross_attn_type="flash", **block_kwargs):
        super().__init__()
        # "triton_linear" is the reference's Triton twin of the same attention (TritonLiteMLA,
        # fastlinear/modules/triton_lite_mla.py:104-121: qkv without bias, proj, no qk-norm): same math, same keys
        if attn_type not in ("linear", "triton_linear") or ffn_type not in ("glumbconv", "glumbconv_linear"):
            raise NotImplementedError("this block is the attn_type='linear' / ffn_type='glumbconv[_linear]' hot path only")
        if attn_type == "triton_linear":
            qk_norm = False
        if cross_attn_type not in ("flash", "linear"):
            raise NotImplementedError(f"cross_attn_type={cross_attn_type!r}")
        if drop_path > 0.0:
            raise NotImplementedError("drop_path > 0 is a training-time option; this block is forward-only")
        self.hidden_size = hidden_size
        self.norm1 = nn.LayerNorm(hidden_size, elementwise_affine=False, eps=1e-6)
        self.attn = LiteLA(hidden_size, hidden_size, heads=hidden_size // linear_head_dim, eps=1e-8, qk_norm=qk_norm)
        self.cross_attn = MultiHeadCrossAttention(hidden_size, num_heads, qk_norm=cross_norm, **block_kwargs)
        self.norm2 = nn.LayerNorm(hidden_size, elementwise_affine=False, eps=1e-6)
        ffn = GLUMBConv if ffn_type == "glumbconv" else GLUMBConvLinear      # sana_multi_scale.py:117-133
        self.mlp = ffn(in_features=hidden_size, hidden_features=int(hidden_size * mlp_ratio),
                       use_bias=(True, True, False), norm=(None, None, None), act=mlp_acts)
        self.drop_path = nn.Identity()
        self.scale_shift_table = nn.Parameter(torch.randn(6, hidden_size) / hidden_size ** 0.5)

    def forward(self, x, y, t, mask=None, HW=None, image_rotary_emb=None, **kwargs):
        """The reference's signature (sana_multi_scale.py:141).  Two optional keywords ride in ``kwargs``:
        ``text_kv`` / ``modulation``, this block's share of a ``StepConditioning`` call (kv_linear(y) and
        scale_shift_table + t computed for all blocks of the step at once); absent, the block computes them."""
        B, N, C = x.shape
        text_kv, modulation = kwargs.get("text_kv"), kwargs.get("modulation")
        if modulation is None:
            modulation = self.scale_shift_table[None] + t.reshape(B, 6, -1)
        shift_msa, scale_msa, gate_msa, shift_mlp, scale_mlp, gate_mlp = modulation.chunk(6, dim=1)
        # (conditioning in another dtype than x -- an fp32 t with a bf16 x -- promotes in the stock op chain; the
        # fused kernels read the modulation rows as x's dtype, so that case takes the stock composition below)
        if x.is_cuda and x.dtype in ops.IO16 and shift_msa.dtype == x.dtype and C % 8 == 0 and C <= 8192 \
                and not torch.is_grad_enabled():
            # fused seams: LayerNorm + modulate in one kernel, gate * out + residual in the GEMM epilogue
            h = ops.layernorm_modulate(x, scale_msa, shift_msa, self.norm1.eps)
            if "forward" in self.attn.__dict__:
                # a guidance processor was patched over attn.forward (dpm_solver.py:486-524): call it
                x = ops.gate_residual(self.attn(h, HW=HW, rotary_emb=image_rotary_emb), gate_msa, x)
            else:
                x = self.attn.forward_gated(h, gate_msa, x, rotary_emb=image_rotary_emb)
            if B * N >= self.cross_attn.RESIDUAL_GEMM_MIN_ROWS:
                # the cross-attention's residual add inside its projection GEMM, then norm2 + modulate
                x = self.cross_attn.forward_residual(x, y, mask, text_kv)
                h = ops.layernorm_modulate(x, scale_mlp, shift_mlp, self.norm2.eps)
            else:
                # the cross-attention's residual add and norm2 + modulate in one pass
                x, h = ops.add_layernorm_modulate(x, self.cross_attn(x, y, mask, text_kv), scale_mlp, shift_mlp,
                                                   self.norm2.eps)
            return self.mlp.forward_gated(h, HW, gate_mlp, x)
        stock_path("SanaMSBlock LayerNorm / modulate / gate / residual seams",
                   f"the fused seams are bf16 / fp16 inference only (C % 8 == 0, C <= 8192); got x {x.dtype}, t {t.dtype}, C = {C}, "
                   f"grad {'on' if torch.is_grad_enabled() else 'off'}")
        x = x + self.drop_path(
            gate_msa * self.attn(t2i_modulate(self.norm1(x), shift_msa, scale_msa), HW=HW, rotary_emb=image_rotary_emb))
        x = x + self.cross_attn(x, y, mask)
        x = x + self.drop_path(gate_mlp * self.mlp(t2i_modulate(self.norm2(x), shift_mlp, scale_mlp), HW=HW))
        return x

    def quantize_w8_(self) -> "SanaMSBlock":
        """W8A16: int8 per-output-channel weights for qkv, proj and the two 1x1
        convs.  The stock cross-attention linears stay bf16."""
        self.attn.quantize_w8_()
        self.mlp.quantize_w8_()
        return self


class StepConditioning:
    """What every block of one denoising step derives from the step's conditioning alone, for all the blocks of a
    model in two launches: the text tokens' keys and values (``cross_attn.kv_linear(y)``, sana_blocks.py:77 -- a few
    hundred rows, i.e. one latency-bound GEMM per block when the blocks run it themselves, and ONE well-filled GEMM
    over the blocks' stacked weights here) and the six modulation rows (``scale_shift_table + t``,
    sana_multi_scale.py:146-148).  The block loop of the model (sana_multi_scale.py:368-383) becomes

        cond = StepConditioning(blocks)             # once per model
        for blk, c in zip(blocks, cond(y, t)):      # every step: nothing is kept from one call to the next
            x = blk(x, y, t, mask, HW, **c)

    The stacked weights are a derived copy (2 * C * C * 2 bytes per block), rebuilt when a block's parameters
    change, and not part of any state_dict.  Outside bf16 inference on the GPU the call returns empty dicts and
    the blocks compute their own."""

    def __init__(self, blocks):
        self.blocks = list(blocks)
        self._key = None

    def _stacked(self):
        ps = [(b.cross_attn.kv_linear.weight, b.cross_attn.kv_linear.bias, b.scale_shift_table) for b in self.blocks]
        flat = tuple(p for trio in ps for p in trio)
        if not _sources_unchanged(self._key, flat):
            with torch.no_grad():
                self._w = torch.cat([w for w, _, _ in ps])                     # [L * 2C, C]
                self._b = torch.cat([b for _, b, _ in ps])                     # [L * 2C]
                self._tab = torch.stack([s for _, _, s in ps])[:, None]        # [L, 1, 6, C]
            self._key = _source_entry(flat)
        return self._w, self._b, self._tab

    def __call__(self, y, t):
        L = len(self.blocks)
        ca = self.blocks[0].cross_attn if L else None
        if not (L and y.is_cuda and y.dtype == torch.bfloat16 and t.dtype == torch.bfloat16 and y.dim() == 3
                and not torch.is_grad_enabled() and ca.kv_linear.weight.dtype == torch.bfloat16
                and self.blocks[0].scale_shift_table.dtype == torch.bfloat16
                and all(b.cross_attn.d_model == ca.d_model for b in self.blocks)):
            return [{} for _ in self.blocks]
        w, b, tab = self._stacked()
        B, Nk, C = y.shape
        mod = tab + t.reshape(1, B, 6, -1)                                     # [L, B, 6, C]
        # the stacked kv GEMM only where the blocks' cross-attention consumes it: the stock composition for 96 <
        # head_dim < 128 applies kv_linear with a padded copy of its weight and would discard the result
        if not all(ops.cross_attention_supported(b.cross_attn.head_dim, Nk) or not 96 < b.cross_attn.head_dim < 128
                   for b in self.blocks):
            return [dict(modulation=mod[i]) for i in range(L)]
        kv = ops.gemm_bf16(y.reshape(B * Nk, C), w, b, "bias").view(B, Nk, L, 2 * C)
        return [dict(text_kv=kv[:, :, i], modulation=mod[i]) for i in range(L)]


class ChunkedLiteLAReLURope(LiteLAReLURope):
    """The reference's memory-bounded evaluation of LiteLAReLURope in token chunks (sana_blocks.py:1790-1802):
    the same function; the kernels here stream any N, so ``chunk_size`` is kept as an attribute only."""

    def __init__(self, *args, chunk_size=200_000, **kwargs):
        super().__init__(*args, **kwargs)
        self.chunk_size = chunk_size


class SanaVideoMSBlock(nn.Module):
    """The video DiT block (reference: sana_multi_scale_video.py:66-333), the caller of the chunk-causal / cached
    attention and of the temporal Mix-FFN variants: same constructor, ``forward(x, y, t, mask, THW, rotary_emb,
    chunk_index, save_kv_cache=, kv_cache=)``, per-frame conditioning (``t`` [B, 1, F, 6C], :204-254), ``block_hook``
    and ``state_dict`` keys.  LayerNorm + modulation run as the fused kernel (one modulation row per batch entry or
    per frame); attention and Mix-FFN are the HIP modules; cross-attention, gates and residual sums are stock ops."""

    ATTN = {"chunkcausal": ChunkCausalAttention, "cachedcausal": CachedCausalAttention, "linear": LiteLA,
            "LiteLAReLURope": LiteLAReLURope, "ChunkedLiteLAReLURope": ChunkedLiteLAReLURope}
    FFN = {"glumbconv": GLUMBConv, "GLUMBConvTemp": GLUMBConvTemp, "ChunkGLUMBConvTemp": ChunkGLUMBConvTemp,
           "CachedGLUMBConvTemp": CachedGLUMBConvTemp}

    def __init__(self, hidden_size, num_heads, mlp_ratio=4.0, drop_path=0.0, qk_norm=False, attn_type="flash",
                 ffn_type="mlp", mlp_acts=("silu", "silu", None), linear_head_dim=32, cross_norm=False,
                 cross_attn_image_embeds=False, t_kernel_size=3, additional_flash_attn=False,
                 flash_attn_window_count=None, **block_kwargs):
        super().__init__()
        if attn_type not in self.ATTN or ffn_type not in self.FFN:
            raise NotImplementedError(f"this block is the linear-attention / GLUMBConv hot path only: attn_type in "
                                      f"{sorted(self.ATTN)}, ffn_type in {sorted(self.FFN)}")
        if additional_flash_attn or cross_attn_image_embeds:
            raise NotImplementedError("additional_flash_attn / cross_attn_image_embeds are outside this path")
        if drop_path > 0.0:
            raise NotImplementedError("drop_path > 0 is a training-time option; this block is forward-only")
        self.hidden_size = hidden_size
        self.norm1 = nn.LayerNorm(hidden_size, elementwise_affine=False, eps=1e-6)
        self.attn = self.ATTN[attn_type](hidden_size, hidden_size, heads=hidden_size // linear_head_dim, eps=1e-8,
                                         qk_norm=qk_norm)
        self.flash_attn_additional = None
        self.cross_attn_image_embeds = cross_attn_image_embeds
        self.cross_attn = MultiHeadCrossAttention(hidden_size, num_heads, qk_norm=cross_norm, **block_kwargs)
        self.norm2 = nn.LayerNorm(hidden_size, elementwise_affine=False, eps=1e-6)
        ffn_kw = dict(in_features=hidden_size, hidden_features=int(hidden_size * mlp_ratio),
                      use_bias=(True, True, False), norm=(None, None, None), act=mlp_acts)
        if ffn_type != "glumbconv":
            ffn_kw["t_kernel_size"] = t_kernel_size
        self.mlp = self.FFN[ffn_type](**ffn_kw)
        self.drop_path = nn.Identity()
        self.scale_shift_table = nn.Parameter(torch.randn(6, hidden_size) / hidden_size ** 0.5)
        self.block_hook = None

    def _fused(self, x) -> bool:
        """bf16 device inference with the attention's own forward (no processor patched over it)."""
        return (x.is_cuda and x.dtype == torch.bfloat16 and not torch.is_grad_enabled()
                and "forward" not in self.attn.__dict__)

    @staticmethod
    def _gate_residual(x, gate, y):
        """x + gate * y (gate [B, 1, C] or per frame [B, F, 1, C]); one fused pass on the bf16 device path."""
        if x.is_cuda and x.dtype == torch.bfloat16 and y.dtype == torch.bfloat16 and gate.dtype == torch.bfloat16 \
                and x.shape[-1] % 8 == 0 and not torch.is_grad_enabled():
            return ops.gate_residual(y, gate, x)
        B, N, C = x.shape
        stock_path("SanaVideoMSBlock gate / residual", f"the fused pass is bf16 inference only; got {x.dtype} / {y.dtype}, "
                   f"C = {C}, grad {'on' if torch.is_grad_enabled() else 'off'}")
        if gate.dim() == 4:
            return x + (gate * y.reshape(B, gate.shape[1], -1, C)).reshape(B, N, C)
        return x + gate * y

    def _norm_modulate(self, norm, x, shift, scale, groups: int):
        """t2i_modulate(norm(x), shift, scale) with ``groups`` modulation rows per batch entry (1, or one per
        frame): shift / scale are [B, groups, 1, C] or [B, 1, C]."""
        B, N, C = x.shape
        if x.is_cuda and x.dtype == torch.bfloat16 and scale.dtype == x.dtype and shift.dtype == x.dtype \
                and C % 8 == 0 and C <= 8192 and not torch.is_grad_enabled():
            h = ops.layernorm_modulate(x.reshape(B * groups, N // groups, C), scale.reshape(B * groups, 1, C),
                                       shift.reshape(B * groups, 1, C), norm.eps)
            return h.view(B, N, C)
        stock_path("SanaVideoMSBlock LayerNorm / modulate", f"the fused kernel is bf16 inference only (C % 8 == 0, "
                   f"C <= 8192); got {x.dtype}, C = {C}, grad {'on' if torch.is_grad_enabled() else 'off'}")
        if groups == 1:
            return t2i_modulate(norm(x), shift, scale)
        return t2i_modulate(norm(x).reshape(B, groups, -1, C), shift, scale).reshape(B, N, C)

    def forward_frame_aware(self, x, y, t, mask=None, THW=None, rotary_emb=None, chunk_index=None, **kwargs):
        B, N, C = x.shape
        num_frames = t.shape[2]
        t = t.reshape(B, num_frames, 6, -1)
        shift_msa, scale_msa, gate_msa, shift_mlp, scale_mlp, gate_mlp = (
            self.scale_shift_table[None, None, :, :] + t).chunk(6, dim=-2)            # each [B, F, 1, C]
        attn_kw = {"HW": THW, "rotary_emb": rotary_emb}
        if chunk_index is not None:
            attn_kw["chunk_index"] = chunk_index[:]
        h = self._norm_modulate(self.norm1, x, shift_msa, scale_msa, num_frames)
        if self._fused(x):
            x = self.attn.forward_gated(h, gate_msa, x, **attn_kw)
        else:
            x = self._gate_residual(x, gate_msa, self.attn(h, **attn_kw))
        x = self.cross_attn.forward_residual(x, y, mask=mask)
        mlp_kw = {"HW": THW}
        if chunk_index is not None:
            mlp_kw["chunk_index"] = chunk_index[:]
        h = self._norm_modulate(self.norm2, x, shift_mlp, scale_mlp, num_frames)
        return self._gate_residual(x, gate_mlp, self.mlp(h, **mlp_kw))

    def forward(self, x, y, t, mask=None, THW=None, rotary_emb=None, chunk_index=None, **kwargs):
        if len(t.shape) > 2:
            return self.forward_frame_aware(x, y, t, mask=mask, THW=THW, rotary_emb=rotary_emb,
                                            chunk_index=chunk_index, **kwargs)
        B, N, C = x.shape
        feats = {"x_in": x, "x_self_attn": None, "x_cross_attn": None, "x_ffn": None}
        shift_msa, scale_msa, gate_msa, shift_mlp, scale_mlp, gate_mlp = (
            self.scale_shift_table[None] + t.reshape(B, 6, -1)).chunk(6, dim=1)
        attn_kw = {"HW": THW, "rotary_emb": rotary_emb}
        if chunk_index is not None:
            attn_kw["chunk_index"] = chunk_index[:]      # the callee may edit its list
        save_kv_cache = kwargs.get("save_kv_cache", None)
        if save_kv_cache is not None:
            attn_kw["save_kv_cache"] = save_kv_cache
        kv_cache = kwargs.get("kv_cache", None)
        if kv_cache is not None:
            attn_kw["kv_cache"] = kv_cache
        h = self._norm_modulate(self.norm1, x, shift_msa, scale_msa, 1)
        if self.block_hook is None and self._fused(x):
            # x + gate * attn(h) inside the attention's proj GEMM (a hook wants the attention output itself)
            x = self.attn.forward_gated(h, gate_msa, x, **attn_kw)
            if kv_cache is not None:
                x, kv_cache = x
        else:
            x_sa = self.attn(h, **attn_kw)
            if kv_cache is not None:
                x_sa, kv_cache = x_sa
            feats["x_self_attn"] = x_sa
            x = self._gate_residual(x, gate_msa, x_sa)
        x = self.cross_attn.forward_residual(x, y, mask=mask)
        feats["x_cross_attn"] = x
        mlp_kw = {"HW": THW}
        if chunk_index is not None:
            mlp_kw["chunk_index"] = chunk_index[:]
        if save_kv_cache is not None:
            mlp_kw["save_kv_cache"] = save_kv_cache
        if kv_cache is not None:
            mlp_kw["kv_cache"] = kv_cache
        mlp_out = self.mlp(self._norm_modulate(self.norm2, x, shift_mlp, scale_mlp, 1), **mlp_kw)
        if kv_cache is not None:
            mlp_out, kv_cache = mlp_out
        x = self._gate_residual(x, gate_mlp, mlp_out)
        feats["x_ffn"] = x
        if self.block_hook is not None:
            self.block_hook(**feats)
        if kv_cache is not None:
            return x, kv_cache
        return x

    def quantize_w8_(self) -> "SanaVideoMSBlock":
        self.attn.quantize_w8_()
        self.mlp.quantize_w8_()
        return self
