"""Stock-PyTorch restatement of the reference's SanaMSBlock hot path.

TEST INFRASTRUCTURE ONLY (see ``oracle/__init__.py``).  Runs on CPU (and on
any torch device) with no timm / mmcv / xformers dependency.  Every function
cites the reference file:line it follows; paths are relative to the
reference tree.

The dtype / rounding flow mirrors the reference exactly: each torch op
returns the io dtype, ``fp32_attention`` is a module attribute that defaults
to absent (= False), the divide of the linear attention always happens in
fp32.
"""
from __future__ import annotations

import math
from typing import List, Optional, Sequence, Tuple

import torch
import torch.nn.functional as F
from torch import nn

# --------------------------------------------------------------------------
# small helpers
# --------------------------------------------------------------------------


def same_padding(kernel_size: int) -> int:
    """diffusion/model/utils.py:173-179: odd kernel -> k // 2."""
    if kernel_size % 2 == 0:
        raise ValueError(f"kernel size {kernel_size} should be odd number")
    return kernel_size // 2


def as_tuple(x, n: int) -> tuple:
    """diffusion/model/utils.py:155-170 (val2tuple with idx_repeat=-1)."""
    xs = list(x) if isinstance(x, (list, tuple)) else [x]
    while len(xs) < n:
        xs.insert(len(xs) - 1, xs[-1])
    return tuple(xs)


def make_act(name: Optional[str], inplace: bool = True) -> Optional[nn.Module]:
    """diffusion/model/act.py:25-51 — only the names this path uses."""
    if name is None or str(name).lower() == "none":
        return None
    table = {
        "silu": lambda: nn.SiLU(inplace=inplace),
        "swish": lambda: nn.SiLU(inplace=inplace),
        "relu": lambda: nn.ReLU(inplace=inplace),
        "gelu": lambda: nn.GELU(approximate="tanh"),
        "identity": lambda: nn.Identity(),
    }
    if name not in table:
        raise ValueError(f"do not support: {name}")
    return table[name]()


def t2i_modulate(x, shift, scale):
    """diffusion/model/nets/sana_blocks.py:44-45."""
    return x * (1 + scale) + shift


class RMSNorm(nn.Module):
    """diffusion/model/norms.py:182-231: w * x.float() * rsqrt(mean(x^2)+eps), cast back."""

    def __init__(self, dim: int, scale_factor: float = 1.0, eps: float = 1e-6):
        super().__init__()
        self.eps = eps
        self.weight = nn.Parameter(torch.ones(dim) * scale_factor)

    def forward(self, x):
        xf = x.float()
        y = xf * torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + self.eps)
        return (self.weight * y).type_as(x)


# --------------------------------------------------------------------------
# A3: ReLU linear attention core
# --------------------------------------------------------------------------


def relu_linear_attention(
    q: torch.Tensor,
    k: torch.Tensor,
    v: torch.Tensor,
    eps: float,
    fp32_attention: bool = False,
    return_state: bool = False,
):
    """``LiteLA.attn_matmul`` — diffusion/model/nets/sana_blocks.py:245-263.

    q, v: (B, h, d, N); k: (B, h, N, d).  Returns fp32 (B, h, d, N) for
    half-precision inputs (the reference upcasts before the divide) and the
    input dtype for fp32 inputs.  ``state`` is ``vk`` of shape
    (B, h, d+1, d); its last row is sum_n relu(k_n).
    """
    q = torch.relu(q)
    k = torch.relu(k)
    if fp32_attention:
        q, k, v = q.float(), k.float(), v.float()
    v = F.pad(v, (0, 0, 0, 1), mode="constant", value=1.0)
    vk = torch.matmul(v, k)
    out = torch.matmul(vk, q)
    if out.dtype in (torch.float16, torch.bfloat16):
        out = out.float()
    out = out[:, :, :-1] / (out[:, :, -1:] + eps)
    if return_state:
        return out, vk
    return out


def rotary_real(x: torch.Tensor, cos_sin: Tuple[torch.Tensor, torch.Tensor]) -> torch.Tensor:
    """``apply_rotary_emb(..., use_real=True, use_real_unbind_dim=-2)`` —
    sana_blocks.py:1549-1586 as called from ``LiteLA.forward`` (:282-284).

    x: (B, h, d, N); cos, sin: (N, d).  Pairs are adjacent channels (2m, 2m+1).
    """
    cos, sin = cos_sin
    cos = cos[None, None].to(x.device).transpose(-1, -2)
    sin = sin[None, None].to(x.device).transpose(-1, -2)
    xr, xi = x.reshape(*x.shape[:-2], -1, 2, x.shape[-1]).unbind(-2)
    x_rot = torch.stack([-xi, xr], dim=-2).flatten(2, 3)
    return (x.float() * cos + x_rot.float() * sin).to(x.dtype)


def rotary_complex(x: torch.Tensor, freqs: torch.Tensor) -> torch.Tensor:
    """Local ``apply_rotary_emb`` of the ReLU-then-RoPE family —
    sana_blocks.py:359-362 / :429-432.  x: (B, h, d, N); freqs complex
    (1, 1, N, d/2).  Rotation runs in fp64 and is cast back to x's dtype.
    """
    # (.contiguous(): the reference gets a unit last stride from the token-major
    # layout its relu output inherits from qkv; values are the same either way)
    xc = torch.view_as_complex(x.permute(0, 1, 3, 2).to(torch.float64).contiguous().unflatten(3, (-1, 2)))
    out = torch.view_as_real(xc * freqs).flatten(3, 4).permute(0, 1, 3, 2)
    return out.type_as(x)


# --------------------------------------------------------------------------
# A1/A2: LiteLA module
# --------------------------------------------------------------------------


class _AttentionBase(nn.Module):
    """What the reference takes from ``timm.models.vision_transformer.Attention``
    (timm==0.6.13, pyproject.toml:44; not vendored — parity unpinned at this
    seam).  Inferred from sana_blocks.py:229,270,289 and the explicit
    constructor of the reference's Triton twin
    (fastlinear/modules/triton_lite_mla.py:116-117): ``qkv`` and ``proj``.
    """

    def __init__(self, dim: int, num_heads: int, qkv_bias: bool):
        super().__init__()
        self.num_heads = num_heads
        self.scale = (dim // num_heads) ** -0.5
        self.qkv = nn.Linear(dim, dim * 3, bias=qkv_bias)
        self.attn_drop = nn.Dropout(0.0)
        self.proj = nn.Linear(dim, dim)
        self.proj_drop = nn.Dropout(0.0)


class LiteLA(_AttentionBase):
    """diffusion/model/nets/sana_blocks.py:211-301."""

    PAD_VAL = 1

    def __init__(self, in_dim, out_dim, heads=None, heads_ratio=1.0, dim=32, eps=1e-15,
                 use_bias=False, qk_norm=False, norm_eps=1e-5):
        heads = heads or int(out_dim // dim * heads_ratio)
        super().__init__(in_dim, num_heads=heads, qkv_bias=use_bias)
        self.in_dim, self.out_dim, self.heads = in_dim, out_dim, heads
        self.dim = out_dim // heads
        self.eps = eps
        self.kernel_func = nn.ReLU(inplace=False)
        if qk_norm:
            self.q_norm = RMSNorm(in_dim, 1.0, norm_eps)
            self.k_norm = RMSNorm(in_dim, 1.0, norm_eps)
        else:
            self.q_norm = nn.Identity()
            self.k_norm = nn.Identity()

    def attn_matmul(self, q, k, v):
        return relu_linear_attention(q, k, v, self.eps, getattr(self, "fp32_attention", False))

    def forward(self, x, mask=None, HW=None, rotary_emb=None, block_id=None, block_mask=None):
        B, N, C = x.shape
        qkv = self.qkv(x).reshape(B, N, 3, C)
        q, k, v = qkv.unbind(2)
        dtype = q.dtype
        q = self.q_norm(q).transpose(-1, -2)
        k = self.k_norm(k).transpose(-1, -2)
        v = v.transpose(-1, -2)
        h = C // self.dim
        q = q.reshape(B, h, self.dim, N)
        k = k.reshape(B, h, self.dim, N)
        v = v.reshape(B, h, self.dim, N)
        if rotary_emb is not None:
            q = rotary_real(q, rotary_emb)
            k = rotary_real(k, rotary_emb)
        out = self.attn_matmul(q, k.transpose(-1, -2), v).to(dtype)
        out = out.view(B, C, N).permute(0, 2, 1)
        return self.proj(out)


# --------------------------------------------------------------------------
# A9/A10/A11: ReLU -> RoPE linear attention, chunk-causal and cached forms
# --------------------------------------------------------------------------


class SelfAttnProcessorLiteLA:
    """diffusion/model/nets/sana_blocks.py:677-717: LiteLA.forward restated on the module's parts
    (``qkv``, ``q_norm``, ``k_norm``, ``dim``, ``kernel_func``, ``attn_matmul``, ``proj``)."""

    def __init__(self, attn):
        self.attn = attn

    def _attend(self, x, rotary_emb):
        a = self.attn
        B, N, C = x.shape
        qkv = a.qkv(x).reshape(B, N, 3, C)
        q, k, v = qkv.unbind(2)
        dtype = q.dtype
        q = a.q_norm(q).transpose(-1, -2).reshape(B, C // a.dim, a.dim, N)
        k = a.k_norm(k).transpose(-1, -2).reshape(B, C // a.dim, a.dim, N)
        v = v.transpose(-1, -2).reshape(B, C // a.dim, a.dim, N)
        if rotary_emb is not None:
            q, k = rotary_real(q, rotary_emb), rotary_real(k, rotary_emb)
        q, k = a.kernel_func(q), a.kernel_func(k)
        out = a.attn_matmul(q, k.transpose(-1, -2), v).to(dtype)
        return a.proj(out.view(B, C, N).permute(0, 2, 1))

    def _identity(self, x_ptb):
        """:615-622: the perturbed path replaces the attention by the identity: proj(v_linear(x))."""
        a = self.attn
        C = x_ptb.shape[-1]
        y = torch.matmul(x_ptb, a.qkv.weight[C * 2:C * 3, :].t())
        if a.qkv.bias is not None:
            y = y + a.qkv.bias[C * 2:C * 3]
        return a.proj(y.to(x_ptb.dtype))

    def __call__(self, x, mask=None, HW=None, rotary_emb=None, block_id=None, block_mask=None, **kwargs):
        return self._attend(x, rotary_emb)


class PAGIdentitySelfAttnProcessorLiteLA(SelfAttnProcessorLiteLA):
    """sana_blocks.py:627-674: batch = [cond | perturbed]."""

    def __call__(self, x, mask=None, HW=None, rotary_emb=None, block_id=None, block_mask=None, **kwargs):
        x_org, x_ptb = x.chunk(2)
        return torch.cat([self._attend(x_org, rotary_emb), self._identity(x_ptb)])


class PAGCFGIdentitySelfAttnProcessorLiteLA(SelfAttnProcessorLiteLA):
    """sana_blocks.py:575-624: batch = [uncond | cond | perturbed]."""

    def __call__(self, x, mask=None, HW=None, rotary_emb=None, block_id=None, block_mask=None, **kwargs):
        x_uncond, x_org, x_ptb = x.chunk(3)
        return torch.cat([self._attend(torch.cat([x_uncond, x_org]), rotary_emb), self._identity(x_ptb)])


class LiteLAReLURope(_AttentionBase):
    """diffusion/model/nets/sana_blocks.py:304-388."""

    def __init__(self, in_dim, out_dim, heads=None, heads_ratio=1.0, dim=32, eps=1e-15,
                 use_bias=False, qk_norm=False, norm_eps=1e-5):
        heads = heads or int(out_dim // dim * heads_ratio)
        super().__init__(in_dim, num_heads=heads, qkv_bias=use_bias)
        self.in_dim, self.out_dim, self.heads = in_dim, out_dim, heads
        self.dim = out_dim // heads
        self.eps = eps
        self.kernel_func = nn.ReLU(inplace=False)
        if qk_norm:
            self.q_norm = RMSNorm(in_dim, 1.0, norm_eps)
            self.k_norm = RMSNorm(in_dim, 1.0, norm_eps)
        else:
            self.q_norm = nn.Identity()
            self.k_norm = nn.Identity()

    def _qkv_heads(self, x):
        """Shared prologue (:343-357): q, k ReLU'd, all as (B, h, d, N)."""
        B, N, C = x.shape
        qkv = self.qkv(x).reshape(B, N, 3, C)
        q, k, v = qkv.unbind(2)
        dtype = q.dtype
        q = self.q_norm(q).transpose(-1, -2)
        k = self.k_norm(k).transpose(-1, -2)
        v = v.transpose(-1, -2)
        h = C // self.dim
        q = torch.relu(q.reshape(B, h, self.dim, N))
        k = torch.relu(k.reshape(B, h, self.dim, N))
        v = v.reshape(B, h, self.dim, N)
        return q, k, v, dtype

    def _rotate(self, q, k, rotary_emb):
        if rotary_emb is None:
            # the reference requires rotary_emb; a unit rotation is its identity element
            return q, k
        return rotary_complex(q, rotary_emb), rotary_complex(k, rotary_emb)

    def forward(self, x, mask=None, HW=None, rotary_emb=None, block_mask=None, **kwargs):
        B, N, C = x.shape
        q, k, v, dtype = self._qkv_heads(x)
        q_rot, k_rot = self._rotate(q, k, rotary_emb)
        if getattr(self, "fp32_attention", False):
            q_rot, k_rot, v = q_rot.float(), k_rot.float(), v.float()
        # denominator from the UNROTATED q, k (:378)
        z = 1 / (k.sum(dim=-1, keepdim=True).transpose(-2, -1) @ q + self.eps)
        vk = torch.matmul(v, k_rot.transpose(-1, -2))
        out = torch.matmul(vk, q_rot)
        out = (out * z).to(dtype)
        out = out.view(B, C, N).permute(0, 2, 1)
        return self.proj(out)


class ChunkCausalAttention(LiteLAReLURope):
    """diffusion/model/nets/sana_blocks.py:391-495.  Chunks are runs of whole
    frames; a chunk attends to itself and every earlier chunk (inclusive
    prefix of the per-chunk states)."""

    def forward(self, x, mask=None, HW=None, rotary_emb=None, block_mask=None,
                chunk_index: Optional[List[int]] = None):
        B, N, C = x.shape
        q, k, v, dtype = self._qkv_heads(x)
        q_rot, k_rot = self._rotate(q, k, rotary_emb)
        if getattr(self, "fp32_attention", False):
            q_rot, k_rot, v = q_rot.float(), k_rot.float(), v.float()
        f, hh, ww = HW
        bounds = (list(chunk_index) if chunk_index is not None else [0]) + [f]
        sizes = [b - a for a, b in zip(bounds[:-1], bounds[1:])]
        h, d = q_rot.shape[1], q_rot.shape[2]

        def split(t):
            return [c.reshape(B, h, d, -1) for c in t.unflatten(-1, (f, hh, ww)).split(sizes, dim=-3)]

        cum_vk = torch.zeros(B, h, d, d, dtype=k_rot.dtype, device=k_rot.device)
        cum_k = torch.zeros(B, h, 1, d, dtype=k_rot.dtype, device=k_rot.device)
        outs = []
        for qr_c, kr_c, v_c, q_c, k_c in zip(split(q_rot), split(k_rot), split(v), split(q), split(k)):
            cum_vk += torch.matmul(v_c, kr_c.transpose(-1, -2))
            cum_k += k_c.sum(dim=-1, keepdim=True).transpose(-2, -1)
            z = 1 / (cum_k @ q_c + self.eps)
            outs.append((torch.matmul(cum_vk, qr_c) * z).to(dtype))
        out = torch.cat(outs, dim=-1)
        out = out.view(B, C, N).permute(0, 2, 1)
        return self.proj(out)


class CachedCausalAttention(LiteLAReLURope):
    """diffusion/model/nets/sana_blocks.py:498-572.  Streaming form: the caller
    supplies the accumulated past state in ``kv_cache[0:2]``; with
    ``save_kv_cache`` this chunk's own (un-accumulated) state replaces it."""

    def forward(self, x, mask=None, HW=None, rotary_emb=None, block_mask=None,
                save_kv_cache=False, kv_cache=None, **kwargs):
        B, N, C = x.shape
        q, k, v, dtype = self._qkv_heads(x)
        q_rot, k_rot = self._rotate(q, k, rotary_emb)
        if getattr(self, "fp32_attention", False):
            q_rot, k_rot, v = q_rot.float(), k_rot.float(), v.float()
        k_sum = k.sum(dim=-1, keepdim=True).transpose(-2, -1)
        vk = torch.matmul(v, k_rot.transpose(-1, -2))
        if kv_cache is not None:
            past_vk, past_k = kv_cache[0], kv_cache[1]
            if save_kv_cache:
                kv_cache[0] = vk.detach().clone()
                kv_cache[1] = k_sum.detach().clone()
            if past_vk is not None and past_k is not None:
                vk = vk + past_vk
                k_sum = k_sum + past_k
        z = 1 / (k_sum @ q + self.eps)
        out = (torch.matmul(vk, q_rot) * z).to(dtype)
        out = out.view(B, C, N).permute(0, 2, 1)
        out = self.proj(out)
        if kv_cache is not None:
            return out, kv_cache
        return out


# --------------------------------------------------------------------------
# A4/A5/A6: GLUMBConv
# --------------------------------------------------------------------------


class ConvLayer(nn.Module):
    """diffusion/model/nets/basic_modules.py:32-99 (2-d branch, no norm/dropout)."""

    def __init__(self, in_dim, out_dim, kernel_size=3, stride=1, dilation=1, groups=1,
                 padding=None, use_bias=False, norm=None, act="relu"):
        super().__init__()
        if norm is not None:
            raise NotImplementedError("the hot path builds every ConvLayer with norm=None")
        if padding is None:
            padding = same_padding(kernel_size) * dilation
        self.conv = nn.Conv2d(in_dim, out_dim, (kernel_size, kernel_size), (stride, stride),
                              padding, (dilation, dilation), groups, use_bias)
        self.norm = None
        self.act = make_act(act)

    def forward(self, x):
        x = self.conv(x)
        if self.act:
            x = self.act(x)
        return x


INT32_SAFE_CONV_ELEMENTS = 1 << 30  # basic_modules.py:108


class GLUMBConv(nn.Module):
    """diffusion/model/nets/basic_modules.py:111-199."""

    def __init__(self, in_features, hidden_features, out_feature=None, kernel_size=3, stride=1,
                 padding=None, use_bias=False, norm=(None, None, None),
                 act=("silu", "silu", None), dilation=1):
        super().__init__()
        out_feature = out_feature or in_features
        use_bias = as_tuple(use_bias, 3)
        norm = as_tuple(norm, 3)
        act = as_tuple(act, 3)
        self.glu_act = make_act(act[1], inplace=False)
        self.inverted_conv = ConvLayer(in_features, hidden_features * 2, 1,
                                       use_bias=use_bias[0], norm=norm[0], act=act[0])
        self.depth_conv = ConvLayer(hidden_features * 2, hidden_features * 2, kernel_size,
                                    stride=stride, groups=hidden_features * 2, padding=padding,
                                    use_bias=use_bias[1], norm=norm[1], act=None, dilation=dilation)
        self.point_conv = ConvLayer(hidden_features, out_feature, 1,
                                    use_bias=use_bias[2], norm=norm[2], act=act[2])

    def _apply_spatial(self, x):
        x = self.inverted_conv(x)
        x = self.depth_conv(x)
        a, g = torch.chunk(x, 2, dim=1)
        g = self.glu_act(g)
        return self.point_conv(a * g)

    def _apply_spatial_autochunked(self, x):
        BT, _, H, W = x.shape
        per_bt = self.inverted_conv.conv.out_channels * H * W
        max_bt = max(1, INT32_SAFE_CONV_ELEMENTS // per_bt)
        if BT <= max_bt:
            return self._apply_spatial(x)
        return torch.cat([self._apply_spatial(x[s:s + max_bt]) for s in range(0, BT, max_bt)], dim=0)

    def forward(self, x, HW=None):
        B, N, C = x.shape
        if HW is None:
            # the reference is broken for HW=None (len(None) at :193); it is effectively required
            raise ValueError("HW is required")
        if len(HW) == 2:
            H, W = HW
            x = x.reshape(B, H, W, C).permute(0, 3, 1, 2)
        else:
            T, H, W = HW
            x = x.reshape(B * T, H, W, C).permute(0, 3, 1, 2)
        x = self._apply_spatial_autochunked(x)
        if len(HW) == 3:
            x = x.reshape(B * T, C, H * W).permute(0, 2, 1).reshape(B, N, C)
        else:
            x = x.reshape(B, C, N).permute(0, 2, 1)
        return x


class GLUMBConvTemp(GLUMBConv):
    """diffusion/model/nets/basic_modules.py:200-264 (single GPU: no halo exchange).  The Mix-FFN per
    frame, then a residual temporal conv (kernel (t, 1), full channel mixing, zero-initialised)."""

    def __init__(self, in_features, hidden_features, out_feature=None, kernel_size=3, stride=1, padding=None,
                 use_bias=False, norm=(None, None, None), act=("silu", "silu", None), t_kernel_size=3):
        super().__init__(in_features, hidden_features, out_feature=out_feature, kernel_size=kernel_size,
                         stride=stride, padding=padding, use_bias=use_bias, norm=norm, act=act)
        out_feature = out_feature or in_features
        self.t_conv = nn.Conv2d(out_feature, out_feature, kernel_size=(t_kernel_size, 1), stride=1,
                                padding=(t_kernel_size // 2, 0), bias=False)
        nn.init.zeros_(self.t_conv.weight)

    def _spatial_bcthw(self, x, HW):
        """:238-246: tokens -> (B, C, T, H*W) after the per-frame Mix-FFN."""
        B, N, C = x.shape
        assert len(HW) == 3, "HW must be a tuple of (T, H, W)"
        T, H, W = HW
        x = x.reshape(B * T, H, W, C).permute(0, 3, 1, 2)
        x = self._apply_spatial_autochunked(x)
        return x.view(B, T, C, H * W).permute(0, 2, 1, 3)

    def forward(self, x, HW=None, **kwargs):
        B, N, C = x.shape
        x_reshaped = self._spatial_bcthw(x, HW)
        frame_mask = kwargs.get("frame_valid_mask", None)
        if frame_mask is not None:
            frame_mask = frame_mask.reshape(B, HW[0]).to(x_reshaped)
            x_reshaped = x_reshaped * frame_mask[:, None, :, None]
        x_out = x_reshaped + self.t_conv(x_reshaped)
        if frame_mask is not None:
            x_out = x_out * frame_mask[:, None, :, None]
        return x_out.permute(0, 2, 3, 1).reshape(B, N, C)


class ChunkGLUMBConvTemp(GLUMBConvTemp):
    """basic_modules.py:267-354 (single GPU).  The temporal conv sees, for every chunk of frames, the
    tail of the previous chunk on the left and zeros on the right."""

    def forward(self, x, HW=None, chunk_index=None, **kwargs):
        if chunk_index is None:
            chunk_index = [0]
        B, N, C = x.shape
        T = HW[0]
        x_reshaped = self._spatial_bcthw(x, HW)
        frame_mask = kwargs.get("frame_valid_mask")
        if frame_mask is not None:
            frame_mask = frame_mask.reshape(B, T).to(x_reshaped)
            x_reshaped = x_reshaped * frame_mask[:, None, :, None]
        pad = self.t_conv.kernel_size[0] // 2
        bounds = sorted({0, *(int(i) for i in chunk_index if 0 < int(i) < T), T})
        outs = []
        for a, b in zip(bounds[:-1], bounds[1:]):
            left = x_reshaped[:, :, a - pad:a] if a > 0 else x_reshaped.new_zeros(B, C, 0, x_reshaped.shape[-1])
            seg = torch.cat([left, x_reshaped[:, :, a:b], x_reshaped.new_zeros(B, C, pad, x_reshaped.shape[-1])], dim=2)
            o = self.t_conv(seg)   # its own zero padding adds `pad` rows either side
            outs.append(o[:, :, left.shape[2]:left.shape[2] + (b - a)])
        x_out = x_reshaped + torch.cat(outs, dim=2)
        if frame_mask is not None:
            x_out = x_out * frame_mask[:, None, :, None]
        return x_out.permute(0, 2, 3, 1).reshape(B, N, C)


class CachedGLUMBConvTemp(GLUMBConvTemp):
    """basic_modules.py:357-399.  Streaming form: the left context of the temporal conv comes from
    the last slot of ``kv_cache`` (the previous chunk's last frames, saved un-convolved)."""

    def forward(self, x, HW=None, save_kv_cache=False, kv_cache=None, **kwargs):
        B, N, C = x.shape
        x_reshaped = self._spatial_bcthw(x, HW)
        pad = self.t_conv.kernel_size[0] // 2
        x_in, padded = x_reshaped, 0
        if kv_cache is not None:
            if kv_cache[-1] is not None:
                x_in = torch.cat([kv_cache[-1][:, :, -pad:], x_reshaped], dim=2)
                padded = x_in.shape[2] - x_reshaped.shape[2]
            if save_kv_cache:
                kv_cache[-1] = x_reshaped[:, :, -pad:, :].detach().clone()
        x_out = x_reshaped + self.t_conv(x_in)[:, :, padded:]
        x_out = x_out.permute(0, 2, 3, 1).reshape(B, N, C)
        if kv_cache is not None:
            return x_out, kv_cache
        return x_out


# --------------------------------------------------------------------------
# A14: cross attention (SDPA branch), A7: the block
# --------------------------------------------------------------------------


class LinearLayer(nn.Module):
    """diffusion/model/nets/basic_modules_linear.py:32-58 (no norm)."""

    def __init__(self, in_dim, out_dim, use_bias=True, norm=None, act=None):
        super().__init__()
        if norm is not None:
            raise NotImplementedError("the hot path builds every LinearLayer with norm=None")
        self.in_dim, self.out_dim, self.use_bias = in_dim, out_dim, use_bias
        self.linear = nn.Linear(in_dim, out_dim, bias=use_bias)
        self.norm = None
        self.act = make_act(act)

    def forward(self, x):
        x = self.linear(x)
        if self.act:
            x = self.act(x)
        return x


class GLUMBConvLinear(nn.Module):
    """diffusion/model/nets/basic_modules_linear.py:133-241: the Mix-FFN with its two 1x1 convolutions held as
    ``nn.Linear`` over tokens (keys ``inverted_conv.linear.*``, ``point_conv.linear.*``); the depthwise 3x3 stays
    a ConvLayer.  ``HW=None`` means a square grid (:206-207)."""

    def __init__(self, in_features, hidden_features, out_feature=None, kernel_size=3, stride=1,
                 padding=None, use_bias=False, norm=(None, None, None),
                 act=("silu", "silu", None), dilation=1):
        out_feature = out_feature or in_features
        super().__init__()
        use_bias = as_tuple(use_bias, 3)
        norm = as_tuple(norm, 3)
        act = as_tuple(act, 3)
        self.hidden_features = hidden_features
        self.out_feature = out_feature
        self.glu_act = make_act(act[1], inplace=False)
        self.inverted_conv = LinearLayer(in_features, hidden_features * 2, use_bias=use_bias[0], norm=norm[0],
                                         act=act[0])
        self.depth_conv = ConvLayer(hidden_features * 2, hidden_features * 2, kernel_size,
                                    stride=stride, groups=hidden_features * 2, padding=padding,
                                    use_bias=use_bias[1], norm=norm[1], act=None, dilation=dilation)
        self.point_conv = LinearLayer(hidden_features, out_feature, use_bias=use_bias[2], norm=norm[2], act=act[2])

    def _frames(self, x, HW):
        """:204-236 up to the point conv: tokens [B, N, C] -> [frames, H*W, hidden]."""
        B, N, C = x.shape
        if HW is None:
            H = W = int(N ** 0.5)
            frames = B
        elif len(HW) == 2:
            (H, W), frames = HW, B
        else:
            T, H, W = HW
            frames = B * T
        x = self.inverted_conv(x)
        x = x.reshape(frames, H, W, -1).permute(0, 3, 1, 2)
        x = self.depth_conv(x)
        a, g = torch.chunk(x, 2, dim=1)
        x = a * self.glu_act(g)
        return x.reshape(frames, self.hidden_features, H * W).permute(0, 2, 1)

    def forward(self, x, HW=None):
        B, N, C = x.shape
        return self.point_conv(self._frames(x, HW).reshape(B, N, self.hidden_features))


class GLUMBConvLinearTemp(GLUMBConvLinear):
    """diffusion/model/nets/basic_modules_linear.py:243-311: GLUMBConvLinear per frame, then ``x + t_conv(x)``."""

    def __init__(self, in_features, hidden_features, out_feature=None, kernel_size=3, stride=1, padding=None,
                 use_bias=False, norm=(None, None, None), act=("silu", "silu", None), t_kernel_size=3):
        super().__init__(in_features, hidden_features, out_feature=out_feature, kernel_size=kernel_size,
                         stride=stride, padding=padding, use_bias=use_bias, norm=norm, act=act)
        out_feature = out_feature or in_features
        self.t_conv = nn.Conv2d(out_feature, out_feature, kernel_size=(t_kernel_size, 1), stride=1,
                                padding=(t_kernel_size // 2, 0), bias=False)
        nn.init.zeros_(self.t_conv.weight)

    def forward(self, x, HW=None, **kwargs):
        B, N, C = x.shape
        assert len(HW) == 3, "HW must be a tuple of (T, H, W)"
        T, H, W = HW
        x = self.point_conv(self._frames(x, HW))                       # (B*T, H*W, out)
        x = x.reshape(B, T, H * W, self.out_feature).permute(0, 3, 1, 2)
        x_out = x + self.t_conv(x)
        return x_out.permute(0, 2, 3, 1).reshape(B, N, self.out_feature)


class MultiHeadCrossAttention(nn.Module):
    """diffusion/model/nets/sana_blocks.py:48-98, branch without xformers (:86-92)."""

    def __init__(self, d_model, num_heads, qk_norm=False):
        super().__init__()
        if d_model % num_heads:
            raise ValueError("d_model must be divisible by num_heads")
        self.d_model, self.num_heads, self.head_dim = d_model, num_heads, d_model // num_heads
        self.q_linear = nn.Linear(d_model, d_model)
        self.kv_linear = nn.Linear(d_model, d_model * 2)
        self.proj = nn.Linear(d_model, d_model)
        if qk_norm:
            self.q_norm = RMSNorm(d_model, 1.0, 1e-6)
            self.k_norm = RMSNorm(d_model, 1.0, 1e-6)
        else:
            self.q_norm = nn.Identity()
            self.k_norm = nn.Identity()

    def forward(self, x, cond, mask=None):
        B, N, C = x.shape
        q = self.q_linear(x)
        kv = self.kv_linear(cond).view(B, -1, 2, C)
        k, v = kv.unbind(2)
        q = self.q_norm(q).view(B, -1, self.num_heads, self.head_dim).transpose(1, 2)
        k = self.k_norm(k).view(B, -1, self.num_heads, self.head_dim).transpose(1, 2)
        v = v.view(B, -1, self.num_heads, self.head_dim).transpose(1, 2)
        if mask is not None and mask.ndim == 2:
            mask = (1 - mask.to(q.dtype)) * -10000.0
            mask = mask[:, None, None].repeat(1, self.num_heads, 1, 1)
        x = F.scaled_dot_product_attention(q, k, v, attn_mask=mask, dropout_p=0.0, is_causal=False)
        x = x.transpose(1, 2).reshape(B, -1, C)
        return self.proj(x)


class SanaMSBlock(nn.Module):
    """diffusion/model/nets/sana_multi_scale.py:54-157 with attn_type="linear",
    ffn_type="glumbconv" (the configuration of every shipped Sana config)."""

    def __init__(self, hidden_size, num_heads, mlp_ratio=4.0, drop_path=0.0, qk_norm=False,
                 attn_type="flash", ffn_type="mlp", mlp_acts=("silu", "silu", None),
                 linear_head_dim=32, cross_norm=False, cross_attn_type="flash", **block_kwargs):
        super().__init__()
        if attn_type != "linear" or ffn_type not in ("glumbconv", "glumbconv_linear"):
            raise NotImplementedError("oracle restates attn_type='linear', ffn_type='glumbconv[_linear]' only")
        self.hidden_size = hidden_size
        self.norm1 = nn.LayerNorm(hidden_size, elementwise_affine=False, eps=1e-6)
        self.attn = LiteLA(hidden_size, hidden_size, heads=hidden_size // linear_head_dim,
                           eps=1e-8, qk_norm=qk_norm)
        self.cross_attn = MultiHeadCrossAttention(hidden_size, num_heads, qk_norm=cross_norm)
        self.norm2 = nn.LayerNorm(hidden_size, elementwise_affine=False, eps=1e-6)
        ffn = GLUMBConv if ffn_type == "glumbconv" else GLUMBConvLinear          # :117-133
        self.mlp = ffn(hidden_size, int(hidden_size * mlp_ratio), use_bias=(True, True, False),
                       norm=(None, None, None), act=mlp_acts)
        self.drop_path = nn.Identity()
        self.scale_shift_table = nn.Parameter(torch.randn(6, hidden_size) / hidden_size ** 0.5)

    def forward(self, x, y, t, mask=None, HW=None, image_rotary_emb=None, **kwargs):
        B, N, C = x.shape
        shift_msa, scale_msa, gate_msa, shift_mlp, scale_mlp, gate_mlp = (
            self.scale_shift_table[None] + t.reshape(B, 6, -1)
        ).chunk(6, dim=1)
        x = x + gate_msa * self.attn(t2i_modulate(self.norm1(x), shift_msa, scale_msa),
                                     HW=HW, rotary_emb=image_rotary_emb)
        x = x + self.cross_attn(x, y, mask)
        x = x + gate_mlp * self.mlp(t2i_modulate(self.norm2(x), shift_mlp, scale_mlp), HW=HW)
        return x


class ChunkedLiteLAReLURope(LiteLAReLURope):
    """diffusion/model/nets/sana_blocks.py:1790-1802 onwards: LiteLAReLURope evaluated in token chunks of
    ``chunk_size`` to bound memory; the same function of its inputs (restated as the unchunked call)."""

    def __init__(self, *args, chunk_size=200_000, **kwargs):
        super().__init__(*args, **kwargs)
        self.chunk_size = chunk_size


class SanaVideoMSBlock(nn.Module):
    """diffusion/model/nets/sana_multi_scale_video.py:66-333: the video DiT block, the caller of the chunk-causal /
    cached attention and of the temporal Mix-FFN variants.  Restated for the linear-attention ``attn_type`` values
    and the GLUMBConv family of ``ffn_type`` values, without the optional extra flash attention, image-embedding
    cross-attention and drop-path (all off in the released SANA-Video configurations)."""

    ATTN = {"chunkcausal": "ChunkCausalAttention", "cachedcausal": "CachedCausalAttention", "linear": "LiteLA",
            "LiteLAReLURope": "LiteLAReLURope", "ChunkedLiteLAReLURope": "ChunkedLiteLAReLURope"}
    FFN = ("glumbconv", "GLUMBConvTemp", "ChunkGLUMBConvTemp", "CachedGLUMBConvTemp")

    def __init__(self, hidden_size, num_heads, mlp_ratio=4.0, drop_path=0.0, qk_norm=False, attn_type="flash",
                 ffn_type="mlp", mlp_acts=("silu", "silu", None), linear_head_dim=32, cross_norm=False,
                 cross_attn_image_embeds=False, t_kernel_size=3, additional_flash_attn=False,
                 flash_attn_window_count=None, **block_kwargs):
        super().__init__()
        if attn_type not in self.ATTN or ffn_type not in self.FFN or additional_flash_attn or \
                cross_attn_image_embeds or drop_path > 0.0:
            raise NotImplementedError("oracle restates the linear-attention / GLUMBConv-family video block only")
        self.hidden_size = hidden_size
        self.norm1 = nn.LayerNorm(hidden_size, elementwise_affine=False, eps=1e-6)
        attn_cls = globals()[self.ATTN[attn_type]]
        self.attn = attn_cls(hidden_size, hidden_size, heads=hidden_size // linear_head_dim, eps=1e-8,
                             qk_norm=qk_norm)                                                    # :101-119
        self.flash_attn_additional = None
        self.cross_attn_image_embeds = cross_attn_image_embeds
        self.cross_attn = MultiHeadCrossAttention(hidden_size, num_heads, qk_norm=cross_norm)
        self.norm2 = nn.LayerNorm(hidden_size, elementwise_affine=False, eps=1e-6)
        ffn_kw = dict(in_features=hidden_size, hidden_features=int(hidden_size * mlp_ratio),
                      use_bias=(True, True, False), norm=(None, None, None), act=mlp_acts)
        if ffn_type == "glumbconv":                                                              # :156-191
            self.mlp = GLUMBConv(**ffn_kw)
        else:
            self.mlp = globals()[ffn_type](t_kernel_size=t_kernel_size, **ffn_kw)
        self.drop_path = nn.Identity()
        self.scale_shift_table = nn.Parameter(torch.randn(6, hidden_size) / hidden_size ** 0.5)
        self.block_hook = None

    def forward_frame_aware(self, x, y, t, mask=None, THW=None, rotary_emb=None, chunk_index=None, **kwargs):
        """:204-254: one modulation row per frame, t = [B, 1, F, 6C]."""
        B, N, C = x.shape
        num_frames = t.shape[2]
        t = t.reshape(B, num_frames, 6, -1)
        shift_msa, scale_msa, gate_msa, shift_mlp, scale_mlp, gate_mlp = (
            self.scale_shift_table[None, None, :, :] + t).chunk(6, dim=-2)            # each B, F, 1, C
        attn_kw = {"HW": THW, "rotary_emb": rotary_emb}
        if chunk_index is not None:
            attn_kw["chunk_index"] = chunk_index[:]
        h = t2i_modulate(self.norm1(x).reshape(B, num_frames, -1, C), shift_msa, scale_msa).reshape(B, N, C)
        x = x + (gate_msa * self.attn(h, **attn_kw).reshape(B, num_frames, -1, C)).reshape(B, N, C)
        x = x + self.cross_attn(x, y, mask=mask)
        mlp_kw = {"HW": THW}
        if chunk_index is not None:
            mlp_kw["chunk_index"] = chunk_index[:]
        h = t2i_modulate(self.norm2(x).reshape(B, num_frames, -1, C), shift_mlp, scale_mlp).reshape(B, N, C)
        x = x + (gate_mlp * self.mlp(h, **mlp_kw).reshape(B, num_frames, -1, C)).reshape(B, N, C)
        return x

    def forward(self, x, y, t, mask=None, THW=None, rotary_emb=None, chunk_index=None, **kwargs):
        """:256-333."""
        if len(t.shape) > 2:
            return self.forward_frame_aware(x, y, t, mask=mask, THW=THW, rotary_emb=rotary_emb,
                                            chunk_index=chunk_index, **kwargs)
        B, N, C = x.shape
        feats = {"x_in": x, "x_self_attn": None, "x_cross_attn": None, "x_ffn": None}
        shift_msa, scale_msa, gate_msa, shift_mlp, scale_mlp, gate_mlp = (
            self.scale_shift_table[None] + t.reshape(B, 6, -1)).chunk(6, dim=1)
        attn_kw = {"HW": THW, "rotary_emb": rotary_emb}
        if chunk_index is not None:
            attn_kw["chunk_index"] = chunk_index[:]
        save_kv_cache = kwargs.get("save_kv_cache", None)
        if save_kv_cache is not None:
            attn_kw["save_kv_cache"] = save_kv_cache
        kv_cache = kwargs.get("kv_cache", None)
        if kv_cache is not None:
            attn_kw["kv_cache"] = kv_cache
        x_sa = self.attn(t2i_modulate(self.norm1(x), shift_msa, scale_msa), **attn_kw)
        if kv_cache is not None:
            x_sa, kv_cache = x_sa
        feats["x_self_attn"] = x_sa
        x = x + gate_msa * x_sa
        x = x + self.cross_attn(x, y, mask=mask)
        feats["x_cross_attn"] = x
        mlp_kw = {"HW": THW}
        if chunk_index is not None:
            mlp_kw["chunk_index"] = chunk_index[:]
        if save_kv_cache is not None:
            mlp_kw["save_kv_cache"] = save_kv_cache
        if kv_cache is not None:
            mlp_kw["kv_cache"] = kv_cache
        mlp_out = self.mlp(t2i_modulate(self.norm2(x), shift_mlp, scale_mlp), **mlp_kw)
        if kv_cache is not None:
            mlp_out, kv_cache = mlp_out
        x = x + gate_mlp * mlp_out
        feats["x_ffn"] = x
        if self.block_hook is not None:
            self.block_hook(**feats)
        if kv_cache is not None:
            return x, kv_cache
        return x


# --------------------------------------------------------------------------
# A8: W8A16 quantiser (defined by the benchmark configuration, not by the
# reference, which has no W8A16 code)
# --------------------------------------------------------------------------

W8A16_KEYS = ("attn.qkv.weight", "attn.proj.weight",
              "mlp.inverted_conv.conv.weight", "mlp.point_conv.conv.weight")


def quantize_w8(weight: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor]:
    """Symmetric per-output-channel int8: s_o = absmax_i |W[o, i]| / 127,
    Wq = clamp(round(W / s), -127, 127).  ``weight`` is [out, in, ...];
    returns (int8 [out, in...], fp32 scale [out])."""
    # fp64 intermediates make the result independent of the device's fp32 division
    w = weight.detach().double().flatten(1)
    scale = (w.abs().amax(dim=1) / 127.0).float()
    scale = torch.where(scale > 0, scale, torch.ones_like(scale))
    wq = torch.clamp(torch.round(w / scale.double()[:, None]), -127, 127).to(torch.int8)
    return wq.view_as(weight), scale


def dequantize_w8(wq: torch.Tensor, scale: torch.Tensor, dtype=torch.bfloat16) -> torch.Tensor:
    """The weight the W8A16 GEMM must behave as: (int8.float() * scale) rounded to ``dtype``."""
    shape = [-1] + [1] * (wq.dim() - 1)
    return (wq.float() * scale.float().view(shape)).to(dtype)


def dequantized_block_state(state: dict, dtype=torch.bfloat16) -> dict:
    """Return a copy of a SanaMSBlock state_dict whose four hot-path GEMM
    weights went through quantise -> dequantise (the W8A16 parity target)."""
    out = dict(state)
    for key in W8A16_KEYS:
        wq, s = quantize_w8(state[key])
        out[key] = dequantize_w8(wq, s, dtype)
    return out


# --------------------------------------------------------------------------
# seeded synthetic inputs shared by tests, smoke and bench
# --------------------------------------------------------------------------


def init_block_(block: nn.Module, seed: int = 0) -> nn.Module:
    """Random init used by every benchmark configuration: trunc-normal(std 0.02)
    weights, zero biases, scale_shift_table = randn(6, C)/sqrt(C)."""
    g = torch.Generator().manual_seed(seed)
    with torch.no_grad():
        for name, p in block.named_parameters():
            if name.endswith("scale_shift_table"):
                p.copy_(torch.randn(p.shape, generator=g) / p.shape[-1] ** 0.5)
            elif name.endswith("bias"):
                p.zero_()
            elif "norm" in name:
                p.fill_(1.0)
            else:
                w = torch.empty(p.shape)
                nn.init.trunc_normal_(w, std=0.02, generator=g)
                p.copy_(w)
    return block


def block_inputs(B: int, N: int, C: int, n_text: int = 300, seed: int = 0):
    """x ~ N(0,1) [B,N,C]; y ~ N(0,1) [B,n_text,C]; t ~ 0.02*N(0,1) [B,6C]."""
    g = torch.Generator().manual_seed(seed + 1000)
    x = torch.randn(B, N, C, generator=g)
    y = torch.randn(B, n_text, C, generator=g)
    t = torch.randn(B, 6 * C, generator=g) * 0.02
    return x, y, t
