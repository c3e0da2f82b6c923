"""Checkpoint keys of the DiT blocks: the reference's own layout and the diffusers layout.

A released Sana checkpoint is ``{"state_dict": {...}}`` (or the bare dict) whose block parameters are
named ``blocks.{i}.<module>.<param>`` -- exactly the ``state_dict`` keys of
:class:`sana_amd.SanaMSBlock`.  ``tools/convert_scripts/convert_sana_to_diffusers.py:152-222`` of the
reference renames them for diffusers (and splits the fused qkv / kv weights); both directions are
restated here for the block keys only (embedders, final layer and VAE are outside this package).
"""
from __future__ import annotations

from typing import Dict, Iterable, List, Sequence

import torch

_PLAIN = [  # (reference suffix, diffusers suffix)
    ("scale_shift_table", "scale_shift_table"),
    ("attn.proj.weight", "attn1.to_out.0.weight"),
    ("attn.proj.bias", "attn1.to_out.0.bias"),
    ("mlp.inverted_conv.conv.weight", "ff.conv_inverted.weight"),
    ("mlp.inverted_conv.conv.bias", "ff.conv_inverted.bias"),
    ("mlp.depth_conv.conv.weight", "ff.conv_depth.weight"),
    ("mlp.depth_conv.conv.bias", "ff.conv_depth.bias"),
    ("mlp.point_conv.conv.weight", "ff.conv_point.weight"),
    ("cross_attn.q_linear.weight", "attn2.to_q.weight"),
    ("cross_attn.q_linear.bias", "attn2.to_q.bias"),
    ("cross_attn.proj.weight", "attn2.to_out.0.weight"),
    ("cross_attn.proj.bias", "attn2.to_out.0.bias"),
]
_QK_NORM = [
    ("attn.q_norm.weight", "attn1.norm_q.weight"),
    ("attn.k_norm.weight", "attn1.norm_k.weight"),
    ("cross_attn.q_norm.weight", "attn2.norm_q.weight"),
    ("cross_attn.k_norm.weight", "attn2.norm_k.weight"),
]


def unwrap(checkpoint: dict) -> Dict[str, torch.Tensor]:
    """``{"state_dict": sd, ...}`` -> sd; a bare state dict is returned as is."""
    sd = checkpoint.get("state_dict", checkpoint)
    if not isinstance(sd, dict):
        raise TypeError("not a checkpoint dictionary")
    return sd


def block_count(state_dict: Dict[str, torch.Tensor], prefix: str = "blocks.") -> int:
    idx = {int(k[len(prefix):].split(".", 1)[0]) for k in state_dict if k.startswith(prefix)}
    if idx != set(range(len(idx))):
        raise KeyError(f"block indices under {prefix!r} are not 0..n-1: {sorted(idx)}")
    return len(idx)


def load_blocks(blocks: Sequence[torch.nn.Module], checkpoint: dict, prefix: str = "blocks.") -> None:
    """Load ``blocks.{i}.*`` of a reference-format checkpoint into ``blocks[i]`` (strict)."""
    sd = unwrap(checkpoint)
    n = block_count(sd, prefix)
    if n != len(blocks):
        raise KeyError(f"checkpoint has {n} blocks, the model {len(blocks)}")
    for i, blk in enumerate(blocks):
        p = f"{prefix}{i}."
        blk.load_state_dict({k[len(p):]: v for k, v in sd.items() if k.startswith(p)}, strict=True)


def blocks_state_dict(blocks: Iterable[torch.nn.Module], prefix: str = "blocks.") -> Dict[str, torch.Tensor]:
    """The reference-format keys of a list of blocks."""
    out = {}
    for i, blk in enumerate(blocks):
        for k, v in blk.state_dict().items():
            out[f"{prefix}{i}.{k}"] = v
    return out


_FFN_POINTWISE = ("inverted_conv", "point_conv")


def ffn_conv_to_linear(state_dict: Dict[str, torch.Tensor]) -> Dict[str, torch.Tensor]:
    """Keys of ``ffn_type="glumbconv"`` -> ``ffn_type="glumbconv_linear"``: ``<pointwise>.conv.weight``
    [out, in, 1, 1] -> ``<pointwise>.linear.weight`` [out, in], biases renamed (the mapping stated at
    basic_modules_linear.py:142-146).  Other keys pass through; tensors are views, not copies."""
    out = {}
    for k, v in unwrap(state_dict).items():
        for base in _FFN_POINTWISE:
            tag = base + ".conv."
            if tag in k:
                k = k.replace(tag, base + ".linear.")
                if k.endswith("weight"):
                    if v.dim() != 4 or v.shape[2:] != (1, 1):
                        raise ValueError(f"{k}: expected a 1x1 convolution weight, got {tuple(v.shape)}")
                    v = v[:, :, 0, 0]
        out[k] = v
    return out


def ffn_linear_to_conv(state_dict: Dict[str, torch.Tensor]) -> Dict[str, torch.Tensor]:
    """The inverse of :func:`ffn_conv_to_linear`."""
    out = {}
    for k, v in unwrap(state_dict).items():
        for base in _FFN_POINTWISE:
            tag = base + ".linear."
            if tag in k:
                k = k.replace(tag, base + ".conv.")
                if k.endswith("weight"):
                    if v.dim() != 2:
                        raise ValueError(f"{k}: expected a linear weight, got {tuple(v.shape)}")
                    v = v[:, :, None, None]
        out[k] = v
    return out


def to_diffusers(state_dict: Dict[str, torch.Tensor], prefix: str = "blocks.") -> Dict[str, torch.Tensor]:
    """Block keys of a reference state dict -> ``transformer_blocks.{i}.*`` (convert_sana_to_diffusers.py:152-222)."""
    sd = unwrap(state_dict)
    out: Dict[str, torch.Tensor] = {}
    for i in range(block_count(sd, prefix)):
        src, dst = f"{prefix}{i}.", f"transformer_blocks.{i}."
        pairs: List = list(_PLAIN)
        if src + "attn.q_norm.weight" in sd:
            pairs += [p for p in _QK_NORM if src + p[0] in sd]
        for a, b in pairs:
            out[dst + b] = sd[src + a]
        q, k, v = torch.chunk(sd[src + "attn.qkv.weight"], 3, dim=0)
        out[dst + "attn1.to_q.weight"], out[dst + "attn1.to_k.weight"], out[dst + "attn1.to_v.weight"] = q, k, v
        k, v = torch.chunk(sd[src + "cross_attn.kv_linear.weight"], 2, dim=0)
        out[dst + "attn2.to_k.weight"], out[dst + "attn2.to_v.weight"] = k, v
        kb, vb = torch.chunk(sd[src + "cross_attn.kv_linear.bias"], 2, dim=0)
        out[dst + "attn2.to_k.bias"], out[dst + "attn2.to_v.bias"] = kb, vb
    return out


def from_diffusers(state_dict: Dict[str, torch.Tensor], prefix: str = "blocks.") -> Dict[str, torch.Tensor]:
    """The inverse of :func:`to_diffusers` for the block keys."""
    n = block_count(state_dict, "transformer_blocks.")
    out: Dict[str, torch.Tensor] = {}
    for i in range(n):
        src, dst = f"transformer_blocks.{i}.", f"{prefix}{i}."
        for a, b in _PLAIN + [p for p in _QK_NORM if src + p[1] in state_dict]:
            out[dst + a] = state_dict[src + b]
        out[dst + "attn.qkv.weight"] = torch.cat([state_dict[src + f"attn1.to_{n_}.weight"] for n_ in "qkv"], dim=0)
        out[dst + "cross_attn.kv_linear.weight"] = torch.cat(
            [state_dict[src + "attn2.to_k.weight"], state_dict[src + "attn2.to_v.weight"]], dim=0)
        out[dst + "cross_attn.kv_linear.bias"] = torch.cat(
            [state_dict[src + "attn2.to_k.bias"], state_dict[src + "attn2.to_v.bias"]], dim=0)
    return out
