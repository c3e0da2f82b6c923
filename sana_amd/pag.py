"""Self-attention processors for perturbed-attention guidance (reference:
diffusion/model/nets/sana_blocks.py:575-717).  The sampler patches one over ``block.attn.forward``
for the guided layers (diffusion/model/dpm_solver.py:486-524) and restores the plain one afterwards:

    block.attn.forward = PAGCFGIdentitySelfAttnProcessorLiteLA(block.attn)

The batch holds [uncond | cond | perturbed] (or [cond | perturbed] without classifier-free
guidance).  The unperturbed part is the attention's own forward; the perturbed part replaces the
attention by the identity, i.e. it is ``proj(v_linear(x))``.

The reference's own processor classes also work unchanged on :class:`sana_amd.LiteLA`
(they only touch ``qkv``, ``q_norm``, ``k_norm``, ``dim``, ``kernel_func``, ``attn_matmul`` and
``proj``); these restatements do the same computation on the token-major kernels without the
channel-major round trip.
"""
from __future__ import annotations

import torch

from .modules import LiteLA, hip_linear


def _identity_attention(attn: LiteLA, x_ptb: torch.Tensor) -> torch.Tensor:
    """proj(x @ Wv^T + bv): sana_blocks.py:615-622."""
    C = x_ptb.shape[-1]
    if attn.qkv.weight is None:
        raise NotImplementedError("perturbed-attention guidance on int8 qkv weights")
    v_weight = attn.qkv.weight[2 * C:3 * C]
    v_bias = None if attn.qkv.bias is None else attn.qkv.bias[2 * C:3 * C]
    return attn.proj(hip_linear(x_ptb, v_weight, v_bias))


class SelfAttnProcessorLiteLA:
    """The plain attention forward as a processor (sana_blocks.py:677-717)."""

    def __init__(self, attn: LiteLA):
        self.attn = attn

    def __call__(self, x, mask=None, HW=None, rotary_emb=None, block_id=None, block_mask=None, **kwargs):
        return type(self.attn).forward(self.attn, x, mask=mask, HW=HW, rotary_emb=rotary_emb)


class PAGIdentitySelfAttnProcessorLiteLA(SelfAttnProcessorLiteLA):
    """[cond | perturbed] (sana_blocks.py:627-674)."""

    def __call__(self, x, mask=None, HW=None, rotary_emb=None, block_id=None, block_mask=None, **kwargs):
        x_org, x_ptb = x.chunk(2)
        out = super().__call__(x_org, mask=mask, HW=HW, rotary_emb=rotary_emb)
        return torch.cat([out, _identity_attention(self.attn, x_ptb)])


class PAGCFGIdentitySelfAttnProcessorLiteLA(SelfAttnProcessorLiteLA):
    """[uncond | cond | perturbed] (sana_blocks.py:575-624)."""

    def __call__(self, x, mask=None, HW=None, rotary_emb=None, block_id=None, block_mask=None, **kwargs):
        x_uncond, x_org, x_ptb = x.chunk(3)
        out = super().__call__(torch.cat([x_uncond, x_org]), mask=mask, HW=HW, rotary_emb=rotary_emb)
        return torch.cat([out, _identity_attention(self.attn, x_ptb)])
