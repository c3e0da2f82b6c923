"""MI355X-native SanaMSBlock hot path: LiteLA linear attention and GLUMBConv
Mix-FFN as drop-in modules over hand-written gfx950 kernels (C ABI in
``include/sana_hip.h``, built by ``python -m sana_amd.build``)."""
from ._lib import LIB_PATH, SanaHipError  # noqa: F401
from .modules import (CachedCausalAttention, ChunkCausalAttention, GLUMBConv, HipLinear, LiteLA,  # noqa: F401
                      LiteLAReLURope, MultiHeadCrossAttention, SanaMSBlock, accumulate_kv_cache, quantize_w8)

__all__ = ["LIB_PATH", "SanaHipError", "LiteLA", "LiteLAReLURope", "ChunkCausalAttention", "CachedCausalAttention",
           "accumulate_kv_cache", "GLUMBConv", "SanaMSBlock", "MultiHeadCrossAttention", "HipLinear", "quantize_w8"]
