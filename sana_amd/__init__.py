"""MI355X-native SanaMSBlock hot path: LiteLA linear attention and GLUMBConv
Mix-FFN as drop-in modules over hand-written gfx950 kernels (C ABI in
``include/sana_hip.h``, built by ``python -m sana_amd.build``)."""
from ._lib import LIB_PATH, SanaHipError  # noqa: F401
from .graph import GraphedCall  # noqa: F401
from .modules import (CachedCausalAttention, CachedGLUMBConvTemp, ChunkCausalAttention,  # noqa: F401
                      ChunkGLUMBConvTemp, GLUMBConv, GLUMBConvLinear, GLUMBConvLinearTemp, GLUMBConvTemp, HipLinear, LiteLA, LiteLAReLURope, MultiHeadCrossAttention, SanaMSBlock, SanaVideoMSBlock, StepConditioning, ChunkedLiteLAReLURope, accumulate_kv_cache, quantize_w8)

__all__ = ["LIB_PATH", "SanaHipError", "LiteLA", "LiteLAReLURope", "ChunkCausalAttention", "CachedCausalAttention",
           "accumulate_kv_cache", "GLUMBConv", "GLUMBConvLinear", "GLUMBConvLinearTemp", "GLUMBConvTemp", "ChunkGLUMBConvTemp", "CachedGLUMBConvTemp", "SanaMSBlock", "SanaVideoMSBlock", "ChunkedLiteLAReLURope", "MultiHeadCrossAttention", "HipLinear", "quantize_w8", "GraphedCall", "StepConditioning"]
