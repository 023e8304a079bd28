"""MI355X-native CASTLE attention (causal attention with lookahead keys).

`Castle` and `Cache` mirror lucidrains/lookahead-keys-attention's public names
(lookahead_keys_attention/__init__.py:1-3, lookahead_keys_attention.py:26,41); the
operators run hand-written HIP kernels for gfx950 through the C ABI in include/castle_hip.h.
"""
from .castle import Castle, Cache
from .ops import castle_attention_hip, castle_attention_packed, castle_decode_step_hip
from .lm import CastleLM, GraphedDecoder

__all__ = ["Castle", "Cache", "CastleLM", "GraphedDecoder", "castle_attention_hip", "castle_attention_packed", "castle_decode_step_hip"]
