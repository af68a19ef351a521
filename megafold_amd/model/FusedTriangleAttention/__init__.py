from .triangle_attention import (Attention, Dropout, PreLayerNormTriangleAttention, TriangleAttention,  # noqa: F401
                                 TriangleAttentionFunction)
