from .triangle_attention import (Attention, Dropout, PreLayerNormTriangleAttention, TriangleAttention,  # noqa: F401
                                 TriangleAttentionFunction, sigmoid_gate_backward, sigmoid_gate_forward)
