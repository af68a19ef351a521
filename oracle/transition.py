"""Eager restatement of SwiGLU and the Transition block (CPU, test-only).

``SwiGLU: x, gates = chunk(2, -1); silu(gates) * x`` and
``Transition: LayerNorm -> Linear(dim, 2*di, no bias) -> SwiGLU -> Linear(di, dim, no bias)``
(reference: benchmarks/transition_speed.py:8-39; kernel form fused_transition.py:22-24; derivative
fused_transition.py:44-47).
"""
from __future__ import annotations

import torch

from .layernorm_linear import layernorm_linear_forward


def swiglu_forward(u: torch.Tensor, dtype=torch.float32) -> torch.Tensor:
    a, g = u.to(dtype).chunk(2, dim=-1)  # gate is the SECOND half (transition_speed.py:38-39)
    return g * torch.sigmoid(g) * a


def swiglu_backward(dy: torch.Tensor, u: torch.Tensor, dtype=torch.float32) -> torch.Tensor:
    a, g = u.to(dtype).chunk(2, dim=-1)
    dy = dy.to(dtype)
    sig = torch.sigmoid(g)
    silu = g * sig
    da = dy * silu                                  # fused_transition.py:46
    dg = dy * (silu * (1 - sig) + sig) * a          # fused_transition.py:47
    return torch.cat([da, dg], dim=-1)


def ln_swiglu_forward(x, gamma, beta, W1, dtype=torch.float32) -> torch.Tensor:
    """FusedTransition.ff[0:2]: LayernormLinear(dim, 2*di, no linear bias) then SwiGLU."""
    return swiglu_forward(layernorm_linear_forward(x, gamma, beta, W1, None, dtype=dtype), dtype)


def transition_forward(x, gamma, beta, W1, W2, dtype=torch.float32) -> torch.Tensor:
    """W1: [dim, 2*di] (``linear_weight`` layout), W2: ``nn.Linear(di, dim).weight`` = [dim, di]."""
    return ln_swiglu_forward(x, gamma, beta, W1, dtype) @ W2.to(dtype).t()
