"""Eager restatement of LayerNorm -> Linear and its gradients (CPU, test-only).

Forward: ``F.linear(F.layer_norm(X, (K,), gamma, beta, 1e-5), W^T, b)`` with ``W`` stored ``[K, N]``
(reference: tests/test_layernormlinear.py:17-22 and the fallback at fused_layernorm_linear.py:541).
Backward: the closed forms of fused_layernorm_linear.py:273-306, 345 written with explicit sums.
"""
from __future__ import annotations

import torch

EPS = 1e-5  # literal in the reference kernel launch, fused_layernorm_linear.py:368


def layernorm_stats(x: torch.Tensor, eps: float = EPS):
    """Row mean and 1/sqrt(biased variance + eps) (fused_layernorm_linear.py:134-137)."""
    mean = x.mean(-1, keepdim=True)
    var = ((x - mean) ** 2).mean(-1, keepdim=True)
    return mean, torch.rsqrt(var + eps)


def layernorm_linear_forward(x, gamma, beta, W, b=None, eps: float = EPS, dtype=torch.float32):
    x, gamma, W = x.to(dtype), gamma.to(dtype), W.to(dtype)
    mean, rstd = layernorm_stats(x, eps)
    y = (x - mean) * rstd * gamma
    if beta is not None:
        y = y + beta.to(dtype)
    out = y @ W
    if b is not None:
        out = out + b.to(dtype)
    return out


def layernorm_linear_backward(dout, x, gamma, beta, W, eps: float = EPS, dtype=torch.float32):
    """Returns dx, dW [K, N], db [N], dgamma [K], dbeta [K]."""
    K = x.shape[-1]
    x2 = x.to(dtype).reshape(-1, K)
    g = dout.to(dtype).reshape(x2.shape[0], -1)
    gamma, W = gamma.to(dtype), W.to(dtype)
    mean, rstd = layernorm_stats(x2, eps)
    xhat = (x2 - mean) * rstd
    y = xhat * gamma + (beta.to(dtype) if beta is not None else 0.0)
    dy = g @ W.t()                                       # fused_layernorm_linear.py:281
    dW = y.t() @ g                                       # :277-278
    db = g.sum(0)                                        # :467
    dgamma = (dy * xhat).sum(0)                          # :298-303
    dbeta = dy.sum(0)                                    # :304-306
    w = dy * gamma                                       # :288
    c1 = (xhat * w).mean(-1, keepdim=True)               # :291-296
    c2 = w.mean(-1, keepdim=True)
    dx = (w - (xhat * c1 + c2)) * rstd                   # :345
    return dx.reshape(x.shape), dW, db, dgamma, dbeta
