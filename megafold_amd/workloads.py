"""Seeded synthetic inputs for the five benchmark configurations (C1..C5).

Every tensor is drawn on the CPU from one ``torch.Generator`` in a fixed order, so the GPU path and
any CPU checker see identical values; callers move them to the device.
"""
from __future__ import annotations

import math

import torch


def _randn(gen, *shape):
    return torch.randn(*shape, generator=gen, dtype=torch.float32)


def evoattention_inputs(B, N, S, H, D, n_masked, dtype=torch.bfloat16, seed=0, bias_dtype=torch.float32,
                        mask_value=float("-inf")):
    """q, k, v ``[B, N, S, H, D]`` ~ N(0, 1); pair bias ``[B, 1, H, S, S]`` ~ N(0, 1); additive key mask
    ``[B, N, 1, 1, S]`` with the last ``n_masked`` keys set to ``mask_value``; dO ~ N(0, 1).
    Draw order: q, k, v, bias, dO."""
    gen = torch.Generator().manual_seed(seed)
    q = _randn(gen, B, N, S, H, D).to(dtype)
    k = _randn(gen, B, N, S, H, D).to(dtype)
    v = _randn(gen, B, N, S, H, D).to(dtype)
    bias = _randn(gen, B, 1, H, S, S).to(bias_dtype)
    dO = _randn(gen, B, N, S, H, D).to(dtype)
    mask = torch.zeros(B, N, 1, 1, S, dtype=torch.float32)
    if n_masked:
        mask[..., S - n_masked:] = mask_value
    return {"q": q, "k": k, "v": v, "bias": bias, "mask": mask, "dO": dO}


def config1():
    """C1: forward only, fp32, [B=1, N=64, H=4, S=64, D=32], last 8 keys masked with -inf."""
    return evoattention_inputs(1, 64, 64, 4, 32, 8, dtype=torch.float32, seed=0)


def config2(dtype=torch.bfloat16):
    """C2: triangle attention fwd+bwd, [1, 384, 384, 4, 32], last 38 of 384 keys padded."""
    return evoattention_inputs(1, 384, 384, 4, 32, 38, dtype=dtype, seed=0)


def config5(dtype=torch.bfloat16):
    """C5: long-crop triangle attention, [1, 768, 768, 4, 32], last 96 of 768 keys padded."""
    return evoattention_inputs(1, 768, 768, 4, 32, 96, dtype=dtype, seed=0)


def lnlinear_inputs(M_shape=(1, 384, 384), K=128, N=512, dtype=torch.bfloat16, seed=0, linear_bias=True):
    """C3: x ~ N(0,1); gamma ~ N(1, 0.1), beta ~ N(0, 0.1); W [K, N] ~ N(0, 1/K); linear bias zeros;
    dY ~ N(0, 1).  Draw order: x, gamma, beta, W, dY."""
    gen = torch.Generator().manual_seed(seed)
    x = _randn(gen, *M_shape, K).to(dtype)
    gamma = (1.0 + 0.1 * _randn(gen, K)).to(dtype)
    beta = (0.1 * _randn(gen, K)).to(dtype)
    W = (_randn(gen, K, N) / math.sqrt(K)).to(dtype)
    dY = _randn(gen, *M_shape, N).to(dtype)
    b = torch.zeros(N, dtype=dtype) if linear_bias else None
    return {"x": x, "gamma": gamma, "beta": beta, "W": W, "b": b, "dY": dY}


def transition_inputs(M_shape=(1, 384, 384), dim=128, expansion_factor=4, dtype=torch.bfloat16, seed=0):
    """C4: x ~ N(0,1); LN affine as C3; W1 [dim, 2*di] ~ N(0, 1/dim); W2 (nn.Linear weight [dim, di])
    ~ N(0, 1/di); dY ~ N(0, 1) shaped like x.  Draw order: x, gamma, beta, W1, W2, dY."""
    di = int(dim * expansion_factor)
    gen = torch.Generator().manual_seed(seed)
    x = _randn(gen, *M_shape, dim).to(dtype)
    gamma = (1.0 + 0.1 * _randn(gen, dim)).to(dtype)
    beta = (0.1 * _randn(gen, dim)).to(dtype)
    W1 = (_randn(gen, dim, 2 * di) / math.sqrt(dim)).to(dtype)
    W2 = (_randn(gen, dim, di) / math.sqrt(di)).to(dtype)
    dY = _randn(gen, *M_shape, dim).to(dtype)
    return {"x": x, "gamma": gamma, "beta": beta, "W1": W1, "W2": W2, "dY": dY}


def _pair_mask(b, n, n_masked):
    if not n_masked:
        return None
    mask = torch.ones(b, n, dtype=torch.bool)
    mask[:, n - n_masked:] = False
    return mask


def triangle_attention_inputs(b=1, n=12, dim=64, heads=2, dim_head=16, n_masked=3, dtype=torch.float32, seed=0):
    """Pair tensor ``[b, n, n, dim]``, key mask ``[b, n]`` (last ``n_masked`` positions off), upstream gradient and
    the parameters of ``PreLayerNorm(TriangleAttention)`` under the reference's state-dict names.
    Draw order: x, dout, then the parameters in the order of the dict."""
    gen = torch.Generator().manual_seed(seed)
    inner = heads * dim_head
    x = _randn(gen, b, n, n, dim).to(dtype)
    dout = _randn(gen, b, n, n, dim).to(dtype)
    params = {
        "norm.weight": 1 + 0.1 * _randn(gen, dim), "norm.bias": 0.1 * _randn(gen, dim),
        "fn.to_attn_bias.0.weight": _randn(gen, heads, dim) * dim ** -0.5,
        "fn.attn.to_q.weight": _randn(gen, inner, dim) * dim ** -0.5, "fn.attn.to_q.bias": 0.1 * _randn(gen, inner),
        "fn.attn.to_kv.weight": _randn(gen, 2 * inner, dim) * dim ** -0.5,
        "fn.attn.to_out.weight": _randn(gen, dim, inner) * inner ** -0.5,
        "fn.attn.to_gates.weight": _randn(gen, inner, dim) * dim ** -0.5,
        "fn.attn.to_gates.bias": 0.1 * _randn(gen, inner) - 1.0,
    }
    params = {k: v.to(dtype) for k, v in params.items()}
    return {"x": x, "dout": dout, "mask": _pair_mask(b, n, n_masked), "params": params}


def triangle_multiplication_inputs(b=1, n=12, dim=64, n_masked=2, dtype=torch.float32, seed=0):
    """As :func:`triangle_attention_inputs` for ``TriangleMultiplication`` (``dim_hidden = dim``)."""
    gen = torch.Generator().manual_seed(seed)
    x = _randn(gen, b, n, n, dim).to(dtype)
    dout = _randn(gen, b, n, n, dim).to(dtype)
    params = {
        "combined.WEIGHT": 1 + 0.1 * _randn(gen, dim), "combined.BIAS": 0.1 * _randn(gen, dim),
        "combined.linear_weight": _randn(gen, dim, 5 * dim) * dim ** -0.5,
        "combined.linear_bias": 0.1 * _randn(gen, 5 * dim),
        "to_out.0.WEIGHT": 1 + 0.1 * _randn(gen, dim), "to_out.0.BIAS": 0.1 * _randn(gen, dim),
        "to_out.0.linear_weight": _randn(gen, dim, dim) * dim ** -0.5,
    }
    params = {k: v.to(dtype) for k, v in params.items()}
    return {"x": x, "dout": dout, "mask": _pair_mask(b, n, n_masked), "params": params}
