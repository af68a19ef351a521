"""Eager restatement of pair-biased, key-masked attention and its gradients (CPU, test-only).

Forward follows tests/test_evoattention.py:45-56 of the reference::

    ref_P = matmul(Q * scale, K^T) + pair_bias + res_mask ; softmax(ref_P.float()) ; @ V

in the layout of the operator API: Q, K, V ``[B, N, S, H, D]``, res_mask ``[B, N, 1, 1, S]`` (additive),
pair_bias ``[B, 1, H, S, S]``.  Backward follows the closed forms the reference kernels implement
(evoattention.py:298 delta, 461-462 / 653-657 dP and dS, 649 dV, 470 dQ, 661 dK, 465 dBias).
"""
from __future__ import annotations

import torch


def additive_mask(res_mask: torch.Tensor, dtype=torch.float32) -> torch.Tensor:
    """Float masks are additive as in the reference kernel (evoattention.py:66).  A bool mask is a
    keep-mask, True -> 0 and False -> -inf (the form of benchmarks/evoattention_speed.py:10-16)."""
    if res_mask.dtype == torch.bool:
        out = torch.zeros(res_mask.shape, dtype=dtype)
        return out.masked_fill(~res_mask, float("-inf"))
    return res_mask.to(dtype)


def logits(Q, K, res_mask, pair_bias, scale=None, dtype=torch.float32) -> torch.Tensor:
    """z[b, n, h, i, j] = scale * <Q[b,n,i,h,:], K[b,n,j,h,:]> + bias[b,0,h,i,j] + mask[b,n,0,0,j]."""
    D = Q.shape[-1]
    scale = D ** -0.5 if scale is None else scale
    q = Q.to(dtype).transpose(-2, -3)  # [B, N, H, S, D]   (tests/test_evoattention.py:45-47)
    k = K.to(dtype).transpose(-2, -3)
    z = torch.matmul(q * scale, k.transpose(-1, -2))  # [B, N, H, S, S]
    return z + pair_bias.to(dtype) + additive_mask(res_mask, dtype)


def evo_attention_forward(Q, K, V, res_mask, pair_bias, scale=None, dtype=torch.float32):
    """Returns (O ``[B, N, S, H, D]``, LSE ``[B, N, H, S]``), both in ``dtype``.

    A query row whose logits are all -inf is defined as O = 0, LSE = -inf (the reference kernel would
    produce NaN there, evoattention.py:72-81)."""
    z = logits(Q, K, res_mask, pair_bias, scale, dtype)
    lse = torch.logsumexp(z, dim=-1)
    dead = torch.isneginf(lse)
    p = torch.exp(z - lse.masked_fill(dead, 0.0).unsqueeze(-1))
    p = p.masked_fill(dead.unsqueeze(-1), 0.0)
    o = torch.matmul(p, V.to(dtype).transpose(-2, -3))  # [B, N, H, S, D]
    return o.transpose(-2, -3).contiguous(), lse


def evo_attention_backward(dO, Q, K, V, res_mask, pair_bias, scale=None, dtype=torch.float32):
    """Closed-form gradients (dQ, dK, dV in ``[B, N, S, H, D]``; dBias ``[B, 1, H, S, S]``)."""
    D = Q.shape[-1]
    scale = D ** -0.5 if scale is None else scale
    z = logits(Q, K, res_mask, pair_bias, scale, dtype)
    lse = torch.logsumexp(z, dim=-1)
    dead = torch.isneginf(lse)
    p = torch.exp(z - lse.masked_fill(dead, 0.0).unsqueeze(-1)).masked_fill(dead.unsqueeze(-1), 0.0)
    q = Q.to(dtype).transpose(-2, -3)
    k = K.to(dtype).transpose(-2, -3)
    v = V.to(dtype).transpose(-2, -3)
    do = dO.to(dtype).transpose(-2, -3)
    o = torch.matmul(p, v)
    delta = (do * o).sum(-1, keepdim=True)              # evoattention.py:298
    dp = torch.matmul(do, v.transpose(-1, -2))          # evoattention.py:461
    ds = p * (dp - delta)                               # evoattention.py:462
    dv = torch.matmul(p.transpose(-1, -2), do)          # evoattention.py:649
    dq = torch.matmul(ds, k) * scale                    # evoattention.py:470
    dk = torch.matmul(ds.transpose(-1, -2), q) * scale  # evoattention.py:661
    dbias = ds.sum(dim=1, keepdim=True)                 # evoattention.py:465 (sum over N)
    tr = lambda t: t.transpose(-2, -3).contiguous()
    return tr(dq), tr(dk), tr(dv), dbias


def evo_attention_chunked(Q, K, V, res_mask, pair_bias, dO=None, chunk=64, dtype=torch.float32):
    """Same results, walking over N in chunks so the [N, H, S, S] scores are never resident at once
    (N is an independent batch axis; dBias is summed over the chunks)."""
    B, N = Q.shape[:2]
    outs, grads, dbias = [], [], None
    mask = res_mask.expand(B, N, 1, 1, res_mask.shape[-1])
    for n0 in range(0, N, chunk):
        sl = slice(n0, min(N, n0 + chunk))
        o, _ = evo_attention_forward(Q[:, sl], K[:, sl], V[:, sl], mask[:, sl], pair_bias, dtype=dtype)
        outs.append(o)
        if dO is not None:
            dq, dk, dv, db = evo_attention_backward(dO[:, sl], Q[:, sl], K[:, sl], V[:, sl], mask[:, sl], pair_bias,
                                                    dtype=dtype)
            grads.append((dq, dk, dv))
            dbias = db if dbias is None else dbias + db
    O = torch.cat(outs, dim=1)
    if dO is None:
        return O
    dQ, dK, dV = (torch.cat([g[i] for g in grads], dim=1) for i in range(3))
    return O, dQ, dK, dV, dbias
