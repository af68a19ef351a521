"""Eager restatement of ``PairwiseBlock.forward`` (megafold/model/megafold.py:726-748) from the oracles of its
five sub-blocks (CPU, test-only).  Parameters are named as in the reference state dict."""
from __future__ import annotations

import torch

from . import transition as ot
from . import triangle_attention as ota
from . import triangle_multiplication as otm


def _sub(params, prefix):
    return {k[len(prefix):]: v for k, v in params.items() if k.startswith(prefix)}


def pairwise_block_forward(x, mask, params, heads, dim_head, dtype=torch.float64):
    x = x.to(dtype)
    x = otm.triangle_multiplication_forward(x, mask, _sub(params, "tri_mult_outgoing."), "outgoing", dtype) + x   # :742
    x = otm.triangle_multiplication_forward(x, mask, _sub(params, "tri_mult_incoming."), "incoming", dtype) + x   # :743
    x = ota.triangle_attention_forward(x, mask, _sub(params, "tri_attn_starting."), heads, dim_head, "starting", dtype) + x  # :744
    x = ota.triangle_attention_forward(x, mask, _sub(params, "tri_attn_ending."), heads, dim_head, "ending", dtype) + x      # :745
    t = _sub(params, "pairwise_transition.")
    # FusedTransition: ff.0 = LayernormLinear(dim, 2*inner, no linear bias), ff.2 = nn.Linear(inner, dim, no bias)
    y = ot.transition_forward(x, t["ff.0.WEIGHT"].to(dtype), t["ff.0.BIAS"].to(dtype), t["ff.0.linear_weight"].to(dtype),
                              t["ff.2.weight"].to(dtype), dtype=dtype)
    return y + x                                                                                                  # :747


def pairwise_block_forward_backward(x, mask, params, dout, heads, dim_head, dtype=torch.float64):
    xs = x.detach().to(dtype).requires_grad_(True)
    ps = {k: v.detach().to(dtype).requires_grad_(True) for k, v in params.items()}
    out = pairwise_block_forward(xs, mask, ps, heads, dim_head, dtype)
    grads = torch.autograd.grad(out, [xs] + list(ps.values()), dout.to(dtype))
    return out.detach(), grads[0], dict(zip(ps.keys(), grads[1:]))
