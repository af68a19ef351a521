"""Eager restatement of the triangle-multiplication block and its gradients (CPU, test-only).

Follows ``TriangleMultiplication.forward`` of the reference (megafold/model/megafold.py:461-493) one tensor
expression per statement; ``combined`` and ``to_out[0]`` are the reference's ``LayernormLinear`` modules
(megafold/model/FusedLayernormLinear/fused_layernorm_linear.py:498-545: LayerNorm with eps 1e-5 followed by
``x @ linear_weight + linear_bias`` with ``linear_weight`` stored ``[K, N]``).  Gradients come from autograd on
this expression in float64.
"""
from __future__ import annotations

import torch
import torch.nn.functional as F

EPS = 1e-5  # fused_layernorm_linear.py:368


def triangle_multiplication_forward(x, mask, params, mix="outgoing", dtype=torch.float64):
    """x ``[b, n, n, d]``; mask ``[b, n]`` bool or None; params: dict of tensors named as the reference state dict:

    ``combined.WEIGHT, combined.BIAS [d], combined.linear_weight [d, 5*dh], combined.linear_bias [5*dh],
    to_out.0.WEIGHT, to_out.0.BIAS [dh], to_out.0.linear_weight [dh, d]``.
    Returns the block output ``[b, n, n, d]`` in ``dtype`` (before dropout and the residual add)."""
    P = {k: v.to(dtype) for k, v in params.items()}
    x = x.to(dtype)
    d = x.shape[-1]
    dh = P["to_out.0.WEIGHT"].shape[0]
    combined = F.layer_norm(x, (d,), P["combined.WEIGHT"], P["combined.BIAS"], EPS) @ P["combined.linear_weight"] \
        + P["combined.linear_bias"]                                                         # megafold.py:475
    left_and_right, out_gate = combined[..., :dh * 4], torch.sigmoid(combined[..., dh * 4:])   # megafold.py:476
    left, right = F.glu(left_and_right, dim=-1).chunk(2, dim=-1)                             # megafold.py:477
    if mask is not None:
        pair = (mask[:, :, None] & mask[:, None, :]).unsqueeze(-1).to(dtype)                # megafold.py:470-472, utils/model_utils.py:630-643
        left, right = left * pair, right * pair                                             # megafold.py:479-481
    eq = "bikd,bjkd->bijd" if mix == "outgoing" else "bkjd,bkid->bijd"                      # megafold.py:444-447
    out = torch.einsum(eq, left, right)                                                     # megafold.py:483
    out = F.layer_norm(out, (dh,), P["to_out.0.WEIGHT"], P["to_out.0.BIAS"], EPS) @ P["to_out.0.linear_weight"]
    return out * out_gate                                                                   # megafold.py:491


def triangle_multiplication_forward_backward(x, mask, params, dout, mix="outgoing", dtype=torch.float64):
    """Returns ``(out, dx, {name: dparam})`` by autograd on :func:`triangle_multiplication_forward`."""
    xs = x.detach().to(dtype).requires_grad_(True)
    ps = {k: v.detach().to(dtype).requires_grad_(True) for k, v in params.items()}
    out = triangle_multiplication_forward(xs, mask, ps, mix, dtype)
    grads = torch.autograd.grad(out, [xs] + list(ps.values()), dout.to(dtype))
    return out.detach(), grads[0], dict(zip(ps.keys(), grads[1:]))
