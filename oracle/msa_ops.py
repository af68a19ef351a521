"""Eager restatements of the two MSA-module operators and their gradients (CPU, test-only).

One tensor expression per reference statement:

* ``MSAPairWeightedAveraging.forward``  megafold/model/megafold.py:862-902 (Algorithm 10)
  ``values, gates = LayernormLinear(msa) -> "b s n (gv h d) -> gv b h s n d"``; ``gates.sigmoid()``;
  ``b = LayernormLinear(pairwise) -> "b i j h -> b h i j"``; masked_fill of masked keys ``j``; softmax over ``j``;
  ``einsum "b h i j, b h s j d -> b h s i d"``; ``out * gates``; ``"b h s n d -> b s n (h d)"``; ``LinearNoBias``
* ``OuterProductMean.forward``          megafold/model/megafold.py:764-824 (Algorithm 9)
  ``a, b = LayernormLinear(msa).chunk(2)``; MSA-row mask on both; ``einsum "b s i d, b s j e -> b i j d e"``;
  divide by the number of kept MSA rows (clamped at eps) or by ``s``; flatten ``(d e)``; pair mask; ``Linear``
* ``LayernormLinear``  megafold/model/FusedLayernormLinear/fused_layernorm_linear.py:498-545
  ``LayerNorm(x; WEIGHT, BIAS, eps 1e-5) @ linear_weight`` with ``linear_weight`` stored ``[K, N]``

Masked keys get -inf where the reference fills with the most negative finite value (megafold.py:886-888): the
same weights whenever at least one key is kept.  Gradients come from autograd on these expressions in float64.

This module is test infrastructure: only tests, the smoke check and the benchmark's CPU leg may import it.
"""
from __future__ import annotations

import torch
import torch.nn.functional as F

EPS = 1e-5


def _ln_linear(x, P, prefix):
    k = x.shape[-1]
    return torch.matmul(F.layer_norm(x, (k,), P[prefix + "WEIGHT"], P[prefix + "BIAS"], EPS), P[prefix + "linear_weight"])


def msa_pair_weighted_averaging_forward(msa, pairwise, params, heads, dim_head, mask=None, dtype=torch.float64):
    """msa ``[b, s, n, dm]``; pairwise ``[b, n, n, dp]``; mask ``[b, n]`` bool or None; params named as the
    reference state dict: ``msa_to_values_and_gates.0.{WEIGHT,BIAS,linear_weight}``,
    ``pairwise_repr_to_attn.0.{WEIGHT,BIAS,linear_weight}``, ``to_out.1.weight [dm, h*dh]``.  Returns ``[b, s, n, dm]``
    (before dropout)."""
    P = {k: v.to(dtype) for k, v in params.items()}
    msa, pairwise = msa.to(dtype), pairwise.to(dtype)
    b, s, n, _ = msa.shape
    vg = _ln_linear(msa, P, "msa_to_values_and_gates.0.")                                # megafold.py:845, 879
    vg = vg.reshape(b, s, n, 2, heads, dim_head).permute(3, 0, 4, 1, 2, 5)               # "b s n (gv h d) -> gv b h s n d"  megafold.py:846
    values, gates = vg[0], torch.sigmoid(vg[1])                                          # megafold.py:879-880
    bias = _ln_linear(pairwise, P, "pairwise_repr_to_attn.0.").permute(0, 3, 1, 2)       # "b i j h -> b h i j"  megafold.py:852-853, 884
    if mask is not None:
        bias = bias.masked_fill(~mask[:, None, None, :], float("-inf"))                  # megafold.py:886-888
    weights = torch.softmax(bias, dim=-1)                                                # megafold.py:892
    out = torch.einsum("bhij,bhsjd->bhsid", weights, values)                             # megafold.py:896
    out = out * gates                                                                    # megafold.py:898
    out = out.permute(0, 2, 3, 1, 4).reshape(b, s, n, heads * dim_head)                  # "b h s n d -> b s n (h d)"  megafold.py:857
    return F.linear(out, P["to_out.1.weight"])                                           # megafold.py:858, 902


def outer_product_mean_forward(msa, params, mask=None, msa_mask=None, eps=1e-5, dtype=torch.float64):
    """msa ``[b, s, n, dm]``; mask ``[b, n]`` bool or None; msa_mask ``[b, s]`` bool or None; params:
    ``to_hidden.{WEIGHT,BIAS,linear_weight [dm, 2*dh]}``, ``to_pairwise_repr.weight [dp, dh*dh]``, ``to_pairwise_repr.bias``.
    Returns ``[b, n, n, dp]``."""
    P = {k: v.to(dtype) for k, v in params.items()}
    msa = msa.to(dtype)
    s = msa.shape[1]
    a, bb = _ln_linear(msa, P, "to_hidden.").chunk(2, dim=-1)                            # megafold.py:784
    if msa_mask is not None:
        m = msa_mask.to(dtype)[:, :, None, None]
        a, bb = a * m, bb * m                                                            # megafold.py:792-793
    outer = torch.einsum("bsid,bsje->bijde", a, bb)                                      # megafold.py:795, 807
    if msa_mask is not None:
        num = msa_mask.to(dtype).sum(dim=-1).clamp(min=eps)[:, None, None, None, None]   # megafold.py:797-804
    else:
        num = s                                                                          # megafold.py:806-808
    outer = (outer / num).flatten(-2)                                                    # megafold.py:812 "... d e -> ... (d e)"
    if mask is not None:
        pair = (mask[:, :, None] & mask[:, None, :]).to(dtype)[..., None]                # megafold.py:816-821
        outer = outer * pair
    return F.linear(outer, P["to_pairwise_repr.weight"], P.get("to_pairwise_repr.bias"))  # megafold.py:823


def _with_grads(fn, tensors, params, dout, dtype):
    ts = [t.detach().to(dtype).requires_grad_(True) for t in tensors]
    ps = {k: v.detach().to(dtype).requires_grad_(True) for k, v in params.items()}
    out = fn(ts, ps)
    leaves = ts + list(ps.values())
    grads = torch.autograd.grad(out, leaves, dout.to(dtype), allow_unused=True)
    grads = [torch.zeros_like(t) if g is None else g for g, t in zip(grads, leaves)]
    return out.detach(), grads[:len(ts)], dict(zip(ps.keys(), grads[len(ts):]))


def msa_pair_weighted_averaging_forward_backward(msa, pairwise, params, dout, heads, dim_head, mask=None,
                                                 dtype=torch.float64):
    """Returns ``(out, dmsa, dpairwise, {name: dparam})``."""
    out, (dm, dz), dp = _with_grads(
        lambda t, p: msa_pair_weighted_averaging_forward(t[0], t[1], p, heads, dim_head, mask, dtype),
        [msa, pairwise], params, dout, dtype)
    return out, dm, dz, dp


def outer_product_mean_forward_backward(msa, params, dout, mask=None, msa_mask=None, eps=1e-5, dtype=torch.float64):
    """Returns ``(out, dmsa, {name: dparam})``."""
    out, (dm,), dp = _with_grads(
        lambda t, p: outer_product_mean_forward(t[0], p, mask, msa_mask, eps, dtype), [msa], params, dout, dtype)
    return out, dm, dp
