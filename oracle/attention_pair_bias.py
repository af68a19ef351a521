"""Eager restatement of single-representation attention with pair bias and its gradients (CPU, test-only).

Follows the reference modules literally, one tensor expression per reference statement, full (not windowed)
form only:

* ``AttentionPairBias.forward``  megafold/model/megafold.py:537-591   ``attn_bias = to_attn_bias(pairwise) + attn_bias``
  with ``to_attn_bias = LayernormLinear(dim_pairwise, heads, no bias) ; "b ... h -> b h ..."`` (megafold.py:530-534),
  then ``attn(single_repr, attn_bias=..., mask=...)``
* ``LayernormLinear``            megafold/model/FusedLayernormLinear/fused_layernorm_linear.py:498-545
  ``LayerNorm(x; WEIGHT, BIAS, eps 1e-5) @ linear_weight`` with ``linear_weight`` stored ``[K, N]``
* ``Attention.forward``          megafold/model/attention.py:158-209  q = to_q(x); k, v = to_kv(x).chunk(2);
  split heads ``"b n (h d) -> b h n d"``; attend; merge heads; ``out * sigmoid(to_gates(x))``; ``to_out``
* ``Attend.forward`` default path megafold/model/attention.py:498-537  softmax(q k^T * d^-0.5 + bias, masked) v

Masked keys get -inf where the reference fills with the most negative finite value (attention.py:524): the
same weights whenever a row keeps at least one key; a row that keeps none attends to nothing here.
Gradients come from autograd on this expression in float64.

This module is test infrastructure: only tests, the smoke check and the benchmark's CPU leg may import it.
"""
from __future__ import annotations

import torch
import torch.nn.functional as F

EPS = 1e-5


def attention_pair_bias_forward(single, pairwise, params, heads, dim_head, mask=None, attn_bias=None,
                                dtype=torch.float64):
    """single ``[b, n, ds]``; pairwise ``[b, n, n, dp]``; mask ``[b, n]`` bool (True = keep) or None; attn_bias
    ``[b, n, n]`` or None; params named as the reference state dict of ``AttentionPairBias``:

    ``to_attn_bias.0.WEIGHT [dp], to_attn_bias.0.BIAS [dp], to_attn_bias.0.linear_weight [dp, h], attn.to_q.weight
    [h*dh, ds], attn.to_q.bias, attn.to_kv.weight [2*h*dh, ds], attn.to_gates.weight, attn.to_gates.bias,
    attn.to_out.weight [ds, h*dh]``.  Returns ``[b, n, ds]`` in ``dtype``."""
    P = {k: v.to(dtype) for k, v in params.items()}
    single, pairwise = single.to(dtype), pairwise.to(dtype)
    b, n, _ = single.shape
    dp = pairwise.shape[-1]
    pn = F.layer_norm(pairwise, (dp,), P["to_attn_bias.0.WEIGHT"], P["to_attn_bias.0.BIAS"], EPS)
    bias = torch.matmul(pn, P["to_attn_bias.0.linear_weight"]).permute(0, 3, 1, 2)       # [b, h, i, j]  megafold.py:530-534, 588
    if attn_bias is not None:
        bias = bias + attn_bias.to(dtype)[:, None]                                       # megafold.py:582-583, 588
    q = F.linear(single, P["attn.to_q.weight"], P.get("attn.to_q.bias"))                 # attention.py:176
    k, v = F.linear(single, P["attn.to_kv.weight"]).chunk(2, dim=-1)                     # attention.py:178-179
    split = lambda t: t.reshape(b, n, heads, dim_head).permute(0, 2, 1, 3)               # attention.py:181
    q, k, v = split(q), split(k), split(v)
    sim = torch.matmul(q * dim_head ** -0.5, k.transpose(-1, -2))                        # attention.py:502-507
    sim = sim + bias                                                                     # attention.py:511-512
    if mask is not None:
        sim = sim.masked_fill(~mask[:, None, None, :], float("-inf"))                    # attention.py:521-524
    attn = torch.nan_to_num(torch.softmax(sim, dim=-1), nan=0.0)                         # attention.py:533
    out = torch.matmul(attn, v)                                                          # attention.py:537
    out = out.permute(0, 2, 1, 3).reshape(b, n, heads * dim_head)                        # attention.py:196
    if "attn.to_gates.weight" in P:
        out = out * torch.sigmoid(F.linear(single, P["attn.to_gates.weight"], P.get("attn.to_gates.bias")))   # attention.py:200-203
    return F.linear(out, P["attn.to_out.weight"])                                        # attention.py:207


def attention_pair_bias_forward_backward(single, pairwise, params, dout, heads, dim_head, mask=None,
                                         attn_bias=None, dtype=torch.float64):
    """Returns ``(out, dsingle, dpairwise, {name: dparam})`` by autograd on the forward expression."""
    s = single.detach().to(dtype).requires_grad_(True)
    z = pairwise.detach().to(dtype).requires_grad_(True)
    ps = {k: v.detach().to(dtype).requires_grad_(True) for k, v in params.items()}
    out = attention_pair_bias_forward(s, z, ps, heads, dim_head, mask, attn_bias, dtype)
    grads = torch.autograd.grad(out, [s, z] + list(ps.values()), dout.to(dtype), allow_unused=True)
    grads = [torch.zeros_like(t) if g is None else g for g, t in zip(grads, [s, z] + list(ps.values()))]
    return out.detach(), grads[0], grads[1], dict(zip(ps.keys(), grads[2:]))
