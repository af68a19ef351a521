"""Eager restatement of the pre-LayerNorm triangle-attention block and its gradients (CPU, test-only).

Follows the reference modules literally, one tensor expression per reference statement:

* ``PreLayerNorm.forward``       megafold/model/megafold.py:322-331   x = LayerNorm(x); fn(x)
* ``TriangleAttention.forward``  megafold/model/megafold.py:617-648   transpose for "ending" nodes,
  ``attn_bias = rearrange(Linear(x), "... i j h -> ... h i j")`` shared by every row, key mask ``mask[b, j]``
* ``Attention.forward``          megafold/model/attention.py:155-209  q = to_q(x); k, v = to_kv(x).chunk(2);
  split heads ``(h d)``; attend; merge heads; ``out * sigmoid(to_gates(x))``; ``to_out``
* ``Attend.forward`` default path megafold/model/attention.py:498-537  softmax(q k^T * d^-0.5 + bias, masked) v

The key mask is applied where the eager path of the reference applies it (masked_fill before the softmax,
attention.py:519-522).  The reference fills with the most negative finite value, here -inf is used: with at
least one kept key both give masked keys exactly zero weight; a row with no kept key is defined as attending
to nothing (the reference would average all values).  Gradients come from
autograd on this expression in float64, so the oracle holds no hand-derived backward formulas.
"""
from __future__ import annotations

import torch
import torch.nn.functional as F

EPS = 1e-5  # nn.LayerNorm default, megafold/model/megafold.py:185


def triangle_attention_forward(x, mask, params, heads, dim_head, node_type="starting", dtype=torch.float64):
    """x ``[b, n, n, d]``; mask ``[b, n]`` bool (True = keep) or None; params: dict of tensors named as the
    reference state dict of ``PreLayerNorm(TriangleAttention(...))``:

    ``norm.weight, norm.bias, fn.to_attn_bias.0.weight [h, d], fn.attn.to_q.weight [h*dh, d], fn.attn.to_q.bias,
    fn.attn.to_kv.weight [2*h*dh, d], fn.attn.to_gates.weight, fn.attn.to_gates.bias, fn.attn.to_out.weight [d, h*dh]``.
    Returns the block output ``[b, n, n, d]`` in ``dtype`` (before dropout and the residual add)."""
    P = {k: v.to(dtype) for k, v in params.items()}
    x = x.to(dtype)
    b, n, _, d = x.shape
    x = F.layer_norm(x, (d,), P["norm.weight"], P["norm.bias"], EPS)                       # megafold.py:330
    if node_type == "ending":
        x = x.transpose(1, 2)                                                              # megafold.py:631-632
    bias = F.linear(x, P["fn.to_attn_bias.0.weight"]).permute(0, 3, 1, 2)                  # [b, h, i, j]  megafold.py:634
    q = F.linear(x, P["fn.attn.to_q.weight"], P.get("fn.attn.to_q.bias"))                  # attention.py:176
    k, v = F.linear(x, P["fn.attn.to_kv.weight"]).chunk(2, dim=-1)                         # attention.py:179
    # rows of the pair tensor are the attention batch: [b, row, seq, (h dh)] -> [b, row, h, seq, dh]
    split = lambda t: t.reshape(b, n, n, heads, dim_head).permute(0, 1, 3, 2, 4)           # attention.py:181
    q, k, v = split(q), split(k), split(v)
    sim = torch.matmul(q, k.transpose(-1, -2)) * dim_head ** -0.5                          # attention.py:501-507
    sim = sim + bias.unsqueeze(1)                                                          # attention.py:511-512
    if mask is not None:
        keep = mask.view(b, 1, 1, 1, n)                                                    # megafold.py:637, attention.py:519-522
        sim = sim.masked_fill(~keep, float("-inf"))
    attn = torch.softmax(sim, dim=-1)                                                      # attention.py:533
    attn = torch.nan_to_num(attn, nan=0.0)     # a row with no key left attends to nothing
    out = torch.matmul(attn, v)                                                            # attention.py:537
    out = out.permute(0, 1, 3, 2, 4).reshape(b, n, n, heads * dim_head)                    # attention.py:196
    gates = F.linear(x, P["fn.attn.to_gates.weight"], P.get("fn.attn.to_gates.bias"))      # attention.py:201
    out = out * torch.sigmoid(gates)                                                       # attention.py:203
    out = F.linear(out, P["fn.attn.to_out.weight"])                                        # attention.py:207
    if node_type == "ending":
        out = out.transpose(1, 2)                                                          # megafold.py:645-646
    return out


def triangle_attention_forward_backward(x, mask, params, dout, heads, dim_head, node_type="starting",
                                        dtype=torch.float64):
    """Returns ``(out, dx, {name: dparam})`` by autograd on :func:`triangle_attention_forward`."""
    xs = x.detach().to(dtype).requires_grad_(True)
    ps = {k: v.detach().to(dtype).requires_grad_(True) for k, v in params.items()}
    out = triangle_attention_forward(xs, mask, ps, heads, dim_head, node_type, dtype)
    grads = torch.autograd.grad(out, [xs] + list(ps.values()), dout.to(dtype))
    return out.detach(), grads[0], dict(zip(ps.keys(), grads[1:]))
