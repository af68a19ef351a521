"""Single-representation attention with pair bias around the fused kernels (MI355X).

Drop-in for ``AttentionPairBias(heads=..., dim_pairwise=..., dim=..., dim_head=...)`` of the reference
(megafold/model/megafold.py:501-591 with ``Attention``, megafold/model/attention.py:88-209) in its full
(not windowed) form, as used by the Pairformer's single track (megafold.py:1221-1222: heads 16, head
dimension 64).  Parameter names and shapes are the reference's::

    to_attn_bias.0.WEIGHT / .BIAS / .linear_weight [dim_pairwise, heads]   LayernormLinear, weight zero-initialised
    attn.to_q.weight / .bias, attn.to_kv.weight, attn.to_gates.weight / .bias, attn.to_out.weight

What runs, per call:

1. the pair bias ``LayerNorm(pairwise) W_b`` through the fused LayerNorm -> Linear kernel (K = 128, N = 16 at
   the model's sizes) and, WITHOUT the ``"b ... h -> b h ..."`` copy, as the strided view ``[b, 1, h, i, j]``
   the attention kernels read directly;
2. the projections of the single representation (q, k | v, gates); K and V are column slices of one GEMM output,
   read in place as the attention operator's ``[B, N = 1, S, H, D]`` operands;
3. the attention kernels (``mf_evoattn_fwd`` / ``mf_evoattn_bwd``) with the key mask as a keep-mask;
4. the sigmoid gate kernel reading the gate columns in place, and the output projection.

The windowed form (``window_size``, the sequence-local atom transformer) and memory key / values are outside
this path and raise ``NotImplementedError``.
"""
from __future__ import annotations

from typing import Optional

import torch
import torch.nn as nn
import torch.nn.functional as F

from ..FusedEvoAttention.evoattention import TritonEvoformer
from ..FusedLayernormLinear.fused_layernorm_linear import LayernormLinear
from ..FusedTriangleAttention.triangle_attention import Attention
from ..gate import sigmoid_gate

__all__ = ["AttentionPairBias"]


class AttentionPairBias(nn.Module):
    """Same constructor and ``forward`` keywords as the reference class (megafold.py:501-591)."""

    def __init__(self, *, heads, dim_pairwise, window_size=None, num_memory_kv=0, **attn_kwargs):
        super().__init__()
        if window_size is not None or num_memory_kv:
            raise NotImplementedError("windowed attention and memory key / values are not part of this path")
        self.window_size = None
        self.attn = Attention(heads=heads, **attn_kwargs)
        ln_linear = LayernormLinear(dim_pairwise, heads, has_linear_bias=False)
        nn.init.zeros_(ln_linear.linear_weight)                       # megafold.py:531
        self.to_attn_bias = nn.Sequential(ln_linear, nn.Identity())   # the reference's Rearrange holds no state

    def forward(self, single_repr: torch.Tensor, *, pairwise_repr: torch.Tensor,
                attn_bias: Optional[torch.Tensor] = None, mask: Optional[torch.Tensor] = None, **kwargs) -> torch.Tensor:
        # keywords the reference forwards to Attention (context, windowed_mask, memory_kv, value_residual, ...)
        # select paths that are not built here: refuse them instead of computing self-attention silently
        extra = [k for k, v in kwargs.items() if v is not None and k != "verbose"]
        if extra:
            raise NotImplementedError("AttentionPairBias.forward: unsupported keyword(s) %s" % ", ".join(sorted(extra)))
        a = self.attn
        b, n, _ = single_repr.shape
        h, d = a.heads, a.dim_head
        inner = h * d
        if pairwise_repr.dim() != 4:
            raise NotImplementedError("windowed pairwise representations are not part of this path")
        # pair bias [b, i, j, h] -> view [b, 1, h, i, j]; an extra bias [b, i, j] is added to every head
        bias = self.to_attn_bias(pairwise_repr).permute(0, 3, 1, 2).unsqueeze(1)
        if attn_bias is not None:
            bias = bias + attn_bias[:, None, None].to(bias.dtype)
        # projections of the single representation (three small GEMMs; their outputs are used in place)
        dtype = bias.dtype
        x = single_repr.to(dtype)
        lin = lambda m: F.linear(x, m.weight.to(dtype), m.bias.to(dtype) if m.bias is not None else None)
        Q = lin(a.to_q).unflatten(-1, (h, d)).unsqueeze(1)                                       # [b, 1, n, h, d]
        KV = lin(a.to_kv)
        K = KV[..., :inner].unflatten(-1, (h, d)).unsqueeze(1)                                   # strided views of KV
        V = KV[..., inner:].unflatten(-1, (h, d)).unsqueeze(1)
        if mask is not None:
            res_mask = mask.view(b, 1, 1, 1, n)                                       # bool keep-mask
        else:
            res_mask = torch.zeros(b, 1, 1, 1, n, dtype=torch.float32, device=x.device)
        O = TritonEvoformer(Q, K, V, res_mask, bias)                                  # [b, 1, n, h, d]
        out = O.reshape(b * n, inner)
        if a.to_gates is not None:
            out = sigmoid_gate(out, lin(a.to_gates).view(b * n, inner))
        return F.linear(out.view(b, n, inner), a.to_out.weight.to(dtype))
