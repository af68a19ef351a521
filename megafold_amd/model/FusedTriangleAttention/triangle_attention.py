"""Pre-LayerNorm triangle attention around the fused kernels (MI355X).

Drop-in for ``PreLayerNorm(TriangleAttention(dim=..., heads=..., node_type=...), dim=...)`` of the
reference (megafold/model/megafold.py:305-331, 594-648 with ``Attention``, megafold/model/attention.py:88-209),
as constructed by ``PairwiseBlock`` (megafold.py:707-722).  Parameter names and shapes are the
reference's, so its checkpoints load unchanged::

    norm.weight, norm.bias                          LayerNorm(dim)
    fn.to_attn_bias.0.weight        [heads, dim]    LinearNoBias
    fn.attn.to_q.weight / .bias     [heads*dh, dim]
    fn.attn.to_kv.weight            [2*heads*dh, dim]
    fn.attn.to_gates.weight / .bias [heads*dh, dim]
    fn.attn.to_out.weight           [dim, heads*dh]

What runs, per call:

1. ONE fused LayerNorm -> Linear (``mf_lnlinear_fwd``) with the five projections concatenated along the
   output axis: ``Y[M, 4*heads*dh + heads (padded to 8)] = LN(x) [Wq | Wk | Wv | Wg | Wb] + [bq | 0 | 0 | bg | 0]``.
   The reference normalises once and then reads the normalised tensor five times.
2. Q, K, V are strided views of ``Y`` in the attention operator's ``[B, N, S, H, D]`` layout and the pair
   bias is the strided view ``Y[(b, i, j), 4*heads*dh + h] -> [B, 1, H, S, S]``: no head split / merge
   copies, no ``repeat`` of the bias over rows (megafold.py:634-640).  "ending" nodes swap the two position
   strides of these views instead of transposing the pair tensor (megafold.py:631-632, 645-646): no copy.
3. The attention kernels (``mf_evoattn_fwd`` / ``mf_evoattn_bwd``).  Backward writes dQ, dK, dV straight
   into the column slices of dY.
4. The sigmoid gate in one pass each way (``mf_sigmoid_gate_fwd`` / ``mf_sigmoid_gate_bwd``, reading the
   gate columns of ``Y`` and writing the gate columns of dY in place), the output projection and its two
   gradients through the BLAS library.

Differences from the reference call path (megafold/model/attention.py:466-492), all on purpose: the key
mask is a real mask (the reference adds the 0/1 values of ``mask.bfloat16()`` to the logits), and the
attention output is merged as ``[b, row, seq, (h d)]`` (the reference reshapes ``[b, n1, n2, h, d]``
storage to ``[(b n1), h, n2, d]`` without permuting).  Both follow the reference's own eager path.
"""
from __future__ import annotations

import ctypes as C
from typing import Optional

import torch
import torch.nn as nn
import torch.nn.functional as F

from ... import _lib
from ..linear import tall_skinny_tn
from ..FusedEvoAttention.evoattention import evoattention_backward, evoattention_forward
from ..FusedLayernormLinear.fused_layernorm_linear import (fused_shape_supported, layernorm_linear_backward,
                                                           layernorm_linear_forward)

__all__ = ["Attention", "Dropout", "PreLayerNormTriangleAttention", "TriangleAttention",
           "TriangleAttentionFunction", "sigmoid_gate_forward", "sigmoid_gate_backward"]


def _gate_args(O2d, G):
    if not (O2d.is_cuda and O2d.dim() == 2 and G.shape == O2d.shape and G.dtype == O2d.dtype):
        raise ValueError("gate operands must be GPU matrices of one shape and dtype")
    if O2d.stride(1) != 1 or G.stride(1) != 1:
        raise ValueError("gate operands need unit stride along the columns")
    a = _lib.GateArgs()
    a.M, a.C = O2d.shape
    a.dtype = _lib.dtype_code(O2d.dtype)
    a.o, a.ldo = O2d.data_ptr(), O2d.stride(0)
    a.g, a.ldg = G.data_ptr(), G.stride(0)
    a.stream = torch.cuda.current_stream(O2d.device).cuda_stream
    return a


def sigmoid_gate_forward(O2d: torch.Tensor, G: torch.Tensor, res: Optional[torch.Tensor] = None) -> torch.Tensor:
    """``O2d * sigmoid(G)`` (megafold/model/attention.py:199-203) in one pass; ``G`` may be a column slice.
    ``res`` (same shape, optional) is added in the same pass (a block's ``x + f(x)``)."""
    a = _gate_args(O2d, G)
    with torch.cuda.device(O2d.device):
        A = torch.empty(O2d.shape, dtype=O2d.dtype, device=O2d.device)
        a.a, a.lda = A.data_ptr(), A.stride(0)
        if res is not None:
            if res.shape != O2d.shape or res.dtype != O2d.dtype or res.stride(1) != 1:
                raise ValueError("res must match the gate operands")
            a.res, a.ldres = res.data_ptr(), res.stride(0)
        _lib.check(_lib.lib().mf_sigmoid_gate_fwd(C.byref(a)), "mf_sigmoid_gate_fwd")
    return A


def sigmoid_gate_backward(dA: torch.Tensor, O2d: torch.Tensor, G: torch.Tensor, dG_out: torch.Tensor,
                          need_product: bool = True):
    """Returns ``(dO, A)`` and writes the gate gradient into ``dG_out`` (may be a column slice):
    ``dO = dA * s``, ``dG = dA * O * s * (1 - s)``, ``A = O * s`` with ``s = sigmoid(G)``; ``A`` is None
    when ``need_product`` is false."""
    a = _gate_args(O2d, G)
    if dA.shape != O2d.shape or dA.dtype != O2d.dtype or dG_out.shape != O2d.shape or dG_out.dtype != O2d.dtype:
        raise ValueError("gate gradients must match the operands' shape and dtype")
    dA = dA if dA.stride(1) == 1 else dA.contiguous()
    with torch.cuda.device(O2d.device):
        dO = torch.empty(O2d.shape, dtype=O2d.dtype, device=O2d.device)
        A = torch.empty(O2d.shape, dtype=O2d.dtype, device=O2d.device) if need_product else None
        if A is not None:
            a.a, a.lda = A.data_ptr(), A.stride(0)
        a.da, a.ldda = dA.data_ptr(), dA.stride(0)
        a.d_o, a.lddo = dO.data_ptr(), dO.stride(0)
        a.dg, a.lddg = dG_out.data_ptr(), dG_out.stride(0)
        _lib.check(_lib.lib().mf_sigmoid_gate_bwd(C.byref(a)), "mf_sigmoid_gate_bwd")
    return dO, A


def _views(Y: torch.Tensor, b: int, n: int, heads: int, dh: int, transposed: bool = False):
    """Q, K, V ``[b, n, n, h, dh]``, gate ``[M, h*dh]`` and pair bias ``[b, 1, h, n, n]`` as views of
    ``Y [b*n*n, Nt]`` (columns: q | k | v | gate | bias | padding; row ``(b, i, j)`` of Y belongs to pair
    position (i, j)).  ``transposed``: the attention runs on the transposed pair tensor ("ending" nodes), i.e.
    attention row r / sequence position s is pair position (s, r): the same memory with the two position
    strides swapped, nothing is copied."""
    Nt = Y.shape[1]
    inner = heads * dh
    s_row, s_seq = (Nt, n * Nt) if transposed else (n * Nt, Nt)
    qkv_strides = (n * n * Nt, s_row, s_seq, dh, 1)
    off = Y.storage_offset()
    Q = Y.as_strided((b, n, n, heads, dh), qkv_strides, off)
    K = Y.as_strided((b, n, n, heads, dh), qkv_strides, off + inner)
    V = Y.as_strided((b, n, n, heads, dh), qkv_strides, off + 2 * inner)
    G = Y[:, 3 * inner:4 * inner]
    Bv = Y.as_strided((b, 1, heads, n, n), (n * n * Nt, 0, 1, s_row, s_seq), off + 4 * inner)
    return Q, K, V, G, Bv


class TriangleAttentionFunction(torch.autograd.Function):
    """x ``[b, n, n, d]`` -> block output ``[b, n, n, d]``, both in the layout of the pair tensor.  With
    ``transposed`` the attention runs along the columns ("ending" nodes: the reference transposes the tensor,
    attends along rows and transposes back, megafold.py:631-632, 645-646): LayerNorm, the projections, the gate
    and the output projection act on single positions, so only the attention operator has to see the
    transposition, and it does so through its strides."""

    @staticmethod
    @torch.amp.custom_fwd(device_type="cuda", cast_inputs=torch.bfloat16)
    def forward(ctx, x, mask, ln_w, ln_b, Wq, bq, Wkv, Wg, bg, Wb, Wo, heads, dim_head, transposed=False,
                add_residual=False):
        b, n, n2, d = x.shape
        assert n == n2, "pairwise representation must be [b, n, n, d]"
        inner = heads * dim_head
        dt = x.dtype
        x2d = x.contiguous().view(b * n * n, d)
        pad = (-(4 * inner + heads)) % 8
        # [d, Nt] as the fused operator stores linear weights (nn.Linear.weight transposed)
        Wcat = torch.cat([Wq, Wkv, Wg, Wb] + ([Wb.new_zeros(pad, d)] if pad else []), dim=0).to(dt).t().contiguous()
        zeros = lambda k: x.new_zeros(k)
        bcat = torch.cat([bq.to(dt) if bq is not None else zeros(inner), zeros(2 * inner),
                          bg.to(dt) if bg is not None else zeros(inner), zeros(heads + pad)])
        Y, _, Wc, Mean, RSTD = layernorm_linear_forward(x2d, Wcat, bcat, ln_w, ln_b, True, True)
        Q, K, V, G, Bv = _views(Y, b, n, heads, dim_head, transposed)
        if mask is None:
            mask5 = torch.ones((b, 1, 1, 1, n), dtype=torch.bool, device=x.device)
        else:
            mask5 = mask.to(torch.bool).view(b, 1, 1, 1, n)
        O = torch.empty((b, n, n, heads, dim_head), dtype=dt, device=x.device)      # indexed by pair position
        _, lse, (Qs, Ks, Vs, masks, biass, tiles) = evoattention_forward(Q, K, V, mask5, Bv,
                                                                         out=O.transpose(1, 2) if transposed else O,
                                                                         save_bias_tiles=True)
        O2d = O.view(b * n * n, inner)
        A = sigmoid_gate_forward(O2d, G)
        out = F.linear(A, Wo.to(dt))
        if add_residual:
            # x + f(x).  (torch.addmm would copy x into the result first and then run the GEMM with beta = 1:
            # 10.6 + 12.6 us more at n = 384 against 18.7 us for this add.)  The backward sum is folded into
            # the LayerNorm backward below.
            out += x2d
        ctx.add_residual = add_residual
        ctx.save_for_backward(x2d, Y, O, lse, Mean, RSTD, masks, Wc, ln_w, ln_b, Wo, tiles)
        ctx.dims = (b, n, d, heads, dim_head, pad, transposed)
        ctx.has_bias = (bq is not None, bg is not None)
        return out.view(b, n, n, d)

    @staticmethod
    @torch.amp.custom_bwd(device_type="cuda")
    def backward(ctx, dout):
        x2d, Y, O, lse, Mean, RSTD, mask5, Wc, ln_w, ln_b, Wo, tiles = ctx.saved_tensors
        b, n, d, heads, dh, pad, transposed = ctx.dims
        inner = heads * dh
        M, Nt = Y.shape
        dt = x2d.dtype
        dout2d = dout.to(dt).reshape(M, d)
        Q, K, V, G, Bv = _views(Y, b, n, heads, dh, transposed)
        O2d = O.view(M, inner)
        dA = dout2d @ Wo.to(dt)                           # [M, inner]
        dY = torch.empty_like(Y)
        dQ, dK, dV, dG, dBv = _views(dY, b, n, heads, dh, transposed)
        dO, A = sigmoid_gate_backward(dA, O2d, G, dG)
        dWo = tall_skinny_tn(dout2d, A)                  # [d, inner]
        dO = dO.view(b, n, n, heads, dh)
        if transposed:
            dO, O = dO.transpose(1, 2), O.transpose(1, 2)
        _, _, _, dbias = evoattention_backward(dO, Q, K, V, mask5, Bv, O, lse, True, out=(dQ, dK, dV), bias_tiles=tiles)
        dBv[:, 0].copy_(dbias[:, 0])
        if pad:
            dY[:, 4 * inner + heads:].zero_()
        dX, dWc, dbc, dlnw, dlnb = layernorm_linear_backward(dY, x2d, Wc, Mean, RSTD, ln_w, ln_b, True, True,
                                                             dx_add=dout2d if ctx.add_residual else None)
        dWt = dWc.t()                                     # [Nt, d] rows: q | k | v | gate | bias
        has_bq, has_bg = ctx.has_bias
        return (dX.view(b, n, n, d), None, dlnw, dlnb,
                dWt[:inner], dbc[:inner] if has_bq else None,
                dWt[inner:3 * inner], dWt[3 * inner:4 * inner], dbc[3 * inner:4 * inner] if has_bg else None,
                dWt[4 * inner:4 * inner + heads], dWo, None, None, None, None)


class Dropout(nn.Module):
    """Row / column structured dropout of the reference (megafold/model/megafold.py:264-298)."""

    def __init__(self, prob: float, *, dropout_type: Optional[str] = None):
        super().__init__()
        self.dropout = nn.Dropout(prob)
        self.dropout_type = dropout_type

    def forward(self, t: torch.Tensor) -> torch.Tensor:
        if self.dropout_type is None:
            return self.dropout(t)
        assert t.ndim == 4, "Tensor `t` must consist of 4 dimensions for row/col structured dropout."
        if not self.training or self.dropout.p == 0.0:
            return t
        batch, row, col, dim = t.shape
        ones_shape = (batch, 1, col, dim) if self.dropout_type == "row" else (batch, row, 1, dim)
        return t * self.dropout(t.new_ones(ones_shape))


class Attention(nn.Module):
    """Parameter container with the names, shapes and initialisation of the reference ``Attention``
    (megafold/model/attention.py:88-158), restricted to what triangle attention uses: full (not windowed)
    attention without memory key / values."""

    def __init__(self, *, dim, dim_head=64, heads=8, gate_output=True, query_bias=True, init_gate_bias=-2.0):
        super().__init__()
        dim_inner = dim_head * heads
        self.heads, self.dim_head = heads, dim_head
        self.to_q = nn.Linear(dim, dim_inner, bias=query_bias)
        self.to_kv = nn.Linear(dim, dim_inner * 2, bias=False)
        self.to_out = nn.Linear(dim_inner, dim, bias=False)
        self.to_gates = None
        if gate_output:
            gate_linear = nn.Linear(dim, dim_inner)
            nn.init.zeros_(gate_linear.weight)
            nn.init.constant_(gate_linear.bias, init_gate_bias)
            self.to_gates = gate_linear


class TriangleAttention(nn.Module):
    """Parameter container of the reference ``TriangleAttention`` (megafold/model/megafold.py:594-615)."""

    def __init__(self, *, dim, heads, node_type, dropout=0.0, dropout_type=None, **attn_kwargs):
        super().__init__()
        assert node_type in ("starting", "ending")
        self.need_transpose = node_type == "ending"
        self.to_attn_bias = nn.Sequential(nn.Linear(dim, heads, bias=False))
        self.dropout = Dropout(dropout, dropout_type=dropout_type)
        self.attn = Attention(dim=dim, heads=heads, **attn_kwargs)


class PreLayerNormTriangleAttention(nn.Module):
    """``PreLayerNorm(TriangleAttention(...), dim=dim)`` of the reference as one fused block.

    ``forward(pairwise_repr [b, n, n, d], mask [b, n] bool or None) -> [b, n, n, d]`` (the caller adds
    the residual, megafold.py:745-746)."""

    def __init__(self, *, dim, heads, node_type, dim_head=32, dropout=0.0, dropout_type=None, **attn_kwargs):
        super().__init__()
        self.fn = TriangleAttention(dim=dim, heads=heads, node_type=node_type, dropout=dropout,
                                    dropout_type=dropout_type, dim_head=dim_head, **attn_kwargs)
        self.norm = nn.LayerNorm(dim)
        if self.fn.attn.to_gates is None:
            raise ValueError("the fused block needs gate_output=True (the reference default)")

    def forward(self, pairwise_repr: torch.Tensor, mask: Optional[torch.Tensor] = None,
                add_residual: bool = False) -> torch.Tensor:
        """``add_residual``: return ``pairwise_repr + block(pairwise_repr)`` (megafold.py:744-745) with both sums
        folded into the block's kernels; needs the dropout to be inactive (the reference drops before it adds)."""
        fn, attn = self.fn, self.fn.attn
        dim = pairwise_repr.shape[-1]
        Nt = 4 * attn.heads * attn.dim_head + attn.heads
        Nt += (-Nt) % 8
        dtype = torch.bfloat16 if torch.is_autocast_enabled() else pairwise_repr.dtype
        if not pairwise_repr.is_cuda:
            raise RuntimeError("PreLayerNormTriangleAttention runs on the GPU only (got device %s)" % pairwise_repr.device)
        if not fused_shape_supported(dim, Nt, dtype) or attn.dim_head % 8 != 0 or attn.dim_head > 64:
            raise ValueError("unsupported shape for the fused block: dim=%d heads=%d dim_head=%d" %
                             (dim, attn.heads, attn.dim_head))
        drops = fn.dropout.training and fn.dropout.dropout.p > 0.0
        # an fp32 stream under autocast keeps its separate fp32 add (megafold.py:744-745 promotes)
        fused_sum = add_residual and not drops and pairwise_repr.dtype == dtype
        out = TriangleAttentionFunction.apply(pairwise_repr, mask, self.norm.weight, self.norm.bias, attn.to_q.weight,
                                              attn.to_q.bias, attn.to_kv.weight, attn.to_gates.weight,
                                              attn.to_gates.bias, fn.to_attn_bias[0].weight, attn.to_out.weight,
                                              attn.heads, attn.dim_head, fn.need_transpose, fused_sum)
        if fused_sum:
            return out
        out = fn.dropout(out)
        return out + pairwise_repr if add_residual else out
