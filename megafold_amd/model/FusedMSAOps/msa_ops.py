"""The two MSA-module operators built on the fused LayerNorm -> Linear kernel (MI355X).

Drop-ins for ``MSAPairWeightedAveraging`` (Algorithm 10, megafold/model/megafold.py:826-902) and
``OuterProductMean`` (Algorithm 9, megafold/model/megafold.py:752-824) with the reference's constructors and
parameter names::

    MSAPairWeightedAveraging   msa_to_values_and_gates.0.{WEIGHT,BIAS,linear_weight}   LayernormLinear(dim_msa, 2*h*dh)
                               pairwise_repr_to_attn.0.{WEIGHT,BIAS,linear_weight}     LayernormLinear(dim_pairwise, h)
                               to_out.1.weight                                         Linear(h*dh, dim_msa), no bias
    OuterProductMean           to_hidden.{WEIGHT,BIAS,linear_weight}                   LayernormLinear(dim_msa, 2*dim_hidden)
                               to_pairwise_repr.weight / .bias                         Linear(dim_hidden^2, dim_pairwise)

``MSAPairWeightedAveraging``: ``out[b,s,i,h,:] = sum_j softmax_j(bias[b,h,i,j] + mask[j]) values[b,s,j,h,:]``.  The
weights do not depend on the MSA row: for the module's shape (16-bit, 8 heads of 32 channels, n <= 384) the softmax is
taken once per (b, h, i) and the averaging, the gate and the backward run in kernels of their own (``mf_pwa_*``,
``PairWeightedAverageFunction``).  Other shapes use the pair-biased attention operator with zero queries and keys
and the MSA rows as its row batch.  Values and gates are column halves of the fused projection output (no
``"b s n (gv h d) -> gv b h s n d"`` copy), the result comes out as ``"b s n (h d)"`` (no merge copy).

``OuterProductMean``: the fused LayerNorm -> Linear, the masks and the division by the number of MSA rows folded into
the two small operands (exact for the 0/1 masks; the division is rounded once, before the product), then for the
module's shape (16-bit, hidden 32, 128 pair channels) the contraction over the MSA rows and the output projection in
one kernel (``mf_opm_fused_fwd``) and the backward in three (``mf_opm_dw``, ``mf_opm_dab`` once per operand): the
``[n, n, hidden^2]`` outer product is never written to memory.  Other shapes run the reference's expressions (one
GEMM per batch element, a layout move to ``"b i j (d e)"``, the projection).
"""
from __future__ import annotations

from typing import Optional

import torch
import torch.nn as nn

import ctypes as C

from ... import _lib
from ..FusedEvoAttention.evoattention import TritonEvoformer
from ..FusedLayernormLinear.fused_layernorm_linear import LayernormLinear
from ..FusedTriangleAttention.triangle_attention import Dropout
from ..FusedTriangleAttention.triangle_attention import sigmoid_gate_backward
from ..gate import sigmoid_gate
from ..linear import linear_no_bias

__all__ = ["MSAPairWeightedAveraging", "OuterProductMean", "PairWeightedAverageFunction", "OuterProductMeanFunction"]


def _pwa_args(b, s, n, h, d, dtype, device):
    a = _lib.PwaArgs()
    a.B, a.S, a.N, a.H, a.D = b, s, n, h, d
    a.dtype = _lib.dtype_code(dtype)
    a.stream = torch.cuda.current_stream(device).cuda_stream
    return a


def _pwa_apply(W, X, G, dims, out=None):
    """``out[(b s i), (h d)] = sum_j W[b, h, i, j] X[(b s j), (h d)]`` (times ``sigmoid(G)`` if given) through
    ``mf_pwa_apply``; X, G, out: matrices of rows with unit stride along the columns (column slices are fine)."""
    b, s, n, h, d = dims
    if out is None:
        out = torch.empty((b * s * n, h * d), dtype=X.dtype, device=X.device)
    a = _pwa_args(b, s, n, h, d, X.dtype, X.device)
    a.w = W.data_ptr()
    a.x, a.ldx = X.data_ptr(), X.stride(0)
    if G is not None:
        a.g, a.ldg = G.data_ptr(), G.stride(0)
    a.y, a.ldy = out.data_ptr(), out.stride(0)
    _lib.check(_lib.lib().mf_pwa_apply(C.byref(a)), "mf_pwa_apply")
    return out


class PairWeightedAverageFunction(torch.autograd.Function):
    """``A[(b s i), (h d)] = (sum_j softmax_j(logits[b, i, j, h] + mask[b, j]) V[(b s j), (h d)]) * sigmoid(G)`` with
    V | G the two column halves of ``vg`` (megafold.py:884-893): the softmax once per (b, h, i), the averaging and
    the gate in one kernel with the weight rows resident in registers across the MSA rows.  Backward: the gate's
    derivative on the recomputed averages, dV through the same kernel on the transposed weights, the weights'
    gradient as a contraction over (MSA row, channel) with the softmax backward behind it."""

    @staticmethod
    def forward(ctx, logits, vg, mask, dims):
        b, s, n, h, d = dims
        inner = h * d
        NP = (n + 31) // 32 * 32
        with torch.cuda.device(vg.device):
            W = torch.empty((b, h, NP, NP), dtype=vg.dtype, device=vg.device)
            a = _pwa_args(b, s, n, h, d, vg.dtype, vg.device)
            a.logits, a.ld_logits = logits.data_ptr(), logits.stride(0)
            a.mask = mask.data_ptr() if mask is not None else None
            a.w = W.data_ptr()
            _lib.check(_lib.lib().mf_pwa_softmax_fwd(C.byref(a)), "mf_pwa_softmax_fwd")
            A = _pwa_apply(W, vg[:, :inner], vg[:, inner:], dims)
        ctx.save_for_backward(W, vg, logits)
        ctx.dims = dims
        return A

    @staticmethod
    def backward(ctx, dA):
        W, vg, logits = ctx.saved_tensors
        b, s, n, h, d = dims = ctx.dims
        inner = h * d
        lib = _lib.lib()
        with torch.cuda.device(vg.device):
            dA = dA.to(vg.dtype)
            dA = dA if dA.stride(1) == 1 else dA.contiguous()
            V, G = vg[:, :inner], vg[:, inner:]
            O = _pwa_apply(W, V, None, dims)                               # the averages before the gate, recomputed
            dvg = torch.empty_like(vg)
            dO, _ = sigmoid_gate_backward(dA, O, G, dvg[:, inner:], need_product=False)
            _pwa_apply(W.transpose(-1, -2).contiguous(), dO, None, dims, out=dvg[:, :inner])    # dV
            a = _pwa_args(b, s, n, h, d, vg.dtype, vg.device)
            a.w = W.data_ptr()
            a.x, a.ldx = V.data_ptr(), V.stride(0)
            a.dy, a.lddy = dO.data_ptr(), dO.stride(0)
            a.n_chunks = lib.mf_pwa_dw_chunks(C.byref(a))
            part = torch.empty((a.n_chunks,) + tuple(W.shape), dtype=torch.float32, device=vg.device)
            a.dw_part = part.data_ptr()
            _lib.check(lib.mf_pwa_dw(C.byref(a)), "mf_pwa_dw")
            dlogits = torch.empty_like(logits)
            a.dlogits, a.ld_dlogits = dlogits.data_ptr(), dlogits.stride(0)
            _lib.check(lib.mf_pwa_softmax_bwd(C.byref(a)), "mf_pwa_softmax_bwd")
        return dlogits, dvg, None, None


class MSAPairWeightedAveraging(nn.Module):
    """Algorithm 10; constructor and ``forward`` keywords as the reference (megafold.py:829-866)."""

    def __init__(self, *, dim_msa=64, dim_pairwise=128, dim_head=32, heads=8, dropout=0.0, dropout_type=None):
        super().__init__()
        dim_inner = dim_head * heads
        self.heads, self.dim_head = heads, dim_head
        self.msa_to_values_and_gates = nn.Sequential(
            LayernormLinear(dim_msa, dim_inner * 2, has_linear_bias=False), nn.Identity())
        self.pairwise_repr_to_attn = nn.Sequential(
            LayernormLinear(dim_pairwise, heads, has_linear_bias=False), nn.Identity())
        self.to_out = nn.Sequential(nn.Identity(), nn.Linear(dim_inner, dim_msa, bias=False),
                                    Dropout(dropout, dropout_type=dropout_type))

    def forward(self, *, msa: torch.Tensor, pairwise_repr: torch.Tensor, mask: Optional[torch.Tensor] = None) -> torch.Tensor:
        b, s, n, _ = msa.shape
        h, d = self.heads, self.dim_head
        inner = h * d
        vg = self.msa_to_values_and_gates(msa)                                   # [b, s, n, (gv h d)]
        logits = self.pairwise_repr_to_attn(pairwise_repr)                       # [b, i, j, h]
        if (h == 8 and d == 32 and n <= 384 and vg.dtype in (torch.float16, torch.bfloat16) and logits.dtype == vg.dtype
                and vg.is_contiguous() and logits.is_contiguous()):
            # the dedicated kernels: softmax once per (b, h, i), then the averaging with the gate in its epilogue
            keep = mask.to(torch.uint8).contiguous() if mask is not None else None
            A = PairWeightedAverageFunction.apply(logits.view(b * n * n, h), vg.view(b * s * n, 2 * inner), keep,
                                                  (b, s, n, h, d))
        else:
            # other shapes: the pair-biased attention operator with zero queries and keys and the MSA rows as
            # its row batch (the bias is shared by all rows), then the gate
            V = vg[..., :inner].unflatten(-1, (h, d))                            # view [b, s, n, h, d]
            bias = logits.permute(0, 3, 1, 2).unsqueeze(1)                       # view [b, 1, h, i, j]
            if mask is not None:
                res_mask = mask.view(b, 1, 1, 1, n)                              # keep-mask, shared by all rows s
            else:
                res_mask = torch.zeros(b, 1, 1, 1, n, dtype=torch.float32, device=msa.device)
            zero = torch.zeros(d, dtype=vg.dtype, device=vg.device).expand(b, s, n, h, d)   # queries = keys = 0
            O = TritonEvoformer(zero, zero, V, res_mask, bias)                    # softmax(bias) @ values
            A = sigmoid_gate(O.reshape(b * s * n, inner), vg.view(b * s * n, 2 * inner)[:, inner:])
        out = linear_no_bias(A.view(b, s, n, inner), self.to_out[1].weight)
        return self.to_out[2](out)


class _Permute0213(torch.autograd.Function):
    """``x [A, B, C, E] -> [A, C, B, E]`` (contiguous) through ``mf_permute_0213``; the gradient is the inverse
    move.  Rows of ``E`` elements must be 16 .. 256 bytes in steps of 16 and ``A <= 65535``, else PyTorch's
    ``permute(...).contiguous()`` does it."""

    @staticmethod
    def _move(x):
        import ctypes as C
        from ... import _lib
        A, B, Cc, E = x.shape
        rb = E * x.element_size()
        x = x.contiguous()
        if not x.is_cuda or rb % 16 != 0 or rb > 256 or A > 65535 or B > 65535 * 32:
            return x.permute(0, 2, 1, 3).contiguous()
        y = torch.empty((A, Cc, B, E), dtype=x.dtype, device=x.device)
        with torch.cuda.device(x.device):
            _lib.check(_lib.lib().mf_permute_0213(x.data_ptr(), y.data_ptr(), A, B, Cc, rb,
                                                  torch.cuda.current_stream(x.device).cuda_stream), "mf_permute_0213")
        return y

    @staticmethod
    def forward(ctx, x):
        return _Permute0213._move(x)

    @staticmethod
    def backward(ctx, g):
        return _Permute0213._move(g)


class OuterProductMean(nn.Module):
    """Algorithm 9; constructor and ``forward`` keywords as the reference (megafold.py:755-778)."""

    def __init__(self, *, dim_msa=64, dim_pairwise=128, dim_hidden=32, eps=1e-5):
        super().__init__()
        self.eps = eps
        self.to_hidden = LayernormLinear(dim_msa, dim_hidden * 2, has_linear_bias=False)
        self.to_pairwise_repr = nn.Linear(dim_hidden ** 2, dim_pairwise)

    def forward(self, msa: torch.Tensor, *, mask: Optional[torch.Tensor] = None,
                msa_mask: Optional[torch.Tensor] = None) -> torch.Tensor:
        b, s, n, _ = msa.shape
        hidden = self.to_hidden(msa)                                             # [b, s, n, 2 dh]
        dtype, dh = hidden.dtype, hidden.shape[-1] // 2
        lin = self.to_pairwise_repr
        # Everything elementwise is applied to the two small operands instead of the [b, n, n, dh*dh] product:
        # the MSA-row mask (0/1, so masking one operand equals masking both), the division by the number of kept
        # rows, and the pair mask mask_i * mask_j as a row mask on each side.
        if msa_mask is not None:
            inv = 1.0 / msa_mask.to(torch.float32).sum(-1).clamp(min=self.eps)               # [b]
            row_scale = msa_mask.to(torch.float32) * inv[:, None]                            # [b, s]
        else:
            row_scale = torch.full((b, s), 1.0 / s, dtype=torch.float32, device=msa.device)
        if (dh == 32 and lin.out_features == 128 and s <= 128 and dtype in (torch.float16, torch.bfloat16) and hidden.is_cuda):
            return OuterProductMeanFunction.apply(hidden, row_scale, mask, lin.weight, lin.bias)
        a, b_ = hidden.chunk(2, dim=-1)                                          # [b, s, n, dh] each (views)
        fa = row_scale[:, :, None, None]
        fb = None
        if mask is not None:
            pos = mask.to(torch.float32)[:, None, :, None]                                   # [b, 1, n, 1]
            fa, fb = fa * pos, pos
        a = (a.float() * fa).to(dtype)             # one rounding: 1 / rows is not a 16-bit number
        if fb is not None:
            b_ = b_ * fb.to(dtype)
        # operand matrices [(i d), s] with the contraction axis contiguous
        A = a.permute(0, 2, 3, 1).reshape(b, n * dh, s)
        B = b_.permute(0, 2, 3, 1).reshape(b, n * dh, s)
        return _outer_project_reference(A, B, lin.weight, lin.bias, n, dh)


def _outer_project_reference(A, B, weight, bias, n, dh):
    """The two-GEMM form: ``outer[(i d), (j e)] = A B^T`` per batch element, one layout move to ``"b i j (d e)"``
    and the projection (shapes the fused kernels do not take)."""
    b = A.shape[0]
    outer = torch.bmm(A, B.transpose(1, 2))                                                  # [b, (i d), (j e)]
    outer = _Permute0213.apply(outer.view(b * n, dh, n, dh)).view(b, n, n, dh * dh)          # "b i j (d e)"
    out = linear_no_bias(outer, weight)
    return out + bias.to(out.dtype) if bias is not None else out


class OuterProductMeanFunction(torch.autograd.Function):
    """``out[b, i, j, :] = W . (sum_s a[b, s, i, :] (x) b[b, s, j, :])_(d e) + bias`` with ``a | b`` the two halves of
    ``hidden`` scaled by ``row_scale[b, s]`` (first half only) and the position mask: operands packed by ``mf_opm_pack``,
    outer blocks and projection in one kernel (``mf_opm_fused_fwd``).  The ``[n, n, dh * dh]`` outer product never
    exists, in the forward or in the backward (``mf_opm_dw`` for the weight, ``mf_opm_dab`` for each operand: the outer
    blocks and their gradient are formed tile by tile in LDS; ``mf_opm_pack`` again for the way back to ``hidden``)."""

    @staticmethod
    def forward(ctx, hidden, row_scale, mask, weight, bias):
        b, s, n, _ = hidden.shape
        dtype, dev = hidden.dtype, hidden.device
        hidden = hidden if hidden.is_contiguous() else hidden.contiguous()
        lib = _lib.lib()
        with torch.cuda.device(dev):
            stream = torch.cuda.current_stream(dev).cuda_stream
            pos = mask.to(torch.uint8).contiguous() if mask is not None else None
            row_scale = row_scale.to(torch.float32).contiguous()
            Ap = torch.empty((b, n * 32, 128), dtype=dtype, device=dev)
            Bp = torch.empty((b, n * 32, 128), dtype=dtype, device=dev)
            _lib.check(lib.mf_opm_pack(hidden.data_ptr(), hidden.shape[-1], row_scale.data_ptr(),
                                       pos.data_ptr() if pos is not None else None, Ap.data_ptr(), Bp.data_ptr(),
                                       b, s, n, 0, _lib.dtype_code(dtype), stream), "mf_opm_pack")
            # the weight with its two hidden indices exchanged (column e * 32 + d)
            wp = weight.to(dtype).view(128, 32, 32).transpose(1, 2).contiguous()
            out = torch.empty((b, n, n, 128), dtype=dtype, device=dev)
            _lib.check(lib.mf_opm_fused_fwd(Ap.data_ptr(), Bp.data_ptr(), wp.data_ptr(),
                                            bias.to(dtype).data_ptr() if bias is not None else None,
                                            out.data_ptr(), b, n, _lib.dtype_code(dtype), stream), "mf_opm_fused_fwd")
        ctx.save_for_backward(Ap, Bp, weight, bias, row_scale, pos)
        ctx.dims = (b, s, n, hidden.shape[-1])
        return out

    @staticmethod
    def backward(ctx, dout):
        Ap, Bp, weight, bias, row_scale, pos = ctx.saved_tensors
        b, s, n, width = ctx.dims
        dh, dtype, dev = 32, Ap.dtype, Ap.device
        dout2 = dout.reshape(b * n * n, 128).to(dtype).contiguous()
        w = weight.to(dtype)
        lib = _lib.lib()
        with torch.cuda.device(dev):
            stream = torch.cuda.current_stream(dev).cuda_stream
            code = _lib.dtype_code(dtype)
            # weight gradient: the outer blocks are formed again tile by tile inside mf_opm_dw, never stored;
            # the kernel returns [e * 32 + d, channel] in fp32
            nbytes = max(lib.mf_opm_dw_workspace_bytes(b, n), lib.mf_opm_dab_workspace_bytes(b, n))
            ws = torch.empty(nbytes, dtype=torch.uint8, device=dev)
            dwt = torch.empty((dh * dh, 128), dtype=torch.float32, device=dev)
            _lib.check(lib.mf_opm_dw(Ap.data_ptr(), Bp.data_ptr(), dout2.data_ptr(), dwt.data_ptr(), ws.data_ptr(), nbytes,
                                     b, n, code, stream), "mf_opm_dw")
            # operand gradients: tiles of dOut . W^T live in LDS between two products inside mf_opm_dab (once per side)
            wt_a = w.t().contiguous()                                                        # row d * 32 + e
            wt_b = w.view(128, dh, dh).permute(2, 1, 0).reshape(dh * dh, 128).contiguous()   # row e * 32 + d
            dAp, dBp = torch.empty_like(Ap), torch.empty_like(Bp)
            _lib.check(lib.mf_opm_dab(dout2.data_ptr(), wt_a.data_ptr(), Bp.data_ptr(), dAp.data_ptr(), ws.data_ptr(), nbytes,
                                      b, n, 0, code, stream), "mf_opm_dab")
            _lib.check(lib.mf_opm_dab(dout2.data_ptr(), wt_b.data_ptr(), Ap.data_ptr(), dBp.data_ptr(), ws.data_ptr(), nbytes,
                                      b, n, 1, code, stream), "mf_opm_dab")
            dhidden = torch.empty((b, s, n, width), dtype=dtype, device=dev)
            _lib.check(lib.mf_opm_pack(dhidden.data_ptr(), width, row_scale.data_ptr(),
                                       pos.data_ptr() if pos is not None else None, dAp.data_ptr(), dBp.data_ptr(),
                                       b, s, n, 1, code, stream), "mf_opm_pack")
        dW = dwt.view(dh, dh, 128).permute(2, 1, 0).reshape(128, dh * dh)          # [channel, d * 32 + e]
        dbias = dout2.sum(0, dtype=torch.float32).to(bias.dtype) if bias is not None else None
        return dhidden, None, None, dW.to(weight.dtype), dbias
