"""Triangle multiplication around the fused kernels (MI355X).

Drop-in for ``TriangleMultiplication(dim=..., dim_hidden=..., mix=...)`` of the reference
(megafold/model/megafold.py:416-493) as ``PairwiseBlock`` builds it (megafold.py:688-701).  Parameter names and
shapes are the reference's (``combined`` and ``to_out.0`` are its ``LayernormLinear`` modules), so its
checkpoints load unchanged::

    combined.WEIGHT, combined.BIAS [dim]; combined.linear_weight [dim, 5*dh]; combined.linear_bias [5*dh]
    to_out.0.WEIGHT, to_out.0.BIAS [dh];  to_out.0.linear_weight [dh, dim]

What runs, per call (one ``torch.autograd.Function``, nothing channel-last is ever permuted by PyTorch):

1. fused LayerNorm -> Linear ``dim -> 5*dh`` (``mf_lnlinear_fwd``): ``Y = [values (2dh) | gates (2dh) | out gate (dh)]``;
2. ``mf_trimul_pack_fwd``: GLU, pair mask and the move to channel-first operand matrices in one pass over Y
   (the reference runs glu, chunk, two mask multiplies and lets einsum permute);
3. the contraction as ONE batched GEMM over the ``b * dh`` channels (BLAS library);
4. ``mf_channels_first_to_last`` back to rows, fused LayerNorm -> Linear ``dh -> dim``, and the sigmoid output
   gate read in place from Y's last columns (``mf_sigmoid_gate_fwd``).

Widths other than 64 and 128 run the same expression from the two fused LayerNorm -> Linear
modules and PyTorch operations on the GPU (``TriangleMultiplication._composed``).

Backward mirrors it with ``mf_sigmoid_gate_bwd``, ``mf_lnlinear_bwd``, ``mf_channels_last_to_first``, two batched
GEMMs, ``mf_trimul_pack_bwd`` (GLU and mask backward fused into the move back, written straight into the
columns of dY) and one ``mf_lnlinear_bwd``.
"""
from __future__ import annotations

import ctypes as C
from typing import Optional

import torch
import torch.nn as nn

from ... import _lib
from ..FusedLayernormLinear.fused_layernorm_linear import (LayernormLinear, fused_shape_supported,
                                                           layernorm_linear_backward, layernorm_linear_forward)
from ..FusedTriangleAttention.triangle_attention import Dropout, sigmoid_gate_backward, sigmoid_gate_forward

__all__ = ["TriangleMultiplication", "TriangleMultiplicationFunction", "trimul_pack_forward",
           "trimul_pack_backward", "channels_last_to_first", "channels_first_to_last"]


def _round8(n: int) -> int:
    return (n + 7) // 8 * 8


def _tm_args(b, n, dh, dtype, device, incoming):
    a = _lib.TriMulArgs()
    a.B, a.n, a.np, a.dh = b, n, _round8(n), dh
    a.dtype = _lib.dtype_code(dtype)
    a.transposed = a.swap = 1 if incoming else 0
    a.stream = torch.cuda.current_stream(device).cuda_stream
    return a


def _new_p(sets, b, dh, n, like):
    npad = _round8(n)
    # rows / columns past n must be zero: the kernels write the column padding of the rows they touch
    alloc = torch.empty if npad == n else torch.zeros
    return alloc((sets, b * dh, npad, npad), dtype=like.dtype, device=like.device)


def _mask_ptr(mask, b, n):
    if mask is None:
        return None, None
    m = mask.to(torch.bool).contiguous()
    assert tuple(m.shape) == (b, n)
    return m, m.data_ptr()


def trimul_pack_forward(Y, mask, b, n, dh, incoming):
    """``(left | right) = Y[:, :2dh] * sigmoid(Y[:, 2dh:4dh]) * pair_mask`` as channel-first operand matrices
    ``P [2, b*dh, np, np]`` with ``einsum = bmm(P[0], P[1]^T)`` (megafold/model/megafold.py:476-483)."""
    P = _new_p(2, b, dh, n, Y)
    a = _tm_args(b, n, dh, Y.dtype, Y.device, incoming)
    a.y, a.ldy = Y.data_ptr(), Y.stride(0)
    keep, a.mask = _mask_ptr(mask, b, n)
    a.p = P.data_ptr()
    with torch.cuda.device(Y.device):
        _lib.check(_lib.lib().mf_trimul_pack_fwd(C.byref(a)), "mf_trimul_pack_fwd")
    return P


def trimul_pack_backward(dP, Y, mask, dY, b, n, dh, incoming):
    """Gradients of Y's value and gate columns (written into ``dY[:, :4dh]``) from the gradients ``dP`` of the
    two operand matrices."""
    a = _tm_args(b, n, dh, Y.dtype, Y.device, incoming)
    a.y, a.ldy = Y.data_ptr(), Y.stride(0)
    a.dy, a.lddy = dY.data_ptr(), dY.stride(0)
    keep, a.mask = _mask_ptr(mask, b, n)
    a.p = dP.data_ptr()
    with torch.cuda.device(Y.device):
        _lib.check(_lib.lib().mf_trimul_pack_bwd(C.byref(a)), "mf_trimul_pack_bwd")


def channels_first_to_last(Pc, b, n, dh):
    """``[b*dh, np, np]`` channel-first matrices -> ``[b*n*n, dh]`` rows."""
    out = torch.empty((b * n * n, dh), dtype=Pc.dtype, device=Pc.device)
    a = _tm_args(b, n, dh, Pc.dtype, Pc.device, False)
    a.dy, a.lddy = out.data_ptr(), out.stride(0)
    a.p = Pc.data_ptr()
    with torch.cuda.device(Pc.device):
        _lib.check(_lib.lib().mf_channels_first_to_last(C.byref(a)), "mf_channels_first_to_last")
    return out


def channels_last_to_first(X2d, b, n, dh):
    """``[b*n*n, dh]`` rows -> ``[b*dh, np, np]`` channel-first matrices, zero padded."""
    P = _new_p(1, b, dh, n, X2d)
    a = _tm_args(b, n, dh, X2d.dtype, X2d.device, False)
    a.y, a.ldy = X2d.data_ptr(), X2d.stride(0)
    a.p = P.data_ptr()
    with torch.cuda.device(X2d.device):
        _lib.check(_lib.lib().mf_channels_last_to_first(C.byref(a)), "mf_channels_last_to_first")
    return P[0]


class TriangleMultiplicationFunction(torch.autograd.Function):
    """x ``[b, n, n, d]`` -> block output ``[b, n, n, d]`` (before dropout)."""

    @staticmethod
    @torch.amp.custom_fwd(device_type="cuda", cast_inputs=torch.bfloat16)
    def forward(ctx, x, mask, g1, b1, W1, lb1, g2, b2, W2, incoming, add_residual=False):
        b, n, n2, d = x.shape
        assert n == n2, "pairwise representation must be [b, n, n, d]"
        dh = W2.shape[0]
        assert W1.shape == (d, 5 * dh) and W2.shape[1] == d and dh == d, "dim_hidden must equal dim"
        M = b * n * n
        x2d = x.contiguous().view(M, d)
        Y, _, W1c, Mean1, RSTD1 = layernorm_linear_forward(x2d, W1, lb1, g1, b1, True, lb1 is not None)
        P = trimul_pack_forward(Y, mask, b, n, dh, incoming)
        out_cf = torch.bmm(P[0], P[1].transpose(1, 2))                    # [b*dh, np, np]
        out_cl = channels_first_to_last(out_cf, b, n, dh)                 # [M, dh]
        Z, _, W2c, Mean2, RSTD2 = layernorm_linear_forward(out_cl, W2, None, g2, b2, True, False)
        res = sigmoid_gate_forward(Z, Y[:, 4 * dh:], x2d if add_residual else None)   # (+ x: the block's x + f(x))
        ctx.add_residual = add_residual
        ctx.save_for_backward(x2d, Y, P, out_cl, Z, Mean1, RSTD1, Mean2, RSTD2, W1c, W2c, g1, b1, g2, b2,
                              mask if mask is not None else x.new_empty(0))
        ctx.dims = (b, n, d, dh, incoming, mask is not None, lb1 is not None)
        return res.view(b, n, n, d)

    @staticmethod
    @torch.amp.custom_bwd(device_type="cuda")
    def backward(ctx, dres):
        x2d, Y, P, out_cl, Z, Mean1, RSTD1, Mean2, RSTD2, W1c, W2c, g1, b1, g2, b2, mask = ctx.saved_tensors
        b, n, d, dh, incoming, has_mask, has_lb = ctx.dims
        mask = mask if has_mask else None
        M = b * n * n
        dres2d = dres.to(x2d.dtype).reshape(M, d)
        dY = torch.empty_like(Y)
        dZ, _ = sigmoid_gate_backward(dres2d, Z, Y[:, 4 * dh:], dY[:, 4 * dh:], need_product=False)
        d_out_cl, dW2, _, dg2, db2 = layernorm_linear_backward(dZ, out_cl, W2c, Mean2, RSTD2, g2, b2, True, False)
        d_out_cf = channels_last_to_first(d_out_cl, b, n, dh)             # [b*dh, np, np], zero padded
        dP = torch.empty_like(P)
        torch.bmm(d_out_cf, P[1], out=dP[0])                              # d(P0) = dOut P1
        torch.bmm(d_out_cf.transpose(1, 2), P[0], out=dP[1])              # d(P1) = dOut^T P0
        trimul_pack_backward(dP, Y, mask, dY, b, n, dh, incoming)
        dX, dW1, dlb1, dg1, db1 = layernorm_linear_backward(dY, x2d, W1c, Mean1, RSTD1, g1, b1, True, has_lb,
                                                            dx_add=dres2d if ctx.add_residual else None)
        return dX.view(b, n, n, d), None, dg1, db1, dW1, dlb1, dg2, db2, dW2, None, None


class TriangleMultiplication(nn.Module):
    """``forward(x [b, n, n, d], mask [b, n] bool or None) -> [b, n, n, d]``; the caller adds the residual
    (megafold.py:742-743), or asks for it with ``add_residual=True``: the sums of ``x + block(x)`` are then folded
    into the block's last forward and last backward kernel (needs the dropout to be inactive: the reference drops
    before it adds)."""

    def __init__(self, *, dim, dim_hidden=None, mix="incoming", dropout=0.0, dropout_type=None):
        super().__init__()
        dim_hidden = dim if dim_hidden is None else dim_hidden
        assert mix in ("incoming", "outgoing")
        self.dim_hidden = dim_hidden
        self.mix = mix
        self.combined = LayernormLinear(dim, dim_hidden * 5)
        self.to_out = nn.Sequential(LayernormLinear(dim_hidden, dim, has_linear_bias=False),
                                    Dropout(dropout, dropout_type=dropout_type))

    def _composed(self, x: torch.Tensor, mask: Optional[torch.Tensor]) -> torch.Tensor:
        """The block for the widths the layout kernels do not take (they move rows of 64 or 128 hidden channels): the two ``LayernormLinear`` modules as they are, and the gated-linear unit, pair mask,
        contraction and output gate of megafold.py:475-491 as PyTorch operations on the GPU, with PyTorch's autograd."""
        dh = self.dim_hidden
        y = self.combined(x)
        gate = torch.sigmoid(y[..., 4 * dh:])
        left, right = torch.nn.functional.glu(y[..., :4 * dh], dim=-1).chunk(2, dim=-1)
        if mask is not None:
            keep = (mask[:, :, None] & mask[:, None, :]).unsqueeze(-1).to(left.dtype)
            left, right = left * keep, right * keep
        eq = "bikd,bjkd->bijd" if self.mix == "outgoing" else "bkjd,bkid->bijd"
        out = torch.einsum(eq, left, right).contiguous()
        return self.to_out[0](out) * gate

    def forward(self, x: torch.Tensor, mask: Optional[torch.Tensor] = None, add_residual: bool = False) -> torch.Tensor:
        dim, dh = x.shape[-1], self.dim_hidden
        dtype = torch.bfloat16 if torch.is_autocast_enabled() else x.dtype
        if not x.is_cuda:
            raise RuntimeError("TriangleMultiplication runs on the GPU only (got device %s)" % x.device)
        if dh != dim:        # the reference multiplies the [.., dim] projection by a [.., dim_hidden] gate (megafold.py:491)
            raise ValueError("dim_hidden (%d) must equal dim (%d): the output gate has dim_hidden columns" % (dh, dim))
        if dh not in (64, 128) or not fused_shape_supported(dim, 5 * dh, dtype):
            out = self._composed(x, mask)         # other widths: the same expression from the module's own parts
            out = self.to_out[1](out)
            return out + x if add_residual else out
        c, o = self.combined, self.to_out[0]
        drop = self.to_out[1]
        # the fused sum adds in the compute dtype: under autocast an fp32 residual stream stays fp32 (x + block(x)
        # promotes, as in the reference, megafold.py:742-743), so it takes the separate add
        fused_sum = add_residual and not (drop.training and drop.dropout.p > 0.0) and x.dtype == dtype
        out = TriangleMultiplicationFunction.apply(x, mask, c.WEIGHT, c.BIAS, c.linear_weight, c.linear_bias,
                                                   o.WEIGHT, o.BIAS, o.linear_weight, self.mix == "incoming", fused_sum)
        if fused_sum:
            return out
        out = drop(out)
        return out + x if add_residual else out
