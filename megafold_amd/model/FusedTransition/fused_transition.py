"""Fused LayerNorm -> SwiGLU Transition on MI355X.

Drop-in for the reference module ``megafold/model/FusedTransition/fused_transition.py``:
``FusedTransition`` (fused_transition.py:118-151), ``FusedSwiGLU`` / ``FusedSwiGLUFunction`` (:96-116) and
the host functions ``swiglu_forward`` / ``swiglu_backward`` (:55-93).  Parameter layout is unchanged
(``ff.0`` LayernormLinear or LayerNorm/Linear, ``ff.2`` / ``ff.3`` output Linear), so checkpoints load.

``SwiGLU(u) = silu(u[..., d:]) * u[..., :d]`` — the gate is the SECOND half (fused_transition.py:22-24).

With ``include_ln`` and ``use_layernormlinear`` (the form the Pairformer uses) the first three stages
run as ONE kernel: LayerNorm statistics in the GEMM prologue, SwiGLU in its epilogue, so the
``[M, 2*dim_inner]`` pre-activation is never written; the backward recomputes it tile by tile.
The other variants use the stand-alone SwiGLU kernels (``mf_swiglu_fwd`` / ``mf_swiglu_bwd``).
"""
from __future__ import annotations

import torch
import torch.nn as nn

from ... import _lib
from ..FusedLayernormLinear.fused_layernorm_linear import (LayernormLinear, fused_shape_supported,
                                                           layernorm_linear_backward, layernorm_linear_forward)
from ..linear import linear_no_bias, tall_skinny_tn

__all__ = ["FusedTransition", "FusedSwiGLU", "FusedSwiGLUFunction", "swiglu_forward", "swiglu_backward"]

_FLOATS = (torch.float32, torch.float16, torch.bfloat16)


def _check(x):
    if not x.is_cuda:
        raise RuntimeError("FusedSwiGLU runs on the GPU only (got device %s)" % x.device)
    if x.dtype not in _FLOATS:
        raise TypeError("unsupported dtype %s" % x.dtype)


def swiglu_forward(x):
    """x = [left, right] -> (x2d, silu(right) * left), as the reference (fused_transition.py:55-75)."""
    _check(x)
    ori_shape = x.shape
    D = ori_shape[-1]
    dim_out = D // 2
    if D % 16 != 0:
        raise ValueError("SwiGLU needs a last dimension that is a multiple of 16, got %d" % D)
    x2 = x.reshape(-1, D).contiguous()
    M = x2.shape[0]
    with torch.cuda.device(x.device):
        y = torch.empty((M, dim_out), device=x.device, dtype=x.dtype)
        rc = _lib.lib().mf_swiglu_fwd(x2.data_ptr(), y.data_ptr(), M, dim_out, _lib.dtype_code(x.dtype),
                                      torch.cuda.current_stream(x.device).cuda_stream)
        _lib.check(rc, "mf_swiglu_fwd")
    return x2, y.view(ori_shape[:-1] + (dim_out,))


def swiglu_backward(x, dy):
    """dy -> [dleft, dright] (fused_transition.py:78-93).  A new tensor is returned; the saved input
    is not overwritten."""
    ori_shape = dy.shape
    D = ori_shape[-1]
    dy2 = dy.reshape(-1, D)
    if dy2.dtype != x.dtype:
        dy2 = dy2.to(x.dtype)
    dy2 = dy2.contiguous()
    M = dy2.shape[0]
    with torch.cuda.device(x.device):
        dx = torch.empty_like(x)
        rc = _lib.lib().mf_swiglu_bwd(dy2.data_ptr(), x.data_ptr(), dx.data_ptr(), M, D, _lib.dtype_code(x.dtype),
                                      torch.cuda.current_stream(x.device).cuda_stream)
        _lib.check(rc, "mf_swiglu_bwd")
    return dx.view(ori_shape[:-1] + (D * 2,))


class FusedSwiGLUFunction(torch.autograd.Function):
    @staticmethod
    @torch.amp.custom_fwd(device_type="cuda", cast_inputs=torch.bfloat16)
    def forward(ctx, input):
        x2, output = swiglu_forward(input)
        ctx.save_for_backward(x2)
        ctx.in_shape = input.shape
        return output

    @staticmethod
    @torch.amp.custom_bwd(device_type="cuda")
    def backward(ctx, grad_output):
        (x2,) = ctx.saved_tensors
        return swiglu_backward(x2, grad_output).view(ctx.in_shape)


class FusedSwiGLU(nn.Module):
    def forward(self, x):
        return FusedSwiGLUFunction.apply(x)


class _TransitionResidualFunction(torch.autograd.Function):
    """``x + Linear(SwiGLU(Linear(LayerNorm(x))))`` (megafold.py:747 around fused_transition.py:128-131) as one
    function, so that the backward sum ``d(x) = d(transition) + d(out)`` is taken inside the LayerNorm backward's
    dx kernel (``dx_add``) instead of by a pass of its own.  The kernels are those of the module's plain path."""

    @staticmethod
    @torch.amp.custom_fwd(device_type="cuda", cast_inputs=torch.bfloat16)
    def forward(ctx, x, ln_w, ln_b, W1, W2):
        x = x.contiguous()
        h, x2d, W1c, Mean, RSTD = layernorm_linear_forward(x, W1, None, ln_w, ln_b, True, False, act=_lib.MF_ACT_SWIGLU)
        w2 = W2 if W2.dtype == x.dtype else W2.to(x.dtype)
        out = torch.nn.functional.linear(h, w2)
        out += x
        ctx.save_for_backward(x2d, W1c, Mean, RSTD, ln_w, ln_b, h, w2)
        return out

    @staticmethod
    @torch.amp.custom_bwd(device_type="cuda")
    def backward(ctx, dout):
        x2d, W1c, Mean, RSTD, ln_w, ln_b, h, w2 = ctx.saved_tensors
        d2 = dout.reshape(-1, dout.shape[-1])
        d2 = (d2 if d2.dtype == x2d.dtype else d2.to(x2d.dtype)).contiguous()
        dh = d2 @ w2
        dW2 = tall_skinny_tn(d2, h.reshape(-1, h.shape[-1]))
        dX, dW1, _, dlnw, dlnb = layernorm_linear_backward(dh, x2d, W1c, Mean, RSTD, ln_w, ln_b, True, False,
                                                           act=_lib.MF_ACT_SWIGLU, dx_add=d2)
        return dX.view(dout.shape), dlnw, dlnb, dW1, dW2


class FusedTransition(nn.Module):
    def __init__(self, dim, expansion_factor=4, include_ln=True, use_layernormlinear=True, device=None, dtype=None):
        factory_kwargs = {"device": device, "dtype": dtype}
        super().__init__()
        self.dim = dim
        dim_inner = int(dim * expansion_factor)
        self.dim_inner = dim_inner
        self._fused_ln_swiglu = bool(include_ln and use_layernormlinear)
        if include_ln:
            if use_layernormlinear:
                self.ff = nn.Sequential(
                    LayernormLinear(dim, dim_inner * 2, has_linear_bias=False, **factory_kwargs),
                    FusedSwiGLU(),
                    nn.Linear(dim_inner, dim, bias=False, **factory_kwargs),
                )
            else:
                self.ff = nn.Sequential(
                    nn.LayerNorm(dim, **factory_kwargs),
                    nn.Linear(dim, dim_inner * 2, bias=False, **factory_kwargs),
                    FusedSwiGLU(),
                    nn.Linear(dim_inner, dim, bias=False, **factory_kwargs),
                )
        else:
            self.ff = nn.Sequential(
                nn.Linear(dim, dim_inner * 2, bias=False, **factory_kwargs),
                FusedSwiGLU(),
                nn.Linear(dim_inner, dim, bias=False, **factory_kwargs),
            )

    def forward(self, input, add_residual=False):
        # the output projection (ff[-1], a bias-free nn.Linear) runs through linear_no_bias: same GEMMs,
        # but a weight gradient that is split along the long row axis.  add_residual: input + transition(input)
        # (megafold.py:747); on the fused path one function whose backward takes the sum inside its dx kernel
        if self._fused_ln_swiglu and add_residual and input.is_cuda:
            ln = self.ff[0]
            dtype = torch.bfloat16 if torch.is_autocast_enabled() else input.dtype
            # (an fp32 stream under autocast keeps its separate fp32 add, as the reference's `x + f(x)` promotes)
            if input.dtype == dtype and fused_shape_supported(ln.K, ln.N, dtype, _lib.MF_ACT_SWIGLU):
                return _TransitionResidualFunction.apply(input, ln.WEIGHT, ln.BIAS, ln.linear_weight, self.ff[2].weight)
        if self._fused_ln_swiglu:
            # LayerNorm -> Linear -> SwiGLU in one kernel, then the output projection
            out = linear_no_bias(self.ff[0](input, act=_lib.MF_ACT_SWIGLU), self.ff[2].weight)
        else:
            h = input
            for layer in list(self.ff)[:-1]:
                h = layer(h)
            out = linear_no_bias(h, self.ff[-1].weight)
        return out + input if add_residual else out

    def extra_repr(self):
        return f"dim={self.dim}, dim_inner={self.dim_inner}"
