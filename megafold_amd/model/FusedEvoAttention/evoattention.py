"""Pair-biased, key-masked attention ("EvoAttention") on MI355X.

Drop-in for the reference module ``megafold/model/FusedEvoAttention/evoattention.py``:
``TritonEvoformer(Q, K, V, res_mask, pair_bias) -> O`` (evoattention.py:905) and the
``EvoformerAttention`` autograd function behind it (evoattention.py:688-903).  The name
``TritonEvoformer`` is kept so call sites (``megafold/model/attention.py:489``) need no change; there
is no Triton here, the work is done by HIP kernels reached through ``mf_evoattn_fwd`` /
``mf_evoattn_bwd``.

Shapes (evoattention.py:691-693)::

    Q, K, V    [B, N, S, H, D]      O [B, N, S, H, D] in Q's dtype
    res_mask   [B, N, 1, 1, S]      added to the logits (0 / -1e9 / -inf); bool = keep-mask
    pair_bias  [B, 1, H, S, S]

Differences from the reference, all on purpose:

* Q, K, V, dO are consumed in place through their strides and O, dQ, dK, dV are written in the API
  layout, so the eight ``transpose(-2, -3).contiguous()`` copies (evoattention.py:700-702, 777, 787,
  899-901) do not exist and nothing transposed is kept for backward.
* Size-1 batch / row dimensions of ``res_mask`` and ``pair_bias`` broadcast.
* A ``bool`` mask is a keep-mask (True = attend).  The reference would add 0/1 to the logits
  (evoattention.py:66), which masks nothing.
* A query row whose keys are all ``-inf`` gives O = 0 and zero gradients instead of NaN.
* The bias gradient is reduced in a fixed order without atomics (bitwise reproducible).
"""
from __future__ import annotations

import ctypes as C

import torch

from ... import _lib

# Default of evoattention_backward's ``lean``: trade one more pass over dO and O for a workspace without the bias
# gradient's partial sums (peak activation memory inside the O(N S H D) bound + the bias tiles).
MEMORY_LEAN = False

__all__ = ["EvoformerAttention", "TritonEvoformer", "evoattention_forward", "evoattention_backward",
           "evoattention_forward_noalloc"]

_FLOATS = (torch.float32, torch.float16, torch.bfloat16)


def _strided_ok(t: torch.Tensor) -> bool:
    """Kernel requirement: unit stride on D, other strides multiples of 16 bytes, base aligned."""
    unit = 16 // t.element_size()
    return (t.stride(-1) == 1 and all(s % unit == 0 for s in t.stride()[:-1]) and t.data_ptr() % 16 == 0)


def _prep_qkv(t: torch.Tensor) -> torch.Tensor:
    return t if _strided_ok(t) else t.contiguous()


def _prep_mask(res_mask: torch.Tensor, B: int, N: int, S: int) -> torch.Tensor:
    if res_mask.dim() != 5 or res_mask.shape[2] != 1 or res_mask.shape[3] != 1 or res_mask.shape[4] != S:
        raise ValueError("res_mask must be [B, N, 1, 1, S], got %s" % (tuple(res_mask.shape),))
    if res_mask.dtype not in _FLOATS and res_mask.dtype != torch.bool:
        res_mask = res_mask.to(torch.float32)
    return res_mask.expand(B, N, 1, 1, S)


def _prep_bias(pair_bias: torch.Tensor, B: int, H: int, S: int) -> torch.Tensor:
    if pair_bias.dim() != 5 or pair_bias.shape[1] != 1 or tuple(pair_bias.shape[2:]) != (H, S, S):
        raise ValueError("pair_bias must be [B, 1, H, S, S], got %s" % (tuple(pair_bias.shape),))
    if pair_bias.dtype not in _FLOATS:
        pair_bias = pair_bias.to(torch.float32)
    return pair_bias.expand(B, 1, H, S, S)


def _fill_common(a: _lib.EvoAttnArgs, Q, K, V, mask, bias, O, lse) -> None:
    B, N, S, H, D = Q.shape
    a.B, a.N, a.S, a.H, a.D = B, N, S, H, D
    a.dtype = _lib.dtype_code(Q.dtype)
    a.bias_dtype = _lib.dtype_code(bias.dtype)
    a.mask_dtype = _lib.dtype_code(mask.dtype)
    a.scale = float(D) ** -0.5  # evoattention.py:705
    a.q, a.k, a.v, a.o = Q.data_ptr(), K.data_ptr(), V.data_ptr(), O.data_ptr()
    a.bias, a.mask, a.lse = bias.data_ptr(), mask.data_ptr(), lse.data_ptr()
    a.q_stride = _lib.I64x4(*Q.stride()[:4])
    a.k_stride = _lib.I64x4(*K.stride()[:4])
    a.v_stride = _lib.I64x4(*V.stride()[:4])
    a.o_stride = _lib.I64x4(*O.stride()[:4])
    bs = bias.stride()
    a.bias_stride = _lib.I64x4(bs[0], bs[2], bs[3], bs[4])
    ms = mask.stride()
    a.mask_stride = _lib.I64x3(ms[0], ms[1], ms[4])
    a.stream = torch.cuda.current_stream(Q.device).cuda_stream


def _check_inputs(Q, K, V) -> None:
    if Q.dim() != 5:
        raise ValueError("Q must be [B, N, S, H, D], got %s" % (tuple(Q.shape),))
    # the reference asserts equal head dims (evoattention.py:695-696)
    assert Q.shape[-1] == K.shape[-1] and K.shape[-1] == V.shape[-1]
    if K.shape != Q.shape or V.shape != Q.shape:
        raise ValueError("Q, K, V must have the same shape")
    if Q.dtype not in _FLOATS or K.dtype != Q.dtype or V.dtype != Q.dtype:
        raise TypeError("Q, K, V must share one of float32 / float16 / bfloat16")
    if not Q.is_cuda:
        raise RuntimeError("EvoformerAttention runs on the GPU only (got device %s)" % Q.device)


def evoattention_forward(Q, K, V, res_mask, pair_bias, out=None, save_bias_tiles=False):
    """O, LSE = forward.  Returns also the tensors exactly as the kernels saw them.  ``out``: optional
    ``[B, N, S, H, D]`` tensor to receive O (any strides the kernels accept, e.g. a transposed view).
    ``save_bias_tiles``: the forward's bias preparation also writes the tiled copy the backward reads; it is
    returned as a sixth saved tensor, to be passed to ``evoattention_backward(..., bias_tiles=)``, which then skips
    its own preparation launch (the copy replaces the same number of bytes in the backward's workspace)."""
    _check_inputs(Q, K, V)
    B, N, S, H, D = Q.shape
    if out is not None and (tuple(out.shape) != (B, N, S, H, D) or out.dtype != Q.dtype or not _strided_ok(out)):
        raise ValueError("out must be [B, N, S, H, D] in Q's dtype with unit stride on D and 16-byte multiples elsewhere")
    Q, K, V = _prep_qkv(Q), _prep_qkv(K), _prep_qkv(V)
    mask = _prep_mask(res_mask, B, N, S)
    bias = _prep_bias(pair_bias, B, H, S)
    lib = _lib.lib()
    with torch.cuda.device(Q.device):
        O = out if out is not None else torch.empty((B, N, S, H, D), dtype=Q.dtype, device=Q.device)
        lse = torch.empty((B, N, H, S), dtype=torch.float32, device=Q.device)
        a = _lib.EvoAttnArgs()
        _fill_common(a, Q, K, V, mask, bias, O, lse)
        nbytes = lib.mf_evoattn_fwd_workspace_bytes(C.byref(a))
        ws = torch.empty(nbytes, dtype=torch.uint8, device=Q.device) if nbytes else None
        a.workspace = ws.data_ptr() if ws is not None else None
        a.workspace_bytes = nbytes
        tiles = None
        if save_bias_tiles:
            tiles = torch.empty(lib.mf_evoattn_bias_tiles_bytes(C.byref(a)), dtype=torch.uint8, device=Q.device)
            a.bias_tiles_bwd = tiles.data_ptr()
        _lib.check(lib.mf_evoattn_fwd(C.byref(a)), "mf_evoattn_fwd")
    if save_bias_tiles:
        return O, lse, (Q, K, V, mask, bias, tiles)
    return O, lse, (Q, K, V, mask, bias)


def evoattention_forward_noalloc(Q, K, V, res_mask, pair_bias, O, lse) -> None:
    """Forward into caller-provided ``O`` ``[B, N, S, H, D]`` and ``lse`` ``[B, N, H, S]`` (fp32, contiguous)
    through ``mf_evoattn_fwd_noalloc``: no device memory is allocated, neither here nor in the library (its
    scratch is a fixed array inside the library, which limits the problem to ``B * H * ceil(S/32)**2 <= 4096``).
    For callers that must not allocate, e.g. while a HIP graph is being captured.  Q, K, V must already
    satisfy the kernels' stride rules (unit stride on D, other strides multiples of 16 bytes)."""
    _check_inputs(Q, K, V)
    B, N, S, H, D = Q.shape
    if not (_strided_ok(Q) and _strided_ok(K) and _strided_ok(V) and _strided_ok(O)):
        raise ValueError("Q, K, V, O must have unit stride on D and 16-byte multiples elsewhere")
    if tuple(O.shape) != (B, N, S, H, D) or O.dtype != Q.dtype:
        raise ValueError("O must be [B, N, S, H, D] in Q's dtype")
    if tuple(lse.shape) != (B, N, H, S) or lse.dtype != torch.float32 or not lse.is_contiguous():
        raise ValueError("lse must be a contiguous fp32 [B, N, H, S] tensor")
    mask = _prep_mask(res_mask, B, N, S)
    bias = _prep_bias(pair_bias, B, H, S)
    a = _lib.EvoAttnArgs()
    _fill_common(a, Q, K, V, mask, bias, O, lse)
    with torch.cuda.device(Q.device):
        _lib.check(_lib.lib().mf_evoattn_fwd_noalloc(C.byref(a)), "mf_evoattn_fwd_noalloc")


def evoattention_backward(dO, Q, K, V, mask, bias, O, lse, need_dbias=True, phase_hook=None, out=None, bias_tiles=None,
                          lean=None):
    """dQ, dK, dV, dBias(fp32 [B, 1, H, S, S] or None) from the saved forward state.

    ``out = (dQ, dK, dV)``, if given, are the tensors to write (``[B, N, S, H, D]`` in Q's dtype, unit
    stride on D and 16-byte multiples elsewhere, e.g. column slices of a wider matrix); otherwise
    contiguous tensors are allocated.  ``bias_tiles``: the sixth saved tensor of
    ``evoattention_forward(..., save_bias_tiles=True)`` for the same inputs.  ``lean`` (default: the module-level
    ``MEMORY_LEAN``): the memory-lean order of ``MF_EVO_BWD_LEAN`` where the library can use it (bias gradient wanted,
    contiguous dQ large enough for its partial sums) — the bias gradient runs first with its partial sums in the dQ
    buffer, at the price of one more pass over dO and O.

    ``phase_hook(name)``, if given, is called before and after each backward phase ("prep", "dqkv",
    "dbias"), which are then enqueued by separate C-ABI calls (used by the benchmark to bracket each
    kernel with events on the launch stream)."""
    B, N, S, H, D = Q.shape
    if dO.dtype != Q.dtype:
        dO = dO.to(Q.dtype)
    dO = _prep_qkv(dO)
    lib = _lib.lib()
    with torch.cuda.device(Q.device):
        if out is None:
            dQ = torch.empty((B, N, S, H, D), dtype=Q.dtype, device=Q.device)
            dK = torch.empty_like(dQ)
            dV = torch.empty_like(dQ)
        else:
            dQ, dK, dV = out
            for t in out:
                if tuple(t.shape) != (B, N, S, H, D) or t.dtype != Q.dtype or not _strided_ok(t):
                    raise ValueError("out tensors must be [B, N, S, H, D] in Q's dtype with kernel-compatible strides")
        dbias = torch.empty((B, 1, H, S, S), dtype=torch.float32, device=Q.device) if need_dbias else None
        a = _lib.EvoAttnArgs()
        _fill_common(a, Q, K, V, mask, bias, O, lse)
        a.dO, a.dq, a.dk, a.dv = dO.data_ptr(), dQ.data_ptr(), dK.data_ptr(), dV.data_ptr()
        a.dbias = dbias.data_ptr() if dbias is not None else None
        a.do_stride = _lib.I64x4(*dO.stride()[:4])
        a.dq_stride = _lib.I64x4(*dQ.stride()[:4])
        a.dk_stride = _lib.I64x4(*dK.stride()[:4])
        a.dv_stride = _lib.I64x4(*dV.stride()[:4])
        if bias_tiles is not None:
            a.bias_tiles_bwd = bias_tiles.data_ptr()
        lean = MEMORY_LEAN if lean is None else lean
        lean_bit = _lib.MF_EVO_BWD_LEAN if (lean and dbias is not None and lib.mf_evoattn_bwd_lean_ok(C.byref(a))) else 0
        a.phases = lean_bit
        nbytes = lib.mf_evoattn_bwd_workspace_bytes(C.byref(a))
        ws = torch.empty(max(nbytes, 16), dtype=torch.uint8, device=Q.device)
        a.workspace = ws.data_ptr()
        a.workspace_bytes = nbytes
        if phase_hook is None:
            _lib.check(lib.mf_evoattn_bwd(C.byref(a)), "mf_evoattn_bwd")
        else:
            order = (("prep", _lib.MF_EVO_BWD_PREP), ("dqkv", _lib.MF_EVO_BWD_DQKV), ("dbias", _lib.MF_EVO_BWD_DBIAS))
            if lean_bit:
                order = (order[0], order[2], order[1])
            for name, bit in order:
                if bit == _lib.MF_EVO_BWD_DBIAS and dbias is None:
                    continue
                a.phases = bit | lean_bit
                phase_hook(name)
                _lib.check(lib.mf_evoattn_bwd(C.byref(a)), "mf_evoattn_bwd[%s]" % name)
                phase_hook(name)
    return dQ, dK, dV, dbias


class EvoformerAttention(torch.autograd.Function):
    """Same contract as the reference class of this name (evoattention.py:688-903)."""

    @staticmethod
    def forward(ctx, Q, K, V, res_mask, pair_bias):
        O, lse, (Qs, Ks, Vs, mask, bias, tiles) = evoattention_forward(Q, K, V, res_mask, pair_bias, save_bias_tiles=True)
        ctx.save_for_backward(Qs, Ks, Vs, mask, bias, O, lse, tiles)
        ctx.bias_shape = tuple(pair_bias.shape)
        return O

    @staticmethod
    def backward(ctx, dO):
        Q, K, V, mask, bias, O, lse, tiles = ctx.saved_tensors
        need_dbias = ctx.needs_input_grad[4]
        dQ, dK, dV, dbias = evoattention_backward(dO, Q, K, V, mask, bias, O, lse, need_dbias, bias_tiles=tiles)
        if dbias is not None:
            if ctx.bias_shape[0] == 1 and dbias.shape[0] != 1:
                dbias = dbias.sum(0, keepdim=True)
            dbias = dbias.to(dO.dtype)  # the reference returns d_pair_bias in dO's dtype (evoattention.py:903)
        return dQ, dK, dV, None, dbias


TritonEvoformer = EvoformerAttention.apply
