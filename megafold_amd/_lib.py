"""ctypes binding of ``libmegafold_amd.so`` (declarations in ``include/megafold_amd.h``).

The library is the only compute path of this package.  There is no fallback: if it cannot be loaded,
or a call returns an error, a ``RuntimeError`` is raised.
"""
from __future__ import annotations

import ctypes as C
import threading
from pathlib import Path

PKG = Path(__file__).resolve().parent
LIB_PATH = PKG / "lib" / "libmegafold_amd.so"

MF_F32, MF_F16, MF_BF16, MF_BOOL = 0, 1, 2, 3
MF_ACT_NONE, MF_ACT_SWIGLU = 0, 1
MF_EVO_BWD_DQKV, MF_EVO_BWD_DBIAS, MF_EVO_BWD_PREP, MF_EVO_BWD_LEAN = 1, 2, 4, 8

I64x4 = C.c_int64 * 4
I64x3 = C.c_int64 * 3


class EvoAttnArgs(C.Structure):
    _fields_ = [
        ("B", C.c_int32), ("N", C.c_int32), ("S", C.c_int32), ("H", C.c_int32), ("D", C.c_int32),
        ("dtype", C.c_int32), ("bias_dtype", C.c_int32), ("mask_dtype", C.c_int32),
        ("scale", C.c_float), ("phases", C.c_int32),
        ("q", C.c_void_p), ("k", C.c_void_p), ("v", C.c_void_p),
        ("bias", C.c_void_p), ("mask", C.c_void_p),
        ("o", C.c_void_p), ("lse", C.c_void_p),
        ("q_stride", I64x4), ("k_stride", I64x4), ("v_stride", I64x4), ("o_stride", I64x4),
        ("bias_stride", I64x4), ("mask_stride", I64x3),
        ("dO", C.c_void_p), ("dq", C.c_void_p), ("dk", C.c_void_p), ("dv", C.c_void_p),
        ("dbias", C.c_void_p),
        ("do_stride", I64x4), ("dq_stride", I64x4), ("dk_stride", I64x4), ("dv_stride", I64x4),
        ("workspace", C.c_void_p), ("workspace_bytes", C.c_uint64), ("stream", C.c_void_p),
        ("bias_tiles_bwd", C.c_void_p),
    ]


class LnLinearArgs(C.Structure):
    _fields_ = [
        ("M", C.c_int64), ("K", C.c_int32), ("N", C.c_int32),
        ("dtype", C.c_int32), ("act", C.c_int32), ("eps", C.c_float), ("param_grad_dtype", C.c_int32),
        ("x", C.c_void_p), ("gamma", C.c_void_p), ("beta", C.c_void_p), ("W", C.c_void_p), ("b", C.c_void_p),
        ("out", C.c_void_p), ("mean", C.c_void_p), ("rstd", C.c_void_p),
        ("dout", C.c_void_p), ("dx", C.c_void_p), ("dx_add", C.c_void_p), ("dW", C.c_void_p), ("db", C.c_void_p),
        ("dgamma", C.c_void_p), ("dbeta", C.c_void_p),
        ("workspace", C.c_void_p), ("workspace_bytes", C.c_uint64), ("stream", C.c_void_p),
    ]


class GateArgs(C.Structure):
    _fields_ = [
        ("M", C.c_int64), ("C", C.c_int32), ("dtype", C.c_int32),
        ("o", C.c_void_p), ("ldo", C.c_int64), ("g", C.c_void_p), ("ldg", C.c_int64),
        ("a", C.c_void_p), ("lda", C.c_int64), ("res", C.c_void_p), ("ldres", C.c_int64),
        ("da", C.c_void_p), ("ldda", C.c_int64), ("d_o", C.c_void_p), ("lddo", C.c_int64),
        ("dg", C.c_void_p), ("lddg", C.c_int64),
        ("stream", C.c_void_p),
    ]


class TriMulArgs(C.Structure):
    _fields_ = [
        ("B", C.c_int32), ("n", C.c_int32), ("np", C.c_int32), ("dh", C.c_int32),
        ("dtype", C.c_int32), ("transposed", C.c_int32), ("swap", C.c_int32), ("reserved0", C.c_int32),
        ("y", C.c_void_p), ("ldy", C.c_int64), ("dy", C.c_void_p), ("lddy", C.c_int64),
        ("mask", C.c_void_p), ("p", C.c_void_p), ("stream", C.c_void_p),
    ]


class PwaArgs(C.Structure):
    _fields_ = [
        ("B", C.c_int32), ("S", C.c_int32), ("N", C.c_int32), ("H", C.c_int32), ("D", C.c_int32),
        ("dtype", C.c_int32), ("n_chunks", C.c_int32), ("reserved0", C.c_int32),
        ("logits", C.c_void_p), ("ld_logits", C.c_int64), ("mask", C.c_void_p), ("w", C.c_void_p),
        ("x", C.c_void_p), ("ldx", C.c_int64), ("g", C.c_void_p), ("ldg", C.c_int64),
        ("y", C.c_void_p), ("ldy", C.c_int64), ("dy", C.c_void_p), ("lddy", C.c_int64),
        ("dw_part", C.c_void_p), ("dlogits", C.c_void_p), ("ld_dlogits", C.c_int64), ("stream", C.c_void_p),
    ]


# every symbol include/megafold_amd.h declares: name -> (restype, argtypes)
SYMBOLS = {
    "mf_version": (C.c_int, []),
    "mf_last_error": (C.c_char_p, []),
    "mf_evoattn_fwd_workspace_bytes": (C.c_uint64, [C.POINTER(EvoAttnArgs)]),
    "mf_evoattn_bwd_workspace_bytes": (C.c_uint64, [C.POINTER(EvoAttnArgs)]),
    "mf_evoattn_bias_tiles_bytes": (C.c_uint64, [C.POINTER(EvoAttnArgs)]),
    "mf_evoattn_bwd_lean_ok": (C.c_int, [C.POINTER(EvoAttnArgs)]),
    "mf_evoattn_fwd": (C.c_int, [C.POINTER(EvoAttnArgs)]),
    "mf_evoattn_bwd": (C.c_int, [C.POINTER(EvoAttnArgs)]),
    "mf_evoattn_fwd_noalloc": (C.c_int, [C.POINTER(EvoAttnArgs)]),
    "mf_lnlinear_fwd_workspace_bytes": (C.c_uint64, [C.POINTER(LnLinearArgs)]),
    "mf_lnlinear_bwd_workspace_bytes": (C.c_uint64, [C.POINTER(LnLinearArgs)]),
    "mf_lnlinear_fwd": (C.c_int, [C.POINTER(LnLinearArgs)]),
    "mf_lnlinear_bwd": (C.c_int, [C.POINTER(LnLinearArgs)]),
    "mf_lnlinear_bwd_takes_dx_add": (C.c_int, [C.POINTER(LnLinearArgs)]),
    "mf_permute_0213": (C.c_int, [C.c_void_p, C.c_void_p, C.c_int64, C.c_int64, C.c_int64, C.c_int32, C.c_void_p]),
    "mf_swiglu_fwd": (C.c_int, [C.c_void_p, C.c_void_p, C.c_int64, C.c_int32, C.c_int32, C.c_void_p]),
    "mf_swiglu_bwd": (C.c_int, [C.c_void_p, C.c_void_p, C.c_void_p, C.c_int64, C.c_int32, C.c_int32, C.c_void_p]),
    "mf_sigmoid_gate_fwd": (C.c_int, [C.POINTER(GateArgs)]),
    "mf_sigmoid_gate_bwd": (C.c_int, [C.POINTER(GateArgs)]),
    "mf_opm_dw_workspace_bytes": (C.c_uint64, [C.c_int32, C.c_int32]),
    "mf_opm_dw": (C.c_int, [C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_uint64, C.c_int32, C.c_int32,
                            C.c_int32, C.c_void_p]),
    "mf_opm_dab_workspace_bytes": (C.c_uint64, [C.c_int32, C.c_int32]),
    "mf_opm_dab": (C.c_int, [C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_uint64, C.c_int32, C.c_int32,
                             C.c_int32, C.c_int32, C.c_void_p]),
    "mf_opm_pack": (C.c_int, [C.c_void_p, C.c_int64, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_int32, C.c_int32,
                              C.c_int32, C.c_int32, C.c_int32, C.c_void_p]),
    "mf_opm_fused_fwd": (C.c_int, [C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_int32, C.c_int32, C.c_int32,
                                   C.c_void_p]),
    "mf_pwa_softmax_fwd": (C.c_int, [C.POINTER(PwaArgs)]),
    "mf_pwa_apply": (C.c_int, [C.POINTER(PwaArgs)]),
    "mf_pwa_dw_chunks": (C.c_int, [C.POINTER(PwaArgs)]),
    "mf_pwa_dw": (C.c_int, [C.POINTER(PwaArgs)]),
    "mf_pwa_softmax_bwd": (C.c_int, [C.POINTER(PwaArgs)]),
    "mf_trimul_pack_fwd": (C.c_int, [C.POINTER(TriMulArgs)]),
    "mf_trimul_pack_bwd": (C.c_int, [C.POINTER(TriMulArgs)]),
    "mf_channels_last_to_first": (C.c_int, [C.POINTER(TriMulArgs)]),
    "mf_channels_first_to_last": (C.c_int, [C.POINTER(TriMulArgs)]),
}

_lock = threading.Lock()
_lib = None


def lib(build_if_missing: bool = True) -> C.CDLL:
    """The loaded library.  Builds it first only when no built library exists."""
    global _lib
    if _lib is not None:
        return _lib
    with _lock:
        if _lib is not None:
            return _lib
        if not LIB_PATH.exists():
            if not build_if_missing:
                raise RuntimeError("%s is missing: run `python -m megafold_amd.build`" % LIB_PATH)
            from . import build as _build
            _build.build()
        try:
            handle = C.CDLL(str(LIB_PATH))
        except OSError as e:  # pragma: no cover - depends on the machine
            raise RuntimeError("cannot load %s: %s" % (LIB_PATH, e)) from e
        for name, (res, args) in SYMBOLS.items():
            try:
                fn = getattr(handle, name)
            except AttributeError as e:
                raise RuntimeError("%s does not export %s" % (LIB_PATH, name)) from e
            fn.restype = res
            fn.argtypes = args
        _lib = handle
        return _lib


def check(rc: int, what: str) -> None:
    """Turn a non-zero return code of the C ABI into a RuntimeError."""
    if rc == 0:
        return
    if rc < 0:
        msg = lib().mf_last_error().decode("utf-8", "replace")
        raise RuntimeError("%s rejected its arguments (code %d): %s" % (what, rc, msg))
    raise RuntimeError("%s: HIP error %d while launching" % (what, rc))


def dtype_code(dtype) -> int:
    import torch
    table = {torch.float32: MF_F32, torch.float16: MF_F16, torch.bfloat16: MF_BF16, torch.bool: MF_BOOL}
    if dtype not in table:
        raise TypeError("unsupported dtype %s" % dtype)
    return table[dtype]
