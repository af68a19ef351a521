"""The C-ABI library: loads, exports every symbol the header declares, rejects bad arguments before
touching the GPU (so this runs without one)."""
import ctypes as C
import os
import re
import subprocess

import pytest

from megafold_amd import _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "megafold_amd.h")


def declared_functions():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(mf_[a-z0-9_]+)\s*\(", text)))


def test_header_and_binding_agree():
    assert declared_functions() == sorted(_lib.SYMBOLS)


def test_library_exports_every_declared_symbol():
    lib = _lib.lib()
    for name in declared_functions():
        assert hasattr(lib, name), name
    out = subprocess.run(["nm", "-D", "--defined-only", str(_lib.LIB_PATH)], capture_output=True, text=True).stdout
    exported = set(re.findall(r"\sT\s+(mf_[a-z0-9_]+)", out))
    assert set(declared_functions()) <= exported
    assert lib.mf_version() >= 100


def test_header_compiles_as_plain_c(tmp_path):
    src = tmp_path / "t.c"
    src.write_text('#include "megafold_amd.h"\nint main(void){mf_evoattn_args a; mf_lnlinear_args b; (void)a; (void)b; return 0;}\n')
    subprocess.run(["gcc", "-std=c99", "-Wall", "-Werror", "-I", os.path.join(ROOT, "include"), "-c", str(src), "-o",
                    str(tmp_path / "t.o")], check=True)


def test_struct_layout_matches_header(tmp_path):
    src = tmp_path / "s.c"
    src.write_text('#include <stdio.h>\n#include "megafold_amd.h"\nint main(void){printf("%zu %zu %zu %zu\\n", '
                   'sizeof(mf_evoattn_args), offsetof(mf_evoattn_args, workspace), sizeof(mf_lnlinear_args), '
                   'offsetof(mf_lnlinear_args, workspace)); return 0;}\n')
    exe = tmp_path / "s"
    subprocess.run(["gcc", "-I", os.path.join(ROOT, "include"), str(src), "-o", str(exe)], check=True)
    a, b, c, d = map(int, subprocess.run([str(exe)], capture_output=True, text=True).stdout.split())
    assert (a, b) == (C.sizeof(_lib.EvoAttnArgs), _lib.EvoAttnArgs.workspace.offset)
    assert (c, d) == (C.sizeof(_lib.LnLinearArgs), _lib.LnLinearArgs.workspace.offset)


def _evo_args():
    a = _lib.EvoAttnArgs()
    a.B, a.N, a.S, a.H, a.D = 1, 2, 64, 2, 32
    a.dtype, a.bias_dtype, a.mask_dtype = _lib.MF_BF16, _lib.MF_F32, _lib.MF_F32
    a.scale = 32 ** -0.5
    fake = 0x10000  # never dereferenced: every check below fails before a launch
    for f in ("q", "k", "v", "o", "bias", "mask", "lse"):
        setattr(a, f, fake)
    st = _lib.I64x4(2 * 64 * 2 * 32, 64 * 2 * 32, 2 * 32, 32)
    a.q_stride = a.k_stride = a.v_stride = a.o_stride = st
    a.bias_stride = _lib.I64x4(2 * 64 * 64, 64 * 64, 64, 1)
    a.mask_stride = _lib.I64x3(2 * 64, 64, 1)
    return a


@pytest.mark.parametrize("mutate, code, text", [
    (lambda a: setattr(a, "q", None), -1, "q is NULL"),
    (lambda a: setattr(a, "D", 12), -2, "D=12"),
    (lambda a: setattr(a, "D", 128), -2, "D=128"),
    (lambda a: setattr(a, "S", 0), -2, "positive"),
    (lambda a: setattr(a, "S", 16385), -2, "at most 16384"),
    (lambda a: setattr(a, "dtype", 7), -3, "dtype 7"),
    (lambda a: setattr(a, "mask_dtype", 9), -3, "mask_dtype"),
    (lambda a: setattr(a, "k_stride", _lib.I64x4(8192, 4096, 63, 32)), -4, "k stride[2]=63"),
    (lambda a: setattr(a, "v", 0x10004), -5, "v is not 16-byte aligned"),
])
def test_attention_argument_errors(mutate, code, text):
    lib = _lib.lib()
    a = _evo_args()
    mutate(a)
    assert lib.mf_evoattn_fwd(C.byref(a)) == code
    assert text in lib.mf_last_error().decode()
    with pytest.raises(RuntimeError, match="rejected"):
        _lib.check(code, "mf_evoattn_fwd")


def test_attention_workspace_contract():
    lib = _lib.lib()
    a = _evo_args()
    need = lib.mf_evoattn_fwd_workspace_bytes(C.byref(a))               # fp32 copy of bias / scale
    assert need >= 1 * 2 * 64 * 64 * 4
    assert lib.mf_evoattn_fwd(C.byref(a)) == -6 and "workspace" in lib.mf_last_error().decode()
    for f in ("dO", "dq", "dk", "dv", "dbias"):
        setattr(a, f, 0x10000)
    a.do_stride = a.dq_stride = a.dk_stride = a.dv_stride = a.q_stride
    bw = lib.mf_evoattn_bwd_workspace_bytes(C.byref(a))
    assert bw >= 1 * 2 * 2 * 64 * 4                                      # at least delta
    assert lib.mf_evoattn_bwd(C.byref(a)) == -6
    # tiles of the pair bias kept from the forward: the backward's workspace shrinks by exactly their size
    tiles = lib.mf_evoattn_bias_tiles_bytes(C.byref(a))
    assert tiles == need
    a.bias_tiles_bwd = 0x30000
    assert lib.mf_evoattn_bwd_workspace_bytes(C.byref(a)) == bw - tiles
    a.workspace, a.workspace_bytes = 0x40000, bw
    a.bias_tiles_bwd = 0x30008
    assert lib.mf_evoattn_bwd(C.byref(a)) == -5 and "bias_tiles_bwd" in lib.mf_last_error().decode()


def test_attention_memory_lean_contract():
    """MF_EVO_BWD_LEAN keeps the bias gradient's partial sums in the dq buffer: accepted only with dbias, a contiguous dq
    and a dq buffer that can hold them; the workspace query with the bit set leaves the partial sums out."""
    lib = _lib.lib()
    a = _evo_args()
    a.N, a.S = 64, 128                                   # 64 rows: several row chunks, dq larger than the partial sums
    B, N, S, H, D = a.B, a.N, a.S, a.H, a.D
    std = _lib.I64x4(N * S * H * D, S * H * D, H * D, D)
    a.q_stride = a.k_stride = a.v_stride = a.o_stride = std
    for f in ("dO", "dq", "dk", "dv", "dbias"):
        setattr(a, f, 0x10000)
    a.do_stride = a.dq_stride = a.dk_stride = a.dv_stride = std
    full = lib.mf_evoattn_bwd_workspace_bytes(C.byref(a))
    assert lib.mf_evoattn_bwd_lean_ok(C.byref(a)) == 1
    a.phases = _lib.MF_EVO_BWD_LEAN
    lean = lib.mf_evoattn_bwd_workspace_bytes(C.byref(a))
    assert lean < full
    a.workspace, a.workspace_bytes = 0x40000, lean
    a.dq_stride = _lib.I64x4(N * S * H * 2 * D, S * H * 2 * D, H * 2 * D, 2 * D)      # a column slice of a wider matrix
    assert lib.mf_evoattn_bwd_lean_ok(C.byref(a)) == 0
    assert lib.mf_evoattn_bwd(C.byref(a)) == -2 and "MF_EVO_BWD_LEAN" in lib.mf_last_error().decode()
    a.dq_stride = std
    a.dbias = None
    assert lib.mf_evoattn_bwd_lean_ok(C.byref(a)) == 0
    a.dbias = 0x10000
    a.phases = 16
    assert lib.mf_evoattn_bwd(C.byref(a)) == -2 and "phases" in lib.mf_last_error().decode()


def test_python_wrapper_fails_loudly_without_gpu_tensors():
    import torch
    from megafold_amd.model.FusedEvoAttention.evoattention import TritonEvoformer
    q = torch.zeros(1, 2, 16, 2, 8)
    with pytest.raises(RuntimeError, match="GPU only"):
        TritonEvoformer(q, q, q, torch.zeros(1, 2, 1, 1, 16), torch.zeros(1, 1, 2, 16, 16))


def _ln_args(backward=False):
    a = _lib.LnLinearArgs()
    a.M, a.K, a.N = 256, 128, 512
    a.dtype, a.act, a.eps = _lib.MF_BF16, 0, 1e-5
    fake = 0x10000  # never dereferenced: every check below fails before a launch
    for f in ("x", "gamma", "beta", "W", "b", "out", "mean", "rstd"):
        setattr(a, f, fake)
    if backward:
        for f in ("dout", "dx", "dW", "db", "dgamma", "dbeta"):
            setattr(a, f, fake)
    return a


@pytest.mark.parametrize("mutate, code, text", [
    (lambda a: setattr(a, "x", None), -1, "x is NULL"),
    (lambda a: setattr(a, "out", None), -1, "out is NULL"),
    (lambda a: setattr(a, "M", 0), -2, "positive"),
    (lambda a: setattr(a, "K", 260), -2, "K=260"),
    (lambda a: (setattr(a, "K", 256), setattr(a, "dtype", _lib.MF_F32)), -2, "fp32"),
    (lambda a: setattr(a, "N", 508), -2, "N=508"),
    (lambda a: setattr(a, "act", 5), -2, "act 5"),
    (lambda a: (setattr(a, "act", 1), setattr(a, "N", 520)), -2, "multiple of 16"),
    (lambda a: setattr(a, "act", 1), -2, "no linear bias"),
    (lambda a: setattr(a, "dtype", 3), -3, "dtype 3"),
    (lambda a: setattr(a, "W", 0x10008), -5, "W is not 16-byte aligned"),
])
def test_lnlinear_argument_errors(mutate, code, text):
    lib = _lib.lib()
    a = _ln_args()
    mutate(a)
    assert lib.mf_lnlinear_fwd(C.byref(a)) == code
    assert text in lib.mf_last_error().decode()


def test_lnlinear_workspace_contract():
    lib = _lib.lib()
    a = _ln_args()
    need = lib.mf_lnlinear_fwd_workspace_bytes(C.byref(a))
    assert need >= 512 * 128 * 2 + 2 * 512 * 4          # transposed scaled weight + two column vectors
    assert lib.mf_lnlinear_fwd(C.byref(a)) == -6 and "workspace" in lib.mf_last_error().decode()
    b = _ln_args(backward=True)
    assert lib.mf_lnlinear_bwd_workspace_bytes(C.byref(b)) >= 128 * 512 * 4
    assert lib.mf_lnlinear_bwd(C.byref(b)) == -6
    b.dx = None
    assert lib.mf_lnlinear_bwd(C.byref(b)) == -1 and "dx is NULL" in lib.mf_last_error().decode()
    a.K = 260                                            # unsupported shapes report a zero workspace
    assert lib.mf_lnlinear_fwd_workspace_bytes(C.byref(a)) == 0


def test_lnlinear_dx_add_is_only_taken_where_the_query_says_so():
    lib = _lib.lib()
    b = _ln_args(backward=True)
    assert lib.mf_lnlinear_bwd_takes_dx_add(C.byref(b)) == 1         # bf16, K = 128, N = 512
    b.dx_add = 0x10008
    assert lib.mf_lnlinear_bwd(C.byref(b)) == -5 and "dx_add" in lib.mf_last_error().decode()   # alignment
    b.dx_add = 0x10000
    assert lib.mf_lnlinear_bwd(C.byref(b)) == -6                     # accepted: the next check is the workspace
    for field, value in (("K", 64), ("N", 2048), ("dtype", _lib.MF_F32)):
        c = _ln_args(backward=True)
        setattr(c, field, value)
        assert lib.mf_lnlinear_bwd_takes_dx_add(C.byref(c)) == 0
        c.dx_add = 0x10000
        assert lib.mf_lnlinear_bwd(C.byref(c)) == -2 and "dx_add" in lib.mf_last_error().decode()


def test_swiglu_argument_errors():
    lib = _lib.lib()
    bf16 = _lib.MF_BF16
    assert lib.mf_swiglu_fwd(None, 0x10000, 16, 64, bf16, None) == -1
    assert lib.mf_swiglu_fwd(0x10000, 0x20000, 16, 60, bf16, None) == -2
    assert lib.mf_swiglu_fwd(0x10000, 0x20000, 16, 64, 9, None) == -3
    assert lib.mf_swiglu_fwd(0x10004, 0x20000, 16, 64, bf16, None) == -5
    assert lib.mf_swiglu_bwd(0x10000, 0x20000, None, 16, 64, bf16, None) == -1
    assert lib.mf_swiglu_bwd(0x10000, 0x20000, 0x30000, 0, 64, bf16, None) == -2


def _gate_args():
    a = _lib.GateArgs()
    a.M, a.C, a.dtype = 64, 128, _lib.MF_BF16
    a.o, a.g, a.a = 0x10000, 0x20000, 0x30000          # never dereferenced: every check fails before a launch
    a.da, a.d_o, a.dg = 0x40000, 0x50000, 0x60000
    a.ldo = a.lda = a.ldda = a.lddo = 128
    a.ldg = a.lddg = 520
    return a


@pytest.mark.parametrize("mutate,code,text", [
    (lambda a: setattr(a, "C", 100), -2, "multiple of 8"),
    (lambda a: setattr(a, "M", 0), -2, "positive"),
    (lambda a: setattr(a, "dtype", 3), -3, "dtype"),
    (lambda a: setattr(a, "g", None), -1, "g is NULL"),
    (lambda a: setattr(a, "o", 0x10008), -5, "o is not 16-byte aligned"),
    (lambda a: setattr(a, "ldg", 516), -4, "g row stride"),
    (lambda a: setattr(a, "ldo", 64), -4, "o row stride"),
])
def test_gate_argument_errors(mutate, code, text):
    lib = _lib.lib()
    a = _gate_args()
    mutate(a)
    assert lib.mf_sigmoid_gate_fwd(C.byref(a)) == code
    assert text in lib.mf_last_error().decode()
    assert lib.mf_sigmoid_gate_bwd(C.byref(a)) == code


def test_gate_backward_needs_its_gradient_operands():
    lib = _lib.lib()
    a = _gate_args()
    a.dg = None
    assert lib.mf_sigmoid_gate_bwd(C.byref(a)) == -1 and "dg is NULL" in lib.mf_last_error().decode()
    a = _gate_args()
    a.a = None                                           # optional in backward, required in forward
    assert lib.mf_sigmoid_gate_fwd(C.byref(a)) == -1 and "a is NULL" in lib.mf_last_error().decode()
    assert lib.mf_sigmoid_gate_fwd(None) == -1


def test_gate_struct_layout_matches_header(tmp_path):
    src = tmp_path / "g.c"
    src.write_text('#include <stdio.h>\n#include "megafold_amd.h"\nint main(void){printf("%zu %zu %zu\\n", '
                   'sizeof(mf_gate_args), offsetof(mf_gate_args, da), offsetof(mf_gate_args, stream)); return 0;}\n')
    exe = tmp_path / "g"
    subprocess.run(["gcc", "-I", os.path.join(ROOT, "include"), str(src), "-o", str(exe)], check=True)
    a, b, c = map(int, subprocess.run([str(exe)], capture_output=True, text=True).stdout.split())
    assert (a, b, c) == (C.sizeof(_lib.GateArgs), _lib.GateArgs.da.offset, _lib.GateArgs.stream.offset)


def _tm_args():
    a = _lib.TriMulArgs()
    a.B, a.n, a.np, a.dh, a.dtype = 1, 20, 24, 128, _lib.MF_BF16
    a.y, a.dy, a.p = 0x10000, 0x20000, 0x30000           # never dereferenced: every check fails before a launch
    a.ldy = a.lddy = 640
    return a


@pytest.mark.parametrize("mutate,code,text", [
    (lambda a: setattr(a, "np", 20), -2, "multiple of 8"),
    (lambda a: setattr(a, "np", 16), -2, ">= n"),
    (lambda a: setattr(a, "n", 0), -2, "positive"),
    (lambda a: setattr(a, "dh", 96), -2, "channels"),
    (lambda a: setattr(a, "dtype", 7), -3, "dtype"),
    (lambda a: setattr(a, "p", None), -1, "p is NULL"),
    (lambda a: setattr(a, "y", None), -1, "y is NULL"),
    (lambda a: setattr(a, "ldy", 500), -4, "y row stride"),
    (lambda a: setattr(a, "y", 0x10002), -5, "y is not 16-byte aligned"),
])
def test_trimul_pack_argument_errors(mutate, code, text):
    lib = _lib.lib()
    a = _tm_args()
    mutate(a)
    assert lib.mf_trimul_pack_fwd(C.byref(a)) == code
    assert text in lib.mf_last_error().decode()
    assert lib.mf_trimul_pack_bwd(C.byref(a)) == code


def test_channel_layout_argument_errors():
    lib = _lib.lib()
    a = _tm_args()
    a.dh = 256                                            # plain forms move dh channels per row: 64, 128 or 256
    a.ldy = a.lddy = 256
    a.dy = None
    assert lib.mf_channels_first_to_last(C.byref(a)) == -1 and "dy is NULL" in lib.mf_last_error().decode()
    a = _tm_args()
    a.dh = 32
    assert lib.mf_channels_last_to_first(C.byref(a)) == -2 and "channels" in lib.mf_last_error().decode()
    a = _tm_args()
    a.lddy = 64
    assert lib.mf_trimul_pack_bwd(C.byref(a)) == -4 and "dy row stride" in lib.mf_last_error().decode()
    assert lib.mf_channels_last_to_first(None) == -1


def test_trimul_struct_layout_matches_header(tmp_path):
    src = tmp_path / "t.c"
    src.write_text('#include <stdio.h>\n#include "megafold_amd.h"\nint main(void){printf("%zu %zu %zu\\n", '
                   'sizeof(mf_trimul_args), offsetof(mf_trimul_args, y), offsetof(mf_trimul_args, stream)); return 0;}\n')
    exe = tmp_path / "t"
    subprocess.run(["gcc", "-I", os.path.join(ROOT, "include"), str(src), "-o", str(exe)], check=True)
    a, b, c = map(int, subprocess.run([str(exe)], capture_output=True, text=True).stdout.split())
    assert (a, b, c) == (C.sizeof(_lib.TriMulArgs), _lib.TriMulArgs.y.offset, _lib.TriMulArgs.stream.offset)


def test_permute_argument_errors():
    lib = _lib.lib()
    ok = (0x10000, 0x20000, 4, 32, 48, 64, None)
    assert lib.mf_permute_0213(None, 0x20000, 4, 32, 48, 64, None) == -1
    assert lib.mf_permute_0213(0x10000, 0x20000, 0, 32, 48, 64, None) == -2
    for rb in (0, 24, 272):
        assert lib.mf_permute_0213(0x10000, 0x20000, 4, 32, 48, rb, None) == -2 and "row_bytes" in lib.mf_last_error().decode()
    assert lib.mf_permute_0213(0x10008, 0x20000, 4, 32, 48, 64, None) == -5
    assert lib.mf_permute_0213(0x10000, 0x20000, 70000, 32, 48, 64, None) == -2 and "grid" in lib.mf_last_error().decode()
    assert len(ok) == 7


def test_outer_product_mean_argument_errors():
    """mf_opm_fused_fwd / mf_opm_dw / mf_opm_dab reject bad arguments before any launch."""
    lib = _lib.lib()
    A, Bm, W, O, D, WS = 0x10000, 0x20000, 0x30000, 0x40000, 0x50000, 0x60000
    bf16 = _lib.MF_BF16
    assert lib.mf_opm_fused_fwd(None, Bm, W, None, O, 1, 16, bf16, None) == -1
    assert lib.mf_opm_fused_fwd(A + 8, Bm, W, None, O, 1, 16, bf16, None) == -5
    assert lib.mf_opm_fused_fwd(A, Bm, W, None, O, 0, 16, bf16, None) == -2
    assert lib.mf_opm_fused_fwd(A, Bm, W, None, O, 1, 16, _lib.MF_F32, None) == -3 and "f16 / bf16" in lib.mf_last_error().decode()
    need = lib.mf_opm_dw_workspace_bytes(1, 16)
    assert need > 0 and need % (1024 * 128 * 4) == 0 and lib.mf_opm_dw_workspace_bytes(0, 16) == 0
    assert lib.mf_opm_dw(A, Bm, D, None, WS, need, 1, 16, bf16, None) == -1
    assert lib.mf_opm_dw(A, Bm, D, O + 4, WS, need, 1, 16, bf16, None) == -5
    assert lib.mf_opm_dw(A, Bm, D, O, WS, need, 1, 16, _lib.MF_F32, None) == -3
    assert lib.mf_opm_dw(A, Bm, D, O, WS, need, 1, 40000, bf16, None) == -2 and "too large" in lib.mf_last_error().decode()
    assert lib.mf_opm_dw(A, Bm, D, O, WS, 1024, 1, 16, bf16, None) == -6 and "workspace bytes" in lib.mf_last_error().decode()
    need = lib.mf_opm_dab_workspace_bytes(2, 37)
    assert need > 0 and need % (2 * 128 * 128 * 4) == 0 and lib.mf_opm_dab_workspace_bytes(1, -3) == 0
    assert lib.mf_opm_dab(D, W, None, O, WS, need, 2, 37, 0, bf16, None) == -1
    assert lib.mf_opm_dab(D, W, Bm, O, WS + 2, need, 2, 37, 0, bf16, None) == -5
    assert lib.mf_opm_dab(D, W, Bm, O, WS, need - 1, 2, 37, 1, bf16, None) == -6
    assert lib.mf_opm_dab(D, W, Bm, O, WS, need, 2, 37, 1, 7, None) == -3
    RS = 0x70000
    assert lib.mf_opm_pack(None, 64, RS, None, A, Bm, 1, 12, 16, 0, bf16, None) == -1
    assert lib.mf_opm_pack(D, 64, RS, None, A + 8, Bm, 1, 12, 16, 0, bf16, None) == -5
    assert lib.mf_opm_pack(D, 64, RS, None, A, Bm, 1, 129, 16, 0, bf16, None) == -2 and "S <= 128" in lib.mf_last_error().decode()
    assert lib.mf_opm_pack(D, 60, RS, None, A, Bm, 1, 12, 16, 1, bf16, None) == -4
    assert lib.mf_opm_pack(D, 64, RS, None, A, Bm, 1, 12, 16, 1, _lib.MF_F32, None) == -3


def test_pair_weighted_averaging_argument_errors():
    """The mf_pwa_* entry points reject shapes their kernels do not take, unaligned or missing operands and a chunk
    count that differs from what mf_pwa_dw_chunks reports."""
    lib = _lib.lib()

    def args(**kw):
        a = _lib.PwaArgs()
        a.B, a.S, a.N, a.H, a.D, a.dtype = 1, 6, 40, 8, 32, _lib.MF_BF16
        a.logits, a.ld_logits = 0x10000, 8
        a.w = 0x20000
        a.x, a.ldx = 0x30000, 512
        a.y, a.ldy = 0x40000, 256
        a.dy, a.lddy = 0x50000, 256
        a.dw_part = 0x60000
        a.dlogits, a.ld_dlogits = 0x70000, 8
        for k, v in kw.items():
            setattr(a, k, v)
        return a

    assert lib.mf_pwa_softmax_fwd(C.byref(args(H=4))) == -2          # eight heads of 32 channels only
    assert lib.mf_pwa_softmax_fwd(C.byref(args(dtype=_lib.MF_F32))) == -3
    assert lib.mf_pwa_softmax_fwd(C.byref(args(logits=None))) == -1
    assert lib.mf_pwa_softmax_fwd(C.byref(args(ld_logits=12))) == -4
    assert lib.mf_pwa_apply(C.byref(args(N=400))) == -2 and "at most 384" in lib.mf_last_error().decode()
    assert lib.mf_pwa_apply(C.byref(args(y=None))) == -1
    assert lib.mf_pwa_apply(C.byref(args(ldy=100))) == -4
    a = args()
    n = lib.mf_pwa_dw_chunks(C.byref(a))
    assert 1 <= n <= 6
    a.n_chunks = n + 1
    assert lib.mf_pwa_dw(C.byref(a)) == -6 and "mf_pwa_dw_chunks" in lib.mf_last_error().decode()
    assert lib.mf_pwa_dw(C.byref(args(dy=None, n_chunks=n))) == -1
    assert lib.mf_pwa_softmax_bwd(C.byref(args(n_chunks=0))) == -1
    assert lib.mf_pwa_softmax_bwd(C.byref(args(n_chunks=n, dlogits=0x70004))) == -1
