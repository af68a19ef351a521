"""Parity of the HIP LayerNorm->Linear / SwiGLU / Transition path against the CPU oracle (GPU box
only); every call goes through the C ABI (``mf_lnlinear_*`` / ``mf_swiglu_*``) via the drop-in modules."""
import os

import numpy as np
import pytest
import torch
import torch.nn as nn

from conftest import tol_for
from megafold_amd import workloads
from megafold_amd.model.FusedLayernormLinear.fused_layernorm_linear import LayernormLinear
from megafold_amd.model.FusedTransition.fused_transition import FusedSwiGLU, FusedTransition
from oracle import layernorm_linear as ol
from oracle import transition as ot

pytestmark = pytest.mark.gpu
GOLD = os.path.join(os.path.dirname(__file__), "golden")
f64 = torch.float64


def close(got, want, dtype, name, scale_atol=1.0):
    t = dict(tol_for(dtype))
    t["atol"] = t["atol"] * scale_atol
    assert not torch.isnan(got).any(), name
    torch.testing.assert_close(got.detach().cpu().to(want.dtype), want, msg=lambda m: "%s: %s" % (name, m), **t)


def make_module(inp, K, N, dtype, bias):
    mod = LayernormLinear(K, N, has_linear_bias=bias, device="cuda", dtype=dtype)
    with torch.no_grad():
        mod.WEIGHT.copy_(inp["gamma"]); mod.BIAS.copy_(inp["beta"]); mod.linear_weight.copy_(inp["W"])
        if bias:
            mod.linear_bias.copy_(inp["b"])
    return mod


# (M-shape, K, N) from the reference's sweep (tests/test_layernormlinear.py:44-60) and the model's (N, K) table
SWEEP = [
    ((16,), 16, 16, torch.float32, True),
    ((3, 37), 64, 48, torch.float32, True),
    ((8000,), 128, 512, torch.bfloat16, True),
    ((777,), 128, 16, torch.bfloat16, True),      # pair-bias heads (16, 128)
    ((2, 300), 64, 64, torch.bfloat16, False),    # outer-product-mean (64, 64)
    ((513,), 16, 8, torch.float16, True),
    ((300,), 256, 264, torch.bfloat16, True),
    ((5000,), 128, 640, torch.bfloat16, False),   # triangle multiplication (640, 128)
    ((1000,), 64, 320, torch.bfloat16, False),    # (320, 64)
    ((1200,), 128, 128, torch.bfloat16, False),   # (128, 128)
    ((900,), 128, 8, torch.bfloat16, False),      # (8, 128)
    ((40000,), 128, 512, torch.bfloat16, True),   # more row blocks than resident work-groups: several iterations each
    ((33001,), 96, 256, torch.bfloat16, False),   # K padded to 128, ragged last row block, several iterations
    ((20000,), 128, 1024, torch.float16, False),  # N > 512: eight-wavefront dx kernel
    ((70000,), 256, 512, torch.bfloat16, True),   # 512-byte rows: one work-group per compute unit, several iterations each
    ((9000,), 128, 256, torch.float32, False),    # the same for fp32 rows
    ((3000,), 256, 64, torch.float32, True),
    ((53,), 128, 8, torch.float32, True),         # 512-byte rows with a single column tile
    ((30928,), 32, 1024, torch.bfloat16, True),   # wide N on a short row: dx takes gamma in fp32 (a dx through the
    ((12736,), 56, 520, torch.bfloat16, True),    # rounded gamma (.) W misses the element-wise bar on these three)
    ((2639,), 64, 1024, torch.bfloat16, False),
    ((700,), 256, 24, torch.bfloat16, False),
    ((100,), 768, 768, torch.float32, True),      # K beyond the kernels: same eager expression as the reference's fallback
]


@pytest.mark.parametrize("mshape,K,N,dtype,bias", SWEEP)
def test_layernorm_linear_parity(mshape, K, N, dtype, bias):
    print("case", mshape, K, N, dtype, bias, flush=True)
    inp = workloads.lnlinear_inputs(mshape, K, N, dtype=dtype, seed=K + N, linear_bias=bias)
    if bias:
        inp["b"] = (0.3 * torch.randn(N, generator=torch.Generator().manual_seed(1))).to(dtype)
    mod = make_module({k: (v.cuda() if v is not None else None) for k, v in inp.items()}, K, N, dtype, bias)
    x = inp["x"].cuda().requires_grad_()
    out = mod(x)
    out.backward(inp["dY"].cuda())
    ref = ol.layernorm_linear_forward(inp["x"], inp["gamma"], inp["beta"], inp["W"], inp["b"], dtype=f64)
    rdx, rdW, rdb, rdg, rdbt = ol.layernorm_linear_backward(inp["dY"], inp["x"], inp["gamma"], inp["beta"], inp["W"], dtype=f64)
    M = int(np.prod(mshape))
    close(out, ref, dtype, "out")
    close(x.grad, rdx, dtype, "dX")
    # parameter gradients are sums over M rows: the absolute bar scales with the magnitude of the sum
    s = max(1.0, M ** 0.5)
    close(mod.linear_weight.grad, rdW, dtype, "dW", s)
    close(mod.WEIGHT.grad, rdg, dtype, "dgamma", s)
    close(mod.BIAS.grad, rdbt, dtype, "dbeta", s)
    if bias:
        close(mod.linear_bias.grad, rdb, dtype, "dLinearBias", s)
    assert out.dtype == dtype and out.shape == tuple(mshape) + (N,)


def test_small_fp32_against_golden():
    g = np.load(os.path.join(GOLD, "lnlinear_small.npz"))
    inp = workloads.lnlinear_inputs((3, 37), 64, 48, dtype=torch.float32, seed=5)
    inp["b"] = torch.from_numpy(g["b"]).float()
    mod = make_module({k: v.cuda() for k, v in inp.items()}, 64, 48, torch.float32, True)
    x = inp["x"].cuda().requires_grad_()
    out = mod(x)
    out.backward(inp["dY"].cuda())
    for name, t in (("out", out), ("dx", x.grad), ("dW", mod.linear_weight.grad), ("db", mod.linear_bias.grad),
                    ("dgamma", mod.WEIGHT.grad), ("dbeta", mod.BIAS.grad)):
        np.testing.assert_allclose(t.detach().cpu().numpy(), g[name], rtol=1e-4, atol=2e-5, err_msg=name)


def test_config3_full_size_parity_and_properties():
    """C3: x [1, 384, 384, 128] bf16 -> 512, the fused q/k/v/gate projection."""
    inp = workloads.lnlinear_inputs()
    mod = make_module({k: v.cuda() for k, v in inp.items()}, 128, 512, torch.bfloat16, True)
    x = inp["x"].cuda().requires_grad_()
    out = mod(x)
    out.backward(inp["dY"].cuda())
    ref = ol.layernorm_linear_forward(inp["x"], inp["gamma"], inp["beta"], inp["W"], inp["b"])
    rdx, rdW, rdb, rdg, rdbt = ol.layernorm_linear_backward(inp["dY"], inp["x"], inp["gamma"], inp["beta"], inp["W"])
    close(out, ref, torch.bfloat16, "out")
    close(x.grad, rdx, torch.bfloat16, "dX")
    s = 147456 ** 0.5
    close(mod.linear_weight.grad, rdW, torch.bfloat16, "dW", s)
    close(mod.WEIGHT.grad, rdg, torch.bfloat16, "dgamma", s)
    close(mod.BIAS.grad, rdbt, torch.bfloat16, "dbeta", s)
    close(mod.linear_bias.grad, rdb, torch.bfloat16, "db", s)
    # LayerNorm backward projects out the constant direction of every row
    assert x.grad.float().sum(-1).abs().max() < 0.25
    # bitwise reproducible (no atomics)
    x2 = inp["x"].cuda().requires_grad_()
    mod.zero_grad()
    out2 = mod(x2)
    g1 = mod.linear_weight.grad
    out2.backward(inp["dY"].cuda())
    assert torch.equal(out, out2) and torch.equal(x.grad, x2.grad)
    # linearity in dOut: backward(2 dY) == 2 backward(dY) exactly (power-of-two scaling)
    x3 = inp["x"].cuda().requires_grad_()
    mod(x3).backward(2 * inp["dY"].cuda())
    assert torch.equal(x3.grad, 2 * x.grad)


def test_autocast_contract_and_state_dict_names():
    mod = LayernormLinear(128, 64, device="cuda")            # fp32 parameters
    assert sorted(mod.state_dict()) == ["BIAS", "WEIGHT", "linear_bias", "linear_weight"]
    assert mod.linear_weight.shape == (128, 64)
    x = torch.randn(50, 128, device="cuda", requires_grad=True)
    with torch.autocast("cuda", dtype=torch.bfloat16):
        out = mod(x)
    assert out.dtype == torch.bfloat16                       # custom_fwd(cast_inputs=bfloat16)
    out.float().sum().backward()
    assert x.grad.dtype == torch.float32 and mod.linear_weight.grad.dtype == torch.float32
    ref = ol.layernorm_linear_forward(x.detach().cpu(), mod.WEIGHT.detach().cpu(), mod.BIAS.detach().cpu(),
                                      mod.linear_weight.detach().cpu(), mod.linear_bias.detach().cpu())
    close(out, ref, torch.bfloat16, "autocast out")


@pytest.mark.parametrize("mshape,dim,ef,dtype", [((2, 29), 32, 4, torch.float32), ((1000,), 128, 4, torch.bfloat16),
                                                   ((4097,), 64, 4, torch.bfloat16), ((300,), 128, 2, torch.float16),
                                                   ((40000,), 256, 2, torch.bfloat16), ((6000,), 128, 1, torch.float32),
                                                   ((37,), 32, 4, torch.bfloat16), ((70001,), 128, 4, torch.float16),
                                                   ((2, 333), 64, 8, torch.bfloat16)])
def test_fused_transition_parity(mshape, dim, ef, dtype):
    inp = workloads.transition_inputs(mshape, dim, ef, dtype=dtype, seed=7)
    mod = FusedTransition(dim, ef, device="cuda", dtype=dtype)
    assert sorted(mod.state_dict()) == ["ff.0.BIAS", "ff.0.WEIGHT", "ff.0.linear_weight", "ff.2.weight"]
    with torch.no_grad():
        mod.ff[0].WEIGHT.copy_(inp["gamma"]); mod.ff[0].BIAS.copy_(inp["beta"])
        mod.ff[0].linear_weight.copy_(inp["W1"]); mod.ff[2].weight.copy_(inp["W2"])
    x = inp["x"].cuda().requires_grad_()
    y = mod(x)
    y.backward(inp["dY"].cuda())
    # oracle: autograd of the float64 eager Transition (benchmarks/transition_speed.py:8-39)
    xr, gr, br, w1, w2 = (inp[n].double().requires_grad_() for n in ("x", "gamma", "beta", "W1", "W2"))
    yr = ot.transition_forward(xr, gr, br, w1, w2, dtype=f64)
    yr.backward(inp["dY"].double())
    M = int(np.prod(mshape))
    s = max(1.0, M ** 0.5)
    close(y, yr.detach(), dtype, "y")
    close(x.grad, xr.grad, dtype, "dX")
    close(mod.ff[0].linear_weight.grad, w1.grad, dtype, "dW1", s)
    close(mod.ff[2].weight.grad, w2.grad, dtype, "dW2", s)
    close(mod.ff[0].WEIGHT.grad, gr.grad, dtype, "dgamma", s)
    close(mod.ff[0].BIAS.grad, br.grad, dtype, "dbeta", s)
    if mshape == (2, 29):
        g = np.load(os.path.join(GOLD, "transition_small.npz"))
        np.testing.assert_allclose(y.detach().cpu().numpy(), g["y"], rtol=1e-4, atol=2e-5)


@pytest.mark.parametrize("include_ln,use_lnl", [(True, False), (False, True)])
def test_transition_variants_use_standalone_swiglu(include_ln, use_lnl):
    dim = 64
    mod = FusedTransition(dim, 2, include_ln=include_ln, use_layernormlinear=use_lnl, device="cuda", dtype=torch.bfloat16)
    x = torch.randn(333, dim, device="cuda", dtype=torch.bfloat16, requires_grad=True)
    y = mod(x)
    y.float().sum().backward()
    ref = nn.Sequential(*[m if not isinstance(m, FusedSwiGLU) else _EagerSwiGLU() for m in mod.ff]).float()
    xr = x.detach().float().requires_grad_()
    yr = ref(xr)
    yr.sum().backward()
    close(y, yr.detach().cpu(), torch.bfloat16, "y")
    close(x.grad, xr.grad.cpu(), torch.bfloat16, "dX")


class _EagerSwiGLU(nn.Module):
    def forward(self, x):
        a, g = x.chunk(2, dim=-1)
        return torch.nn.functional.silu(g) * a


def test_config4_full_size_transition():
    """C4: x [1, 384, 384, 128] bf16, 128 -> 1024 -> SwiGLU -> 512 -> 128."""
    inp = workloads.transition_inputs()
    mod = FusedTransition(128, 4, device="cuda", dtype=torch.bfloat16)
    with torch.no_grad():
        mod.ff[0].WEIGHT.copy_(inp["gamma"]); mod.ff[0].BIAS.copy_(inp["beta"])
        mod.ff[0].linear_weight.copy_(inp["W1"]); mod.ff[2].weight.copy_(inp["W2"])
    x = inp["x"].cuda().requires_grad_()
    y = mod(x)
    y.backward(inp["dY"].cuda())
    # fp32 oracle on a slice of rows (rows are independent); parameter gradients by linearity are
    # checked on the small cases above
    sl = slice(200, 204)
    xr = inp["x"][:, sl].float().requires_grad_()
    yr = ot.transition_forward(xr, inp["gamma"], inp["beta"], inp["W1"], inp["W2"])
    yr.backward(inp["dY"][:, sl].float())
    close(y[:, sl], yr.detach(), torch.bfloat16, "y")
    close(x.grad[:, sl], xr.grad, torch.bfloat16, "dX")
    # the four parameter gradients at full size (M = 147 456 rows: 128 row ranges in the weight-gradient
    # kernel) against the fp32 oracle, accumulated over chunks of rows on the CPU
    gam, bet = inp["gamma"].float().requires_grad_(), inp["beta"].float().requires_grad_()
    W1, W2 = inp["W1"].float().requires_grad_(), inp["W2"].float().requires_grad_()
    xf, dyf = inp["x"].reshape(-1, 128), inp["dY"].reshape(-1, 128)
    for r0 in range(0, xf.shape[0], 16384):
        yr = ot.transition_forward(xf[r0:r0 + 16384].float(), gam, bet, W1, W2)
        yr.backward(dyf[r0:r0 + 16384].float())
    M = xf.shape[0]
    s = M ** 0.5
    close(mod.ff[0].linear_weight.grad, W1.grad, torch.bfloat16, "dW1", s)
    close(mod.ff[0].WEIGHT.grad, gam.grad, torch.bfloat16, "dgamma", s)
    close(mod.ff[0].BIAS.grad, bet.grad, torch.bfloat16, "dbeta", s)
    close(mod.ff[2].weight.grad, W2.grad, torch.bfloat16, "dW2", s)


def test_param_grads_float_and_typed_outputs_agree():
    """mf_lnlinear_bwd writes dW / db / dgamma / dbeta as float (param_grad_dtype = 0) or already rounded to
    x's dtype (1, what the drop-in module asks for); the second is the first rounded once."""
    import ctypes as C
    from megafold_amd import _lib
    from megafold_amd.model.FusedLayernormLinear import fused_layernorm_linear as fl
    torch.manual_seed(5)
    M, K, N, dt = 3000, 128, 192, torch.bfloat16
    x = torch.randn(M, K, device="cuda", dtype=dt)
    W = (torch.randn(K, N, device="cuda") * 0.1).to(dt)
    g = torch.randn(K, device="cuda").to(dt)
    be = torch.randn(K, device="cuda").to(dt)
    dY = torch.randn(M, N, device="cuda", dtype=dt)
    c, x2, W2, Mean, RSTD = fl.layernorm_linear_forward(x, W, None, g, be, True, False)
    dX1, dB1, dLin1, dG1, dBe1 = fl.layernorm_linear_backward(dY, x2, W2, Mean, RSTD, g, be, True, True)
    lib = _lib.lib()
    dX0 = torch.empty_like(x)
    dB0 = torch.empty(K, N, device="cuda", dtype=torch.float32)
    dLin0 = torch.empty(N, device="cuda", dtype=torch.float32)
    dG0 = torch.empty(K, device="cuda", dtype=torch.float32)
    dBe0 = torch.empty(K, device="cuda", dtype=torch.float32)
    args = fl._args(x2, W2, None, g, be, _lib.MF_ACT_NONE, x.device)
    args.mean, args.rstd = Mean.data_ptr(), RSTD.data_ptr()
    args.dout, args.dx, args.dW = dY.data_ptr(), dX0.data_ptr(), dB0.data_ptr()
    args.db, args.dgamma, args.dbeta = dLin0.data_ptr(), dG0.data_ptr(), dBe0.data_ptr()
    args.param_grad_dtype = 0
    nbytes = lib.mf_lnlinear_bwd_workspace_bytes(C.byref(args))
    ws = torch.empty(max(nbytes, 16), dtype=torch.uint8, device="cuda")
    args.workspace, args.workspace_bytes = ws.data_ptr(), nbytes
    _lib.check(lib.mf_lnlinear_bwd(C.byref(args)), "mf_lnlinear_bwd")
    torch.cuda.synchronize()
    assert torch.equal(dX0, dX1)
    assert torch.equal(dB0.to(dt), dB1) and torch.equal(dLin0.to(dt), dLin1)
    assert torch.equal(dG0.to(dt), dG1) and torch.equal(dBe0.to(dt), dBe1)
    args.param_grad_dtype = 7
    assert lib.mf_lnlinear_bwd(C.byref(args)) == -3


@pytest.mark.gpu
@pytest.mark.parametrize("K,N,act", [(128, 128, 0), (96, 256, 0), (128, 512, 0), (128, 520, 0), (128, 640, 0),
                                     (128, 1024, 0), (128, 1024, 1), (128, 2048, 0), (64, 128, 0)])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
def test_backward_dx_add_matches_the_separate_sum(K, N, act, dtype):
    """``dx_add`` of ``layernorm_linear_backward`` (the gradient that skips the operator in x + f(x)): every
    instantiation of the dx kernel that adds it in place, and the shapes where the wrapper adds it afterwards,
    against dx + dx_add formed separately.  The fused sum rounds once, the separate one twice."""
    from megafold_amd import _lib
    from megafold_amd.model.FusedLayernormLinear.fused_layernorm_linear import (layernorm_linear_backward,
                                                                                 layernorm_linear_forward)
    M = 1000                                                     # not a multiple of the 32-row blocks
    g = torch.Generator().manual_seed(5)
    rnd = lambda *sh: torch.randn(*sh, generator=g).to(dtype).cuda()
    x, W, gamma, beta = rnd(M, K), rnd(K, N) * K ** -0.5, 1 + 0.1 * rnd(K), 0.1 * rnd(K)
    _, x2, Wc, Mean, RSTD = layernorm_linear_forward(x, W, None, gamma, beta, True, False, act=act)
    dout, skip = rnd(M, N // 2 if act else N), rnd(M, K)
    want = layernorm_linear_backward(dout, x2, Wc, Mean, RSTD, gamma, beta, True, False, act=act)
    got = layernorm_linear_backward(dout, x2, Wc, Mean, RSTD, gamma, beta, True, False, act=act, dx_add=skip)
    torch.testing.assert_close(got[0].float(), want[0].float() + skip.float(), **tol_for(dtype))
    for a, b in zip(got[1:], want[1:]):                          # parameter gradients do not see it
        if a is not None:
            assert torch.equal(a, b)


@pytest.mark.gpu
@pytest.mark.parametrize("kind", ["lnlinear", "transition"])
def test_outputs_beyond_two_to_the_31_elements_match_their_row_slices(kind):
    """M = 2 200 001 rows of K = 128 into N = 1024 columns: 2.25e9 elements of output (and of incoming gradient) in the
    plain form, as many of pre-activation in the transition.  Rows are independent: out and dx of the full call must
    equal, bit for bit, those of calls on row slices near the end and on both halves; the parameter gradients of the
    halves must add up to the full ones within the rounding of the 16-bit results."""
    torch.manual_seed(0)
    dt, M, K = torch.bfloat16, 2_200_001, 128
    if kind == "lnlinear":
        mod, n_out = LayernormLinear(K, 1024, has_linear_bias=True, device="cuda", dtype=dt), 1024
    else:
        mod, n_out = FusedTransition(K, 4, device="cuda", dtype=dt), K
    x = torch.randn(M, K, device="cuda").to(dt)
    dy = torch.randn(M, n_out, device="cuda").to(dt)

    def run(sl):
        xx = x[sl].detach().clone().requires_grad_()
        for p in mod.parameters():
            p.grad = None
        y = mod(xx)
        y.backward(dy[sl])
        return y.detach(), xx.grad, [p.grad.float().clone() for p in mod.parameters()]

    full = run(slice(0, M))
    halves = []
    for sl in (slice(M - 1000, M), slice(M - 70001, M - 69000), slice(0, M // 2), slice(M // 2, M)):
        part = run(sl)
        assert torch.equal(full[0][sl], part[0]), "out of rows %s differs from the sliced call" % (sl,)
        assert torch.equal(full[1][sl], part[1]), "dx of rows %s differs from the sliced call" % (sl,)
        if sl.stop - sl.start >= M // 2:
            halves.append(part[2])
        del part
    for a, b, c in zip(full[2], halves[0], halves[1]):
        torch.testing.assert_close(a, b + c, rtol=2 ** -6, atol=2 ** -6 * float(a.abs().max()))
