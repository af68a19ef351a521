"""Parity of the HIP attention path against the CPU oracle (GPU box only).  Every call goes through
the C ABI (``mf_evoattn_fwd`` / ``mf_evoattn_bwd``) via the Python operator, never through a fallback."""
import os

import numpy as np
import pytest
import torch

from conftest import tol_for
from megafold_amd import workloads
from megafold_amd.model.FusedEvoAttention.evoattention import (EvoformerAttention, TritonEvoformer,
                                                                evoattention_backward, evoattention_forward)
from oracle import evoattention as oe

pytestmark = pytest.mark.gpu
GOLD = os.path.join(os.path.dirname(__file__), "golden")
f64 = torch.float64


def to_dev(inp):
    return {k: v.cuda() for k, v in inp.items()}


def run_op(dev, need_bias_grad=True):
    q, k, v = (dev[n].clone().requires_grad_() for n in "qkv")
    bias = dev["bias"].clone().requires_grad_(need_bias_grad)
    out = TritonEvoformer(q, k, v, dev["mask"], bias)
    out.backward(dev["dO"])
    return out.detach(), q.grad, k.grad, v.grad, bias.grad


def oracle_all(inp, chunk=64):
    dt = f64 if inp["q"].numel() < 4_000_000 else torch.float32
    return oe.evo_attention_chunked(inp["q"], inp["k"], inp["v"], inp["mask"], inp["bias"], inp["dO"], chunk=chunk, dtype=dt)


def check(got, want, dtype, names=("O", "dQ", "dK", "dV", "dBias"), tol=None):
    for name, g, w in zip(names, got, want):
        assert not torch.isnan(g).any(), name
        torch.testing.assert_close(g.cpu().to(w.dtype), w, msg=lambda m, n=name: "%s: %s" % (n, m), **(tol or tol_for(dtype)))


# shapes from the reference's sweep (tests/test_evoattention.py:85-135), sized for a quick oracle
SWEEP = [
    # B, N, S, H, D, masked, dtype
    (1, 1, 23, 16, 8, 3, torch.float16),
    (1, 4, 64, 4, 32, 8, torch.bfloat16),
    (2, 3, 77, 3, 32, 5, torch.bfloat16),
    (1, 2, 160, 2, 64, 0, torch.bfloat16),
    (1, 2, 96, 1, 16, 3, torch.float16),
    (1, 1, 384, 16, 64, 0, torch.bfloat16),   # single attention with pair bias (N=1, H=16, D=64)
    (1, 5, 200, 5, 32, 17, torch.bfloat16),
    (1, 2, 499, 4, 32, 33, torch.bfloat16),
    (1, 2, 800, 2, 32, 40, torch.bfloat16),   # 25 key tiles: three passes of the persistent dQ/dK/dV kernel, odd tile count
    (1, 1, 1824, 1, 32, 7, torch.bfloat16),   # too long for the per-row carrier table of the D <= 32 kernel
    (1, 1, 1280, 1, 64, 0, torch.bfloat16),   # longest sequence of the reference sweep
    (1, 3, 50, 2, 8, 3, torch.float32),
    (1, 2, 130, 2, 64, 9, torch.float32),
    (1, 6, 384, 5, 64, 20, torch.float16),    # odd head count at D = 64 (one head per dBias work-group)
    (2, 3, 304, 4, 32, 0, torch.float16),     # 10 key tiles: three per wavefront with idle slots, batch 2
    (1, 3, 640, 3, 32, 50, torch.bfloat16),   # 20 key tiles: two passes of the persistent dQ/dK/dV kernel
    (1, 2, 520, 2, 32, 9, torch.float16),     # 17 key tiles in float16: the second pass holds five tiles and seven empty slots
    (1, 2, 768, 2, 24, 96, torch.bfloat16),   # two full passes, padded head dimension
    (1, 300, 416, 4, 32, 20, torch.bfloat16),  # 13 key tiles and 1200 (row, head) problems: every work-group of the
                                               # persistent dQ/dK/dV kernel walks several two-pass problems in a row
]


@pytest.mark.parametrize("B,N,S,H,D,nm,dtype", SWEEP)
def test_forward_backward_parity(B, N, S, H, D, nm, dtype):
    print("case", B, N, S, H, D, nm, dtype, flush=True)
    inp = workloads.evoattention_inputs(B, N, S, H, D, nm, dtype=dtype, seed=S + D)
    got = run_op(to_dev(inp))
    check(got, oracle_all(inp), dtype)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("kind", ["ramp", "wide"])
def test_wide_logit_range_exercises_the_offset_refresh(dtype, kind):
    """Logits with a real dynamic range: with N(0, 1) inputs the forward's running softmax offset is set once
    (on the first key tile) and never again.  Here the bias grows by 15 nats per key tile ("ramp": every later
    tile overtakes the running offset, so the accumulated output and sum are rescaled mid-sequence, and in
    float16 the un-refreshed probabilities would overflow) or has a standard deviation of 8 ("wide")."""
    B, N, S, H, D = 1, 3, 160, 2, 32
    inp = workloads.evoattention_inputs(B, N, S, H, D, 7, dtype=dtype, seed=77)
    if kind == "ramp":
        inp["bias"] = inp["bias"] + 15.0 * (torch.arange(S) // 32).to(torch.float32)
    else:
        inp["bias"] = inp["bias"] * 8.0
    got = run_op(to_dev(inp))
    assert all(torch.isfinite(g).all() for g in got)
    # fp32: the logits themselves reach 60..80 here, where one fp32 rounding of a logit is 4e-6..8e-6, i.e.
    # that much RELATIVE error in a probability; the 1e-5 / 1e-4 bar is meant for logits of order one
    want = oracle_all(inp)
    if dtype == torch.float32:
        check(got, want, dtype, tol=dict(rtol=2e-3, atol=1e-4))
        return
    # 16-bit types: O and dV at the usual bar.  With near one-hot rows dS = P (dP - delta) is a cancellation
    # (dP_j -> delta where P_j -> 1) whose delta = <dO, O> is formed from the ROUNDED output O, in the
    # reference (evoattention.py:298) as here: an absolute error of |dO| |O| 2^-9 sqrt(D) ~ 0.03 that no
    # kernel can avoid; dQ, dK and dBias, which are sums of dS, get 3x the absolute bar.
    check((got[0], got[3]), (want[0], want[3]), dtype, names=("O", "dV"))
    check((got[1], got[2], got[4]), (want[1], want[2], want[4]), dtype, names=("dQ", "dK", "dBias"),
          tol=dict(rtol=2e-2, atol=6e-2))


# the largest cases of the reference's own sweep (tests/test_evoattention.py:121-135, float16 there too)
LARGE = [(5, 200, 384, 10, 64), (1, 200, 640, 15, 64), (1, 100, 768, 5, 64)]


@pytest.mark.parametrize("B,N,S,H,D", LARGE)
def test_reference_large_cases(B, N, S, H, D):
    """Full-size run; O, dQ, dK, dV of a few rows against the oracle (rows are independent problems), the bias
    gradient through what does not need the N * H * S * S scores on the CPU: it is additive over rows, zero
    at masked keys and reproducible bit for bit."""
    print("large case", B, N, S, H, D, flush=True)
    dtype, nm = torch.float16, 21
    gen = torch.Generator(device="cuda").manual_seed(S + H)
    q, k, v, dO = (torch.randn(B, N, S, H, D, generator=gen, device="cuda", dtype=torch.float32).to(dtype) for _ in range(4))
    bias = torch.randn(B, 1, H, S, S, generator=gen, device="cuda")
    mask = torch.zeros(B, N, 1, 1, S, device="cuda")
    mask[..., S - nm:] = float("-inf")
    dev = {"q": q, "k": k, "v": v, "dO": dO, "bias": bias, "mask": mask}
    got = run_op(dev)
    for b, n in ((0, 0), (B - 1, N - 1), (B // 2, 77 % N)):
        sl = (slice(b, b + 1), slice(n, n + 1))
        want = oe.evo_attention_chunked(q[sl].cpu(), k[sl].cpu(), v[sl].cpu(), mask[sl].cpu(), bias[b:b + 1].cpu(),
                                        dO[sl].cpu(), dtype=f64)
        check([g[sl] for g in got[:4]], want[:4], dtype, names=("O", "dQ", "dK", "dV"))
    dB = got[4]
    assert torch.count_nonzero(dB[..., -nm:]) == 0
    assert torch.count_nonzero(got[2][:, :, -nm:]) == 0 and torch.count_nonzero(got[3][:, :, -nm:]) == 0
    half = N // 2
    parts = []
    for rows in (slice(0, half), slice(half, N)):
        sub = {n_: (t[:, rows] if n_ != "bias" else t) for n_, t in dev.items()}
        parts.append(run_op(sub)[4].float())
    # float16 rounding of three different sums of up to N terms: compare at the scale of the gradient
    torch.testing.assert_close(dB.float(), parts[0] + parts[1], rtol=2e-2, atol=2e-2 * float(dB.float().abs().max()) / 8)
    again = run_op(dev)
    assert all(torch.equal(a_, b_) for a_, b_ in zip(got, again))


def test_config1_fp32_forward_against_golden():
    inp = workloads.config1()
    dev = to_dev(inp)
    O, lse, _ = evoattention_forward(dev["q"], dev["k"], dev["v"], dev["mask"], dev["bias"])
    g = np.load(os.path.join(GOLD, "evoattn_c1.npz"))
    np.testing.assert_allclose(O[0, ::16, ::8].cpu().numpy(), g["o_rows"], rtol=1e-4, atol=1e-5)
    np.testing.assert_allclose(lse[0, ::16, :, ::8].cpu().numpy(), g["lse_rows"], rtol=1e-4, atol=1e-5)
    np.testing.assert_allclose(O.double().sum(dim=(0, 1, 2)).cpu().numpy(), g["o_colsum"], rtol=1e-4, atol=1e-3)
    # masked keys (last 8) have exactly zero probability: perturbing them changes no bit
    k2, v2 = dev["k"].clone(), dev["v"].clone()
    k2[:, :, -8:] += 7.0
    v2[:, :, -8:] -= 3.0
    O2, lse2, _ = evoattention_forward(dev["q"], k2, v2, dev["mask"], dev["bias"])
    assert torch.equal(O, O2) and torch.equal(lse, lse2)


def test_small_fp32_backward_against_golden():
    g = np.load(os.path.join(GOLD, "evoattn_small_bwd.npz"))
    inp = workloads.evoattention_inputs(2, 3, 45, 2, 16, 7, dtype=torch.float32, seed=3, mask_value=-1e9)
    got = run_op(to_dev(inp))
    for name, t in zip(("o", "dq", "dk", "dv", "dbias"), got):
        np.testing.assert_allclose(t.cpu().numpy(), g[name], rtol=1e-4, atol=1e-5, err_msg=name)


def test_config2_full_size_parity_and_properties():
    """C2: [1, 384, 384, 4, 32] bf16, last 38 keys padded — the headline workload."""
    inp = workloads.config2()
    dev = to_dev(inp)
    got = run_op(dev)
    check(got, oracle_all(inp, chunk=48), torch.bfloat16)
    O, dQ, dK, dV, dB = got
    # masked keys: exactly zero gradient
    assert torch.count_nonzero(dK[:, :, -38:]) == 0 and torch.count_nonzero(dV[:, :, -38:]) == 0
    assert torch.count_nonzero(dB[..., -38:]) == 0
    # rows of dS sum to zero, hence rows of dBias do (sum over 384 rows of bf16-rounded terms)
    assert dB.float().sum(-1).abs().max() < 0.5
    # run-to-run bitwise reproducibility (no atomics anywhere)
    again = run_op(dev)
    for a, b in zip(got, again):
        assert torch.equal(a, b)
    # every row n is an independent problem: a slice of rows reproduces the same bits
    sl = slice(100, 108)
    O_sl, _, _ = evoattention_forward(dev["q"][:, sl], dev["k"][:, sl], dev["v"][:, sl], dev["mask"][:, sl], dev["bias"])
    assert torch.equal(O_sl, O[:, sl])


@pytest.mark.parametrize("kind", ["-inf", "-1e9", "bool", "bf16", "broadcast", "fully_masked_row"])
def test_mask_conventions(kind):
    B, N, S, H, D = 2, 3, 96, 2, 32
    inp = workloads.evoattention_inputs(B, N, S, H, D, 11, dtype=torch.bfloat16, seed=21)
    ref_inp = dict(inp)
    if kind == "-1e9":
        inp = workloads.evoattention_inputs(B, N, S, H, D, 11, dtype=torch.bfloat16, seed=21, mask_value=-1e9)
        ref_inp = dict(inp)
    elif kind == "bool":
        inp["mask"] = inp["mask"] == 0
        ref_inp = dict(inp)
    elif kind == "bf16":
        inp["mask"] = inp["mask"].to(torch.bfloat16)
    elif kind == "broadcast":
        inp["mask"] = inp["mask"][:1, :1].clone()
        inp["bias"] = inp["bias"][:1].clone()
        ref_inp = dict(inp, mask=inp["mask"].expand(B, N, 1, 1, S), bias=inp["bias"].expand(B, 1, H, S, S))
    elif kind == "fully_masked_row":
        inp["mask"][0, 1] = float("-inf")
        ref_inp = dict(inp)
    got = run_op(to_dev(inp))
    want = list(oe.evo_attention_chunked(ref_inp["q"], ref_inp["k"], ref_inp["v"], ref_inp["mask"], ref_inp["bias"],
                                         ref_inp["dO"], dtype=f64))
    if kind == "broadcast":
        want[4] = want[4].sum(0, keepdim=True)
    check(got, want, torch.bfloat16)
    assert torch.count_nonzero(got[2][:, :, -11:]) == 0      # dK at masked keys
    if kind == "fully_masked_row":
        assert torch.count_nonzero(got[0][0, 1]) == 0 and torch.count_nonzero(got[1][0, 1]) == 0


def test_strided_views_of_a_fused_projection_and_bf16_bias():
    """q and k/v as the model produces them: views of [B*N, S, H*D] / chunk(2) of [.., 2*H*D]
    (megafold/model/attention.py:177-182, 469-479), bias in bf16."""
    B, N, S, H, D = 1, 6, 128, 4, 32
    inp = workloads.evoattention_inputs(B, N, S, H, D, 9, dtype=torch.bfloat16, seed=5, bias_dtype=torch.bfloat16)
    dev = to_dev(inp)
    kv = torch.cat([dev["k"].reshape(B, N, S, H * D), dev["v"].reshape(B, N, S, H * D)], dim=-1)
    k_view, v_view = (t.reshape(B, N, S, H, D) for t in kv.chunk(2, dim=-1))
    assert not k_view.is_contiguous()
    dev2 = dict(dev, k=k_view, v=v_view)
    got = run_op(dev2)
    check(got, oracle_all(inp), torch.bfloat16)
    assert got[4].dtype == torch.bfloat16


def test_no_bias_gradient_requested_and_function_signature():
    inp = workloads.evoattention_inputs(1, 2, 64, 2, 32, 4, dtype=torch.bfloat16, seed=9)
    dev = to_dev(inp)
    got = run_op(dev, need_bias_grad=False)
    assert got[4] is None
    check(got[:4], oracle_all(inp)[:4], torch.bfloat16)
    assert TritonEvoformer.__self__ is EvoformerAttention
    with pytest.raises(AssertionError):   # the reference asserts equal head dims (evoattention.py:695-696)
        TritonEvoformer(dev["q"], dev["k"][..., :16], dev["v"], dev["mask"], dev["bias"])


@pytest.mark.parametrize("B,N,S,H,D,nm,dtype,bias_dtype", [(1, 5, 100, 4, 32, 7, torch.bfloat16, torch.float32),
                                                           (2, 3, 64, 2, 16, 0, torch.float16, torch.bfloat16),
                                                           (1, 4, 72, 3, 64, 5, torch.float32, torch.float32)])
def test_backward_reads_the_bias_tiles_the_forward_left(B, N, S, H, D, nm, dtype, bias_dtype):
    """The forward can leave the pair bias in the backward's tile order (one preparation launch for both orders);
    a backward given those tiles must return exactly what it returns after preparing its own copy, from a smaller
    workspace, and the forward's own results must not depend on the option."""
    import ctypes as C
    from megafold_amd import _lib
    inp = workloads.evoattention_inputs(B, N, S, H, D, nm, dtype=dtype, seed=21, bias_dtype=bias_dtype)
    dev = to_dev(inp)
    O1, lse1, saved1 = evoattention_forward(dev["q"], dev["k"], dev["v"], dev["mask"], dev["bias"])
    O2, lse2, saved2 = evoattention_forward(dev["q"], dev["k"], dev["v"], dev["mask"], dev["bias"], save_bias_tiles=True)
    assert len(saved1) == 5 and len(saved2) == 6
    assert torch.equal(O1, O2) and torch.equal(lse1, lse2)
    want = evoattention_backward(dev["dO"], *saved1, O1, lse1, True)
    got = evoattention_backward(dev["dO"], *saved2[:5], O2, lse2, True, bias_tiles=saved2[5])
    for w, g_ in zip(want, got):
        assert torch.equal(w, g_)
    a = _lib.EvoAttnArgs()
    a.B, a.N, a.S, a.H, a.D = B, N, S, H, D
    a.dtype = _lib.dtype_code(dtype)
    a.dbias = 0x10000
    full = _lib.lib().mf_evoattn_bwd_workspace_bytes(C.byref(a))
    a.bias_tiles_bwd = 0x20000
    assert full - _lib.lib().mf_evoattn_bwd_workspace_bytes(C.byref(a)) == _lib.lib().mf_evoattn_bias_tiles_bytes(C.byref(a)) == saved2[5].numel()


@pytest.mark.parametrize("B,N,S,H,D,nm,dtype", [(1, 24, 100, 4, 32, 7, torch.bfloat16), (2, 9, 64, 2, 16, 0, torch.float16),
                                                 (1, 40, 72, 3, 64, 5, torch.float32), (1, 300, 416, 4, 32, 20, torch.bfloat16)])
def test_memory_lean_order_matches_the_default_order(B, N, S, H, D, nm, dtype):
    """MF_EVO_BWD_LEAN: delta from its own kernel, the bias gradient before dQ/dK/dV with its partial sums in the dQ
    buffer.  dQ, dK, dV come from the same kernel on the same inputs and must be identical; the bias gradient sees a
    delta summed in another order and must agree to fp32 rounding; the workspace must be smaller by the partial sums."""
    import ctypes as C
    from megafold_amd import _lib
    inp = workloads.evoattention_inputs(B, N, S, H, D, nm, dtype=dtype, seed=33)
    dev = to_dev(inp)
    O, lse, saved = evoattention_forward(dev["q"], dev["k"], dev["v"], dev["mask"], dev["bias"])
    want = evoattention_backward(dev["dO"], *saved, O, lse, True, lean=False)
    got = evoattention_backward(dev["dO"], *saved, O, lse, True, lean=True)
    for w, g_ in zip(want[:3], got[:3]):
        assert torch.equal(w, g_)
    scale = float(want[3].abs().max())
    assert float((want[3] - got[3]).abs().max()) <= 2e-5 * max(scale, 1.0)
    calls = []
    got2 = evoattention_backward(dev["dO"], *saved, O, lse, True, lean=True, phase_hook=calls.append)   # split phases
    # the order is taken where dQ can hold the partial sums (the wrapper asks mf_evoattn_bwd_lean_ok); small dQ buffers
    # keep the default order
    assert calls[::2] in (["prep", "dbias", "dqkv"], ["prep", "dqkv", "dbias"])
    if (N, S) in ((300, 416), (40, 72)):
        assert calls[::2] == ["prep", "dbias", "dqkv"]
    for a_, b_ in zip(got, got2):
        assert torch.equal(a_, b_)
    # a strided dQ cannot hold the partial sums: the library says so and the wrapper keeps the default order
    wide = torch.empty((B, N, S, H, 2 * D), dtype=dtype, device="cuda")
    outs = (wide[..., :D], torch.empty_like(O), torch.empty_like(O))
    got3 = evoattention_backward(dev["dO"], *saved, O, lse, True, lean=True, out=outs)
    for w, g_ in zip(want, got3):
        assert torch.equal(w, g_)


def test_config2_memory_lean_peak_activation():
    """C2 with the memory-lean order: the peak of forward + backward stays within the O(N S H D) bound (150.75 MiB) plus the
    tiled copies of the pair bias (two of 2.25 MiB: the forward's and the one kept for the backward)."""
    from megafold_amd.model.FusedEvoAttention import evoattention as ev
    dev = to_dev(workloads.config2())
    q, k, v = (dev[n_].requires_grad_() for n_ in "qkv")
    bias = dev["bias"].requires_grad_()
    old = ev.MEMORY_LEAN
    ev.MEMORY_LEAN = True
    try:
        torch.cuda.synchronize()
        torch.cuda.empty_cache()
        torch.cuda.reset_peak_memory_stats()
        base = torch.cuda.memory_allocated()
        o = TritonEvoformer(q, k, v, dev["mask"], bias)
        o.backward(dev["dO"])
        torch.cuda.synchronize()
        peak = (torch.cuda.max_memory_allocated() - base) / 2 ** 20
    finally:
        ev.MEMORY_LEAN = old
    print("C2 memory-lean peak %.2f MiB" % peak, flush=True)
    assert peak <= 155.5


def test_config5_peak_activation_memory():
    """C5 [1, 768, 768, 4, 32]: peak extra memory of fwd+bwd stays at the O(N*S*H*D) bound — O, dQ, dK,
    dV (144 MiB each) + LSE, delta, dBias (9 MiB each) — plus the declared workspace (the 9 MiB tiled copy of
    the pair bias and six partial bias gradients of 9 MiB: seven row chunks, the first of which sums into dBias
    itself); nothing of size N*H*S*S (6.75 GiB) is ever allocated."""
    inp = workloads.config5()
    dev = to_dev(inp)
    q, k, v = (dev[n].requires_grad_() for n in "qkv")
    bias = dev["bias"].requires_grad_()
    torch.cuda.synchronize()
    torch.cuda.reset_peak_memory_stats()
    base = torch.cuda.memory_allocated()
    out = TritonEvoformer(q, k, v, dev["mask"], bias)
    out.backward(dev["dO"])
    torch.cuda.synchronize()
    peak_mib = (torch.cuda.max_memory_allocated() - base) / 2 ** 20
    bound = 4 * 144 + 3 * 9
    workspace = 6 * 9 + 9
    print("C5 peak activation MiB: %.1f (bound %d + workspace %d)" % (peak_mib, bound, workspace), flush=True)
    assert peak_mib <= bound + workspace + 1
    # Parity of O, dQ, dK, dV on row slices against the float64 oracle (rows are independent problems; the full-size
    # oracle would need 6.75 GiB of scores).  The persistent dQ/dK/dV kernel walks twelve (row, head) problems of two
    # passes each per work-group here and reuses its fp32 dQ array from problem to problem: rows 0..3 are first
    # problems of their work-groups, rows 300.. and 764.. are handled as second or later ones.
    dev_bias = inp["bias"]
    for lo in (0, 300, 764):
        sl = slice(lo, lo + 4)
        want = oe.evo_attention_chunked(inp["q"][:, sl], inp["k"][:, sl], inp["v"][:, sl], inp["mask"][:, sl], dev_bias,
                                        inp["dO"][:, sl], dtype=f64)
        check([out[:, sl].detach(), q.grad[:, sl], k.grad[:, sl], v.grad[:, sl]], want[:4], torch.bfloat16,
              names=("O", "dQ", "dK", "dV"))
    assert torch.count_nonzero(k.grad[:, :, -96:]) == 0 and torch.count_nonzero(v.grad[:, :, -96:]) == 0
    # The bias gradient through what does not need the N * H * S * S scores on the CPU: zero at masked keys, additive
    # over the rows (two half-size calls), rows of dS sum to zero, reproducible bit for bit.
    dB = bias.grad
    assert torch.count_nonzero(dB[..., -96:]) == 0
    assert dB.float().sum(-1).abs().max() < 1.0
    parts = []
    for rows in (slice(0, 384), slice(384, 768)):
        sub = {n_: (t[:, rows] if n_ != "bias" else t) for n_, t in dev.items()}
        parts.append(run_op({k_: v_.detach() for k_, v_ in sub.items()})[4].float())
    # bf16 roundings of three different sums of up to 768 terms: compare at the scale of the gradient
    torch.testing.assert_close(dB.float(), parts[0] + parts[1], rtol=2e-2, atol=2e-2 * float(dB.float().abs().max()) / 8)
    again = run_op({k_: v_.detach() for k_, v_ in dev.items()})
    assert torch.equal(again[1], q.grad) and torch.equal(again[2], k.grad) and torch.equal(again[3], v.grad)
    assert torch.equal(again[4], dB)


@pytest.mark.gpu
def test_tensors_beyond_two_to_the_31_elements_match_their_row_slices():
    """[1, 17000, 512, 8, 32] bf16: 2.2e9 elements (4.4 GB) per tensor, so that element and byte offsets of the later
    rows pass 2^31.  The rows n are independent problems: O, dQ, dK, dV of the full call must equal, bit for bit, those
    of calls on row slices (whose offsets are small), near the end of the tensors and over both halves; dBias of the
    halves must add up to the full one within the rounding of the 16-bit outputs."""
    B, N, S, H, D = 1, 17000, 512, 8, 32
    torch.manual_seed(0)
    mk = lambda *sh: torch.randn(*sh, device="cuda").to(torch.bfloat16)
    q, k, v, dO = (mk(B, N, S, H, D) for _ in range(4))
    bias = mk(B, 1, H, S, S)
    mask = torch.zeros(B, N, 1, 1, S, device="cuda")
    mask[..., S - 37:] = float("-inf")

    def run(sl):
        qq, kk, vv = (t[:, sl].detach().clone().requires_grad_() for t in (q, k, v))
        bb = bias.detach().clone().requires_grad_()
        o = TritonEvoformer(qq, kk, vv, mask[:, sl], bb)
        o.backward(dO[:, sl])
        return o.detach(), qq.grad, kk.grad, vv.grad, bb.grad

    full = run(slice(0, N))
    assert all(bool(torch.isfinite(t.float()).all()) for t in full)
    halves = []
    for sl in (slice(N - 8, N), slice(N - 305, N - 295), slice(0, N // 2), slice(N // 2, N)):
        part = run(sl)
        for name, a, b in zip(("O", "dQ", "dK", "dV"), full[:4], part[:4]):
            assert torch.equal(a[:, sl], b), "%s of rows %s differs from the sliced call" % (name, sl)
        if sl.stop - sl.start == N // 2:
            halves.append(part[4].float())
        del part
    want = halves[0] + halves[1]
    torch.testing.assert_close(full[4].float(), want, rtol=2 ** -7, atol=2 ** -7 * float(want.abs().max()))
