"""Pins the LayerNorm->Linear, SwiGLU and Transition oracles (CPU) against library routines
(F.layer_norm, F.linear, F.silu), autograd in float64, explicit loops and identities."""
import os

import numpy as np
import pytest
import torch
import torch.nn.functional as F

from megafold_amd import workloads
from oracle import layernorm_linear as ol
from oracle import transition as ot

f64 = torch.float64
GOLD = os.path.join(os.path.dirname(__file__), "golden")


def small(seed=5, bias=True):
    inp = workloads.lnlinear_inputs((3, 7), 16, 24, dtype=torch.float32, seed=seed)
    inp["b"] = torch.linspace(-1, 1, 24) if bias else None
    return inp


@pytest.mark.parametrize("bias", [True, False])
def test_forward_matches_library_routines(bias):
    inp = small(bias=bias)
    out = ol.layernorm_linear_forward(inp["x"], inp["gamma"], inp["beta"], inp["W"], inp["b"], dtype=f64)
    ref = F.linear(F.layer_norm(inp["x"].double(), (16,), inp["gamma"].double(), inp["beta"].double(), 1e-5),
                   inp["W"].double().t(), inp["b"].double() if bias else None)
    torch.testing.assert_close(out, ref, rtol=1e-12, atol=1e-12)
    # the reference's test form: nn.Linear(nn.LayerNorm(x)) with weight = linear_weight^T (tests/test_layernormlinear.py:17-22)
    ln, lin = torch.nn.LayerNorm(16).double(), torch.nn.Linear(16, 24, bias=bias).double()
    with torch.no_grad():
        ln.weight.copy_(inp["gamma"]); ln.bias.copy_(inp["beta"]); lin.weight.copy_(inp["W"].t())
        if bias:
            lin.bias.copy_(inp["b"])
    torch.testing.assert_close(out, lin(ln(inp["x"].double())), rtol=1e-12, atol=1e-12)


def test_forward_matches_explicit_loops():
    inp = small()
    out = ol.layernorm_linear_forward(inp["x"], inp["gamma"], inp["beta"], inp["W"], inp["b"], dtype=f64).numpy()
    x, g, bt, W, b = (inp[n].double().numpy() for n in ("x", "gamma", "beta", "W", "b"))
    for i in range(3):
        for j in range(7):
            row = x[i, j]
            mu = sum(row) / 16
            var = sum((v - mu) ** 2 for v in row) / 16
            y = [(row[k] - mu) / np.sqrt(var + 1e-5) * g[k] + bt[k] for k in range(16)]
            for n in range(24):
                np.testing.assert_allclose(out[i, j, n], sum(y[k] * W[k, n] for k in range(16)) + b[n], rtol=1e-11, atol=1e-12)


def test_backward_closed_forms_match_autograd():
    inp = small()
    x, g, bt, W, b = (inp[n].double().requires_grad_() for n in ("x", "gamma", "beta", "W", "b"))
    out = F.linear(F.layer_norm(x, (16,), g, bt, 1e-5), W.t(), b)
    out.backward(inp["dY"].double())
    dx, dW, db, dg, dbt = ol.layernorm_linear_backward(inp["dY"], inp["x"], inp["gamma"], inp["beta"], inp["W"], dtype=f64)
    for got, want in ((dx, x.grad), (dW, W.grad), (db, b.grad), (dg, g.grad), (dbt, bt.grad)):
        torch.testing.assert_close(got, want, rtol=1e-9, atol=1e-11)


def test_layernorm_invariants():
    inp = small()
    x = inp["x"].double()
    out = ol.layernorm_linear_forward(x, inp["gamma"], inp["beta"], inp["W"], None, eps=0.0, dtype=f64)
    out2 = ol.layernorm_linear_forward(3.5 * x + 2.0, inp["gamma"], inp["beta"], inp["W"], None, eps=0.0, dtype=f64)
    torch.testing.assert_close(out, out2, rtol=1e-9, atol=1e-10)     # affine invariance per row
    eye = ol.layernorm_linear_forward(x, torch.ones(16), torch.zeros(16), torch.eye(16), None, dtype=f64)
    assert eye.mean(-1).abs().max() < 1e-12 and (eye.var(-1, unbiased=False) - 1).abs().max() < 1e-3
    dx, *_ = ol.layernorm_linear_backward(inp["dY"], inp["x"], inp["gamma"], inp["beta"], inp["W"], dtype=f64)
    assert dx.sum(-1).abs().max() < 1e-12                           # LN backward projects out the constant direction
    mean, rstd = ol.layernorm_stats(x)
    xhat = (x - mean) * rstd
    assert (dx * xhat).sum(-1).abs().max() < 1e-3                   # ... and x_hat, up to eps / (var + eps)


def test_swiglu_matches_silu_and_autograd_and_special_values():
    u = torch.randn(5, 12, generator=torch.Generator().manual_seed(1)).double().requires_grad_()
    y = ot.swiglu_forward(u, f64)
    a, g = u.chunk(2, -1)
    torch.testing.assert_close(y, F.silu(g) * a, rtol=1e-13, atol=1e-14)   # gate = SECOND half
    dy = torch.randn(5, 6, generator=torch.Generator().manual_seed(2)).double()
    y.backward(dy)
    torch.testing.assert_close(ot.swiglu_backward(dy, u.detach(), f64), u.grad, rtol=1e-11, atol=1e-13)
    z = torch.tensor([[2.0, -3.0, 0.0, 0.0]])                      # gate 0: y = 0 and d/dgate = dy * 0.5 * a
    assert ot.swiglu_forward(z, f64).abs().max() == 0
    torch.testing.assert_close(ot.swiglu_backward(torch.ones(1, 2), z, f64)[:, 2:], torch.tensor([[1.0, -1.5]], dtype=f64))
    big = torch.tensor([[2.0, 40.0]])                               # gate -> +inf: y -> a * gate
    torch.testing.assert_close(ot.swiglu_forward(big, f64), torch.tensor([[80.0]], dtype=f64))


def test_transition_is_the_composition():
    inp = workloads.transition_inputs((2, 5), 16, 4, dtype=torch.float32, seed=7)
    y = ot.transition_forward(inp["x"], inp["gamma"], inp["beta"], inp["W1"], inp["W2"], dtype=f64)
    h = F.layer_norm(inp["x"].double(), (16,), inp["gamma"].double(), inp["beta"].double(), 1e-5) @ inp["W1"].double()
    a, g = h.chunk(2, -1)
    torch.testing.assert_close(y, F.linear(F.silu(g) * a, inp["W2"].double()), rtol=1e-12, atol=1e-12)


def test_golden_fixtures_reproduce():
    g = np.load(os.path.join(GOLD, "lnlinear_small.npz"))
    inp = workloads.lnlinear_inputs((3, 37), 64, 48, dtype=torch.float32, seed=5)
    out = ol.layernorm_linear_forward(inp["x"], inp["gamma"], inp["beta"], inp["W"], torch.from_numpy(g["b"]), dtype=f64)
    np.testing.assert_allclose(out.numpy(), g["out"], rtol=1e-12, atol=1e-13)
    t = np.load(os.path.join(GOLD, "transition_small.npz"))
    inp = workloads.transition_inputs((2, 29), 32, 4, dtype=torch.float32, seed=7)
    y = ot.transition_forward(inp["x"], inp["gamma"], inp["beta"], inp["W1"], inp["W2"], dtype=f64)
    np.testing.assert_allclose(y.numpy(), t["y"], rtol=1e-12, atol=1e-13)
