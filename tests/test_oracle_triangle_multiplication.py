"""Pins the triangle-multiplication oracle (CPU) against library modules (nn.LayerNorm, nn.Linear, nn.GLU),
explicit loops over the contraction, identities of the block and finite differences; checks the parameter
names of the fused module against the reference's state-dict keys."""
import pytest
import torch
import torch.nn as nn

from megafold_amd.model.FusedTriangleMultiplication import TriangleMultiplication
from oracle import triangle_multiplication as otm

f64 = torch.float64

# state-dict keys of TriangleMultiplication(dim, mix=...) in the reference (megafold/model/megafold.py:441, 455-458;
# LayernormLinear parameters: megafold/model/FusedLayernormLinear/fused_layernorm_linear.py:511-521)
REFERENCE_KEYS = {"combined.WEIGHT", "combined.BIAS", "combined.linear_weight", "combined.linear_bias",
                  "to_out.0.WEIGHT", "to_out.0.BIAS", "to_out.0.linear_weight"}


def make(b=2, n=6, d=8, seed=0, masked=2):
    g = torch.Generator().manual_seed(seed)
    r = lambda *s: torch.randn(*s, generator=g, dtype=f64)
    params = {
        "combined.WEIGHT": 1 + 0.1 * r(d), "combined.BIAS": 0.1 * r(d),
        "combined.linear_weight": r(d, 5 * d) * d ** -0.5, "combined.linear_bias": 0.1 * r(5 * d),
        "to_out.0.WEIGHT": 1 + 0.1 * r(d), "to_out.0.BIAS": 0.1 * r(d),
        "to_out.0.linear_weight": r(d, d) * d ** -0.5,
    }
    x = r(b, n, n, d)
    mask = torch.ones(b, n, dtype=torch.bool)
    if masked:
        mask[:, n - masked:] = False
        mask[0, 1] = False
    return x, mask, params


def library_composition(x, mask, P, mix):
    """The block written with torch.nn modules and an explicit loop over the contracted index."""
    b, n, _, d = x.shape
    ln1, lin1 = nn.LayerNorm(d).double(), nn.Linear(d, 5 * d).double()
    ln2, lin2 = nn.LayerNorm(d).double(), nn.Linear(d, d, bias=False).double()
    with torch.no_grad():
        ln1.weight.copy_(P["combined.WEIGHT"]); ln1.bias.copy_(P["combined.BIAS"])
        lin1.weight.copy_(P["combined.linear_weight"].t()); lin1.bias.copy_(P["combined.linear_bias"])
        ln2.weight.copy_(P["to_out.0.WEIGHT"]); ln2.bias.copy_(P["to_out.0.BIAS"])
        lin2.weight.copy_(P["to_out.0.linear_weight"].t())
        c = lin1(ln1(x))
        lr = nn.GLU(dim=-1)(c[..., :4 * d])
        left, right = lr[..., :d].clone(), lr[..., d:].clone()
        if mask is not None:
            for bi in range(b):
                for i in range(n):
                    for j in range(n):
                        if not (mask[bi, i] and mask[bi, j]):
                            left[bi, i, j] = 0
                            right[bi, i, j] = 0
        out = torch.zeros(b, n, n, d, dtype=f64)
        for k in range(n):
            if mix == "outgoing":
                out += left[:, :, k, None, :] * right[:, None, :, k, :]          # left[i,k] * right[j,k]
            else:
                out += left[:, k, None, :, :] * right[:, k, :, None, :]          # left[k,j] * right[k,i]
        return lin2(ln2(out)) * torch.sigmoid(c[..., 4 * d:])


@pytest.mark.parametrize("mix", ["outgoing", "incoming"])
@pytest.mark.parametrize("masked", [0, 2])
def test_forward_matches_library_composition(mix, masked):
    x, mask, P = make(masked=masked)
    got = otm.triangle_multiplication_forward(x, mask if masked else None, P, mix)
    want = library_composition(x, mask if masked else None, P, mix)
    torch.testing.assert_close(got, want, rtol=1e-10, atol=1e-12)


def test_incoming_is_outgoing_on_the_transposed_pair_tensor():
    x, mask, P = make(seed=3)
    inc = otm.triangle_multiplication_forward(x, mask, P, "incoming")
    out_t = otm.triangle_multiplication_forward(x.transpose(1, 2), mask, P, "outgoing").transpose(1, 2)
    torch.testing.assert_close(inc, out_t, rtol=1e-12, atol=1e-12)


def test_masked_positions_do_not_reach_kept_outputs():
    x, mask, P = make(seed=4, masked=2)
    base = otm.triangle_multiplication_forward(x, mask, P, "outgoing")
    n = x.shape[1]
    x2 = x.clone()
    x2[:, :, n - 1, :] += torch.linspace(-2, 2, x.shape[-1], dtype=f64)       # column n-1 is masked
    pert = otm.triangle_multiplication_forward(x2, mask, P, "outgoing")
    # left[i, k] / right[j, k] with k = n-1 are zeroed by the mask; the out gate at (i, n-1) still sees x
    torch.testing.assert_close(pert[:, :, : n - 1], base[:, :, : n - 1], rtol=1e-12, atol=1e-12)
    assert not torch.allclose(pert[:, :, n - 1], base[:, :, n - 1])


def test_rank_one_inputs_give_the_closed_form():
    # with LayerNorm weight 0 the projections see only the LayerNorm bias: every position carries the same
    # (left, right) vector, so out[i, j, :] = n * left * right before the output stage
    x, _, P = make(seed=5, masked=0)
    P["combined.WEIGHT"] = torch.zeros_like(P["combined.WEIGHT"])
    got = otm.triangle_multiplication_forward(x, None, P, "incoming")
    n, d = x.shape[1], x.shape[-1]
    c = P["combined.BIAS"] @ P["combined.linear_weight"] + P["combined.linear_bias"]
    lr = c[: 2 * d] * torch.sigmoid(c[2 * d: 4 * d])
    prod = n * lr[:d] * lr[d:]
    o = torch.nn.functional.layer_norm(prod, (d,), P["to_out.0.WEIGHT"], P["to_out.0.BIAS"], 1e-5) @ P["to_out.0.linear_weight"]
    want = (o * torch.sigmoid(c[4 * d:])).expand_as(got)
    torch.testing.assert_close(got, want, rtol=1e-10, atol=1e-12)


def test_gradients_match_finite_differences():
    x, mask, P = make(b=1, n=4, d=8, seed=7, masked=1)
    dout = torch.randn(x.shape, generator=torch.Generator().manual_seed(8), dtype=f64)
    _, dx, dP = otm.triangle_multiplication_forward_backward(x, mask, P, dout, "incoming")
    loss = lambda xx, PP: (otm.triangle_multiplication_forward(xx, mask, PP, "incoming") * dout).sum()
    eps = 1e-6
    for idx in [(0, 1, 2, 3), (0, 2, 0, 5)]:
        xp, xm = x.clone(), x.clone()
        xp[idx] += eps; xm[idx] -= eps
        assert abs((loss(xp, P) - loss(xm, P)) / (2 * eps) - dx[idx]) < 1e-6
    for name, idx in [("combined.linear_weight", (3, 2)), ("combined.linear_weight", (1, 35)), ("combined.WEIGHT", (5,)),
                      ("combined.linear_bias", (20,)), ("to_out.0.linear_weight", (2, 7)), ("to_out.0.BIAS", (0,))]:
        Pp, Pm = dict(P), dict(P)
        Pp[name] = P[name].clone(); Pm[name] = P[name].clone()
        Pp[name][idx] += eps; Pm[name][idx] -= eps
        assert abs((loss(x, Pp) - loss(x, Pm)) / (2 * eps) - dP[name][idx]) < 1e-6, name


@pytest.mark.parametrize("mix", ["outgoing", "incoming"])
def test_fused_module_has_the_reference_parameter_names(mix):
    m = TriangleMultiplication(dim=128, mix=mix, dropout=0.25, dropout_type="row")
    sd = m.state_dict()
    assert set(sd.keys()) == REFERENCE_KEYS
    assert sd["combined.linear_weight"].shape == (128, 640) and sd["to_out.0.linear_weight"].shape == (128, 128)
    with pytest.raises(RuntimeError):
        m(torch.zeros(1, 4, 4, 128))          # no CPU path


@pytest.mark.parametrize("mix", ["outgoing", "incoming"])
def test_golden_fixture_reproduces(mix):
    import os
    import numpy as np
    from megafold_amd import workloads
    g = np.load(os.path.join(os.path.dirname(__file__), "golden", "triangle_blocks_small.npz"))
    w = workloads.triangle_multiplication_inputs(seed=13)
    out, dx, dp = otm.triangle_multiplication_forward_backward(w["x"], w["mask"], w["params"], w["dout"], mix)
    for name, got in (("out", out), ("dx", dx), ("dW1", dp["combined.linear_weight"])):
        torch.testing.assert_close(got.float(), torch.from_numpy(g["mult_%s_%s" % (mix, name)]), rtol=1e-5, atol=1e-6)
