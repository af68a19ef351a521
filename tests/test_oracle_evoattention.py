"""Pins the attention oracle (CPU).  The reference holds no golden vectors for this op, so the oracle
is pinned against a library routine, an explicit float64 loop, autograd and invariants chosen so that
a dropped term, a wrong sign, a transposed operand or a wrong mask convention fails at least one."""
import os

import numpy as np
import pytest
import torch
import torch.nn.functional as F

from megafold_amd import workloads
from oracle import evoattention as oe

f64 = torch.float64
GOLD = os.path.join(os.path.dirname(__file__), "golden")


def small(B=2, N=3, S=13, H=2, D=8, nm=4, seed=11, mask_value=float("-inf")):
    return workloads.evoattention_inputs(B, N, S, H, D, nm, dtype=torch.float32, seed=seed, mask_value=mask_value)


def test_forward_matches_library_sdpa():
    inp = small()
    O, _ = oe.evo_attention_forward(inp["q"], inp["k"], inp["v"], inp["mask"], inp["bias"], dtype=f64)
    q, k, v = (inp[n].double().permute(0, 1, 3, 2, 4) for n in "qkv")  # [B, N, H, S, D]
    attn_mask = inp["bias"].double() + inp["mask"].double()             # broadcast to [B, N, H, S, S]
    ref = F.scaled_dot_product_attention(q, k, v, attn_mask=attn_mask.expand(2, 3, 2, 13, 13))
    torch.testing.assert_close(O, ref.permute(0, 1, 3, 2, 4), rtol=1e-10, atol=1e-12)


def test_forward_matches_bruteforce_loops():
    inp = small(B=1, N=2, S=6, H=2, D=4, nm=2)
    O, lse = oe.evo_attention_forward(inp["q"], inp["k"], inp["v"], inp["mask"], inp["bias"], dtype=f64)
    q, k, v, b, m = (inp[n].double().numpy() for n in ("q", "k", "v", "bias", "mask"))
    B, N, S, H, D = q.shape
    for n in range(N):
        for h in range(H):
            for i in range(S):
                z = np.array([sum(q[0, n, i, h, d] * k[0, n, j, h, d] for d in range(D)) / np.sqrt(D)
                              + b[0, 0, h, i, j] + m[0, n, 0, 0, j] for j in range(S)])
                mx = z.max()
                e = np.exp(z - mx)
                p = e / e.sum()
                o = sum(p[j] * v[0, n, j, h] for j in range(S))
                np.testing.assert_allclose(O[0, n, i, h].numpy(), o, rtol=1e-12, atol=1e-13)
                np.testing.assert_allclose(lse[0, n, h, i].item(), mx + np.log(e.sum()), rtol=1e-12)


def test_masked_keys_cannot_influence_output():
    inp = small()
    O1, l1 = oe.evo_attention_forward(inp["q"], inp["k"], inp["v"], inp["mask"], inp["bias"], dtype=f64)
    k2, v2 = inp["k"].clone(), inp["v"].clone()
    k2[:, :, -4:] += 3.0
    v2[:, :, -4:] -= 5.0
    O2, l2 = oe.evo_attention_forward(inp["q"], k2, v2, inp["mask"], inp["bias"], dtype=f64)
    assert torch.equal(O1, O2) and torch.equal(l1, l2)


def test_shift_invariance_and_lse_shift():
    inp = small(nm=0)
    c = torch.randn(2, 1, 2, 13, 1, generator=torch.Generator().manual_seed(1)).double()
    O1, l1 = oe.evo_attention_forward(inp["q"], inp["k"], inp["v"], inp["mask"], inp["bias"].double(), dtype=f64)
    O2, l2 = oe.evo_attention_forward(inp["q"], inp["k"], inp["v"], inp["mask"], inp["bias"].double() + c, dtype=f64)
    torch.testing.assert_close(O1, O2, rtol=1e-10, atol=1e-12)
    torch.testing.assert_close(l2 - l1, c[:, 0, :, :, 0].unsqueeze(1).expand_as(l1), rtol=1e-10, atol=1e-10)


def test_zero_query_zero_bias_gives_mean_of_unmasked_values():
    inp = small()
    O, _ = oe.evo_attention_forward(torch.zeros_like(inp["q"]), inp["k"], inp["v"], inp["mask"],
                                    torch.zeros_like(inp["bias"]), dtype=f64)
    mean_v = inp["v"].double()[:, :, :9].mean(dim=2, keepdim=True).expand_as(O)
    torch.testing.assert_close(O, mean_v, rtol=1e-12, atol=1e-12)


def test_rows_are_independent_and_chunking_is_exact():
    inp = small(N=5)
    O, _ = oe.evo_attention_forward(inp["q"], inp["k"], inp["v"], inp["mask"], inp["bias"], dtype=f64)
    for n in range(5):
        On, _ = oe.evo_attention_forward(inp["q"][:, n:n + 1], inp["k"][:, n:n + 1], inp["v"][:, n:n + 1],
                                         inp["mask"][:, n:n + 1], inp["bias"], dtype=f64)
        torch.testing.assert_close(O[:, n:n + 1], On, rtol=0, atol=0)
    full = oe.evo_attention_backward(inp["dO"], inp["q"], inp["k"], inp["v"], inp["mask"], inp["bias"], dtype=f64)
    Oc, dq, dk, dv, db = oe.evo_attention_chunked(inp["q"], inp["k"], inp["v"], inp["mask"], inp["bias"], inp["dO"],
                                                  chunk=2, dtype=f64)
    torch.testing.assert_close(Oc, O, rtol=0, atol=0)
    for a, b in zip((dq, dk, dv, db), full):
        torch.testing.assert_close(a, b, rtol=1e-12, atol=1e-13)


@pytest.mark.parametrize("mask_value", [float("-inf"), -1e9])
def test_backward_closed_forms_match_autograd(mask_value):
    inp = small(mask_value=mask_value)
    q, k, v, b = (inp[n].double().requires_grad_() for n in ("q", "k", "v", "bias"))
    O, _ = oe.evo_attention_forward(q, k, v, inp["mask"], b, dtype=f64)
    O.backward(inp["dO"].double())
    dq, dk, dv, db = oe.evo_attention_backward(inp["dO"], inp["q"], inp["k"], inp["v"], inp["mask"], inp["bias"], dtype=f64)
    for got, want in ((dq, q.grad), (dk, k.grad), (dv, v.grad), (db, b.grad)):
        torch.testing.assert_close(got, want, rtol=1e-9, atol=1e-11)


def test_backward_invariants():
    inp = small(N=1)
    dq, dk, dv, db = oe.evo_attention_backward(inp["dO"], inp["q"], inp["k"], inp["v"], inp["mask"], inp["bias"], dtype=f64)
    # softmax Jacobian: every row of dS sums to zero (N = 1, so dBias == dS)
    assert db.sum(-1).abs().max() < 1e-12
    # masked keys: exactly zero gradients
    assert torch.count_nonzero(dk[:, :, -4:]) == 0 and torch.count_nonzero(dv[:, :, -4:]) == 0
    assert torch.count_nonzero(db[..., -4:]) == 0
    assert dk[:, :, :9].abs().max() > 0


def test_bool_mask_is_keep_mask_and_fully_masked_rows_are_zero():
    inp = small()
    keep = torch.ones(2, 3, 1, 1, 13, dtype=torch.bool)
    keep[..., -4:] = False
    O1, _ = oe.evo_attention_forward(inp["q"], inp["k"], inp["v"], keep, inp["bias"], dtype=f64)
    O2, _ = oe.evo_attention_forward(inp["q"], inp["k"], inp["v"], inp["mask"], inp["bias"], dtype=f64)
    assert torch.equal(O1, O2)
    dead = inp["mask"].clone()
    dead[:, 1] = float("-inf")
    O3, l3 = oe.evo_attention_forward(inp["q"], inp["k"], inp["v"], dead, inp["bias"], dtype=f64)
    assert torch.count_nonzero(O3[:, 1]) == 0 and torch.isneginf(l3[:, 1]).all() and not torch.isnan(O3).any()
    grads = oe.evo_attention_backward(inp["dO"], inp["q"], inp["k"], inp["v"], dead, inp["bias"], dtype=f64)
    assert all(not torch.isnan(g).any() for g in grads)
    assert torch.count_nonzero(grads[0][:, 1]) == 0


def test_golden_fixtures_reproduce():
    g = np.load(os.path.join(GOLD, "evoattn_c1.npz"))
    inp = workloads.config1()
    O, lse = oe.evo_attention_forward(inp["q"], inp["k"], inp["v"], inp["mask"], inp["bias"], dtype=f64)
    np.testing.assert_allclose(O[0, ::16, ::8].numpy(), g["o_rows"], rtol=1e-12, atol=1e-14)
    np.testing.assert_allclose(O.sum(dim=(0, 1, 2)).numpy(), g["o_colsum"], rtol=1e-10)
    np.testing.assert_allclose(lse.sum().numpy(), g["lse_sum"], rtol=1e-12)
    # fp32 evaluation of the same formula stays inside the fp32 parity bar
    O32, _ = oe.evo_attention_forward(inp["q"], inp["k"], inp["v"], inp["mask"], inp["bias"], dtype=torch.float32)
    np.testing.assert_allclose(O32[0, ::16, ::8].numpy(), g["o_rows"], rtol=1e-4, atol=1e-5)
