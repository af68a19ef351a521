"""Writes the golden fixtures under tests/golden/ from the CPU oracle.

The reference ships no known-answer vectors for its kernels (its tests draw unseeded random inputs
and compare with an inline eager formula), so the fixtures are produced by this repository's oracle,
in float64, on the seeded inputs of ``megafold_amd.workloads`` — after the oracle itself has been
pinned by ``tests/test_oracle_*.py``.  Run from the repository root:

    python tests/golden/make_golden.py
"""
import os
import sys

import numpy as np
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
HERE = os.path.dirname(os.path.abspath(__file__))

from megafold_amd import workloads  # noqa: E402
from oracle import evoattention as oe  # noqa: E402
from oracle import layernorm_linear as ol  # noqa: E402
from oracle import transition as ot  # noqa: E402
from oracle import triangle_attention as ota  # noqa: E402
from oracle import triangle_multiplication as otm  # noqa: E402

f64 = torch.float64


def attention_c1():
    """Config 1: forward only, fp32 inputs [1, 64, 64, 4, 32], last 8 keys masked with -inf."""
    inp = workloads.config1()
    O, lse = oe.evo_attention_forward(inp["q"], inp["k"], inp["v"], inp["mask"], inp["bias"], dtype=f64)
    np.savez_compressed(os.path.join(HERE, "evoattn_c1.npz"),
                        o_rows=O[0, ::16, ::8].numpy(),            # [4, 8, 4, 32] slice of the output
                        lse_rows=lse[0, ::16, :, ::8].numpy(),
                        o_sum=O.sum().numpy(), o_abs_sum=O.abs().sum().numpy(),
                        o_colsum=O.sum(dim=(0, 1, 2)).numpy(), lse_sum=lse.sum().numpy())


def attention_small_bwd():
    """fwd+bwd on a small ragged shape, -1e9 style mask, fp32 inputs."""
    inp = workloads.evoattention_inputs(2, 3, 45, 2, 16, 7, dtype=torch.float32, seed=3, mask_value=-1e9)
    O, lse = oe.evo_attention_forward(inp["q"], inp["k"], inp["v"], inp["mask"], inp["bias"], dtype=f64)
    dq, dk, dv, db = oe.evo_attention_backward(inp["dO"], inp["q"], inp["k"], inp["v"], inp["mask"], inp["bias"], dtype=f64)
    np.savez_compressed(os.path.join(HERE, "evoattn_small_bwd.npz"), o=O.numpy(), lse=lse.numpy(), dq=dq.numpy(),
                        dk=dk.numpy(), dv=dv.numpy(), dbias=db.numpy())


def lnlinear_small():
    inp = workloads.lnlinear_inputs((3, 37), 64, 48, dtype=torch.float32, seed=5)
    b = torch.linspace(-1, 1, 48)
    out = ol.layernorm_linear_forward(inp["x"], inp["gamma"], inp["beta"], inp["W"], b, dtype=f64)
    dx, dW, db, dg, dbt = ol.layernorm_linear_backward(inp["dY"], inp["x"], inp["gamma"], inp["beta"], inp["W"], dtype=f64)
    np.savez_compressed(os.path.join(HERE, "lnlinear_small.npz"), out=out.numpy(), dx=dx.numpy(), dW=dW.numpy(),
                        db=db.numpy(), dgamma=dg.numpy(), dbeta=dbt.numpy(), b=b.numpy())


def transition_small():
    inp = workloads.transition_inputs((2, 29), 32, 4, dtype=torch.float32, seed=7)
    h = ot.ln_swiglu_forward(inp["x"], inp["gamma"], inp["beta"], inp["W1"], dtype=f64)
    y = ot.transition_forward(inp["x"], inp["gamma"], inp["beta"], inp["W1"], inp["W2"], dtype=f64)
    np.savez_compressed(os.path.join(HERE, "transition_small.npz"), h=h.numpy(), y=y.numpy())


def triangle_blocks_small():
    """fwd+bwd of the two pair-stack blocks on small ragged shapes, fp32 inputs, both variants each."""
    out = {}
    for node in ("starting", "ending"):
        w = workloads.triangle_attention_inputs(seed=11)
        o, dx, dp = ota.triangle_attention_forward_backward(w["x"], w["mask"], w["params"], w["dout"], 2, 16, node)
        out["attn_%s_out" % node], out["attn_%s_dx" % node] = o.numpy(), dx.numpy()
        out["attn_%s_dWkv" % node] = dp["fn.attn.to_kv.weight"].numpy()
        out["attn_%s_dWb" % node] = dp["fn.to_attn_bias.0.weight"].numpy()
    for mix in ("outgoing", "incoming"):
        w = workloads.triangle_multiplication_inputs(seed=13)
        o, dx, dp = otm.triangle_multiplication_forward_backward(w["x"], w["mask"], w["params"], w["dout"], mix)
        out["mult_%s_out" % mix], out["mult_%s_dx" % mix] = o.numpy(), dx.numpy()
        out["mult_%s_dW1" % mix] = dp["combined.linear_weight"].numpy()
    np.savez_compressed(os.path.join(HERE, "triangle_blocks_small.npz"), **{k: v.astype(np.float32) for k, v in out.items()})


if __name__ == "__main__":
    triangle_blocks_small()
    attention_c1()
    attention_small_bwd()
    lnlinear_small()
    transition_small()
    for f in sorted(os.listdir(HERE)):
        if f.endswith(".npz"):
            print(f, os.path.getsize(os.path.join(HERE, f)), "bytes")
