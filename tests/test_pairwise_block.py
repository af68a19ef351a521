"""PairwiseBlock assembled from the fused blocks: parameter names against the reference's state-dict keys
(CPU), and parity of output, input gradient and every parameter gradient against the composed oracle (GPU)."""
import pytest
import torch

from megafold_amd.model.PairwiseBlock import PairwiseBlock
from oracle import pairwise_block as opb

# state-dict keys of PairwiseBlock() in the reference (megafold/model/megafold.py:659-723 with the sub-modules'
# own parameters: TriangleMultiplication :441-458, PreLayerNorm :318-319, TriangleAttention :609-615, Attention
# attention.py:135-158, FusedTransition FusedTransition/fused_transition.py:128-131)
TM = ["combined.WEIGHT", "combined.BIAS", "combined.linear_weight", "combined.linear_bias",
      "to_out.0.WEIGHT", "to_out.0.BIAS", "to_out.0.linear_weight"]
TA = ["norm.weight", "norm.bias", "fn.to_attn_bias.0.weight", "fn.attn.to_q.weight", "fn.attn.to_q.bias",
      "fn.attn.to_kv.weight", "fn.attn.to_out.weight", "fn.attn.to_gates.weight", "fn.attn.to_gates.bias"]
TR = ["ff.0.WEIGHT", "ff.0.BIAS", "ff.0.linear_weight", "ff.2.weight"]
REFERENCE_KEYS = ({"tri_mult_outgoing." + k for k in TM} | {"tri_mult_incoming." + k for k in TM} |
                  {"tri_attn_starting." + k for k in TA} | {"tri_attn_ending." + k for k in TA} |
                  {"pairwise_transition." + k for k in TR})


def test_parameter_names_match_the_reference():
    m = PairwiseBlock()
    assert set(m.state_dict().keys()) == REFERENCE_KEYS
    assert m.tri_attn_ending.fn.dropout.dropout_type == "col" and m.tri_mult_incoming.to_out[1].dropout_type == "row"


@pytest.mark.gpu
@pytest.mark.parametrize("n,masked,dtype", [(40, 4, torch.bfloat16), (24, 0, torch.float32)])
def test_block_parity(n, masked, dtype):
    from conftest import tol_for
    torch.manual_seed(n)
    m = PairwiseBlock(dropout_row_prob=0.0, dropout_col_prob=0.0)
    g = torch.Generator().manual_seed(n + 1)
    with torch.no_grad():
        for name, p in m.named_parameters():
            if name.endswith(("WEIGHT", "norm.weight")):
                p.copy_(1 + 0.1 * torch.randn(p.shape, generator=g))
            elif p.dim() == 1:
                p.copy_(0.1 * torch.randn(p.shape, generator=g))
            else:
                fan_in = p.shape[0] if name.endswith("linear_weight") else p.shape[1]
                p.copy_(torch.randn(p.shape, generator=g) * fan_in ** -0.5)
    m = m.to(dtype)
    x = torch.randn(1, n, n, 128, generator=g).to(dtype)
    dout = torch.randn(1, n, n, 128, generator=g).to(dtype)
    mask = None
    if masked:
        mask = torch.ones(1, n, dtype=torch.bool)
        mask[:, n - masked:] = False
    params = {k: v.detach().clone() for k, v in m.state_dict().items()}
    want_out, want_dx, want_dp = opb.pairwise_block_forward_backward(x, mask, params, dout, 4, 32)

    m = m.cuda()
    xg = x.cuda().requires_grad_(True)
    out = m(pairwise_repr=xg, mask=mask.cuda() if mask is not None else None)
    out.backward(dout.cuda())
    from conftest import rel_rms, stream_tol
    tol = tol_for(dtype)

    def close(name, got, want, t):
        assert not torch.isnan(got).any(), name
        torch.testing.assert_close(got.detach().cpu().double(), want, msg=lambda msg: "%s: %s" % (name, msg), **t)

    # element-wise; five blocks on a 16-bit residual stream, each of which rounds its own result and the sum with
    # the stream: ten roundings of stream-sized values on the way of either tensor.  (With the bar at four roundings
    # the test passed or failed with the summation order inside one kernel: one or two elements of 204800 at
    # 0.08 - 0.09 against 0.075.)  The aggregate (relative RMS) error is held below the element-wise relative bar;
    # measured 0.006 for the output and 0.009 for the input gradient.
    close("out", out, want_out, stream_tol(dtype, want_out, roundings=10))
    close("dx", xg.grad, want_dx, stream_tol(dtype, want_dx, roundings=10))
    rms_bar = 1e-5 if dtype == torch.float32 else 1.5e-2
    assert rel_rms(out, want_out) < rms_bar and rel_rms(xg.grad, want_dx) < rms_bar, \
        (rel_rms(out, want_out), rel_rms(xg.grad, want_dx))
    ptol = dict(tol, atol=stream_tol(dtype, want_dx)["atol"] * max(1.0, float(n * n) ** 0.5))   # sums over n*n rows
    for name, p in m.named_parameters():
        close(name, p.grad, want_dp[name], ptol)


@pytest.mark.gpu
@pytest.mark.parametrize("kind", ["tri_mult_outgoing", "tri_mult_incoming", "tri_attn_starting", "tri_attn_ending",
                                  "pairwise_transition"])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_add_residual_matches_the_separate_sum(kind, dtype):
    """x + block(x) with the sums folded into the block's kernels (add_residual=True) against the block followed
    by PyTorch's add: output, input gradient and every parameter gradient.  The folded sums round once where the
    separate ones round twice, hence the element-wise bar of the dtype instead of equality."""
    from conftest import tol_for
    n = 40
    g = torch.Generator().manual_seed(11)
    blk = getattr(PairwiseBlock(dropout_row_prob=0.0, dropout_col_prob=0.0), kind).cuda().to(dtype)
    with torch.no_grad():
        for p in blk.parameters():
            p.copy_((torch.randn(p.shape, generator=g) * 0.3).to(dtype))
    x = torch.randn(1, n, n, 128, generator=g).to(dtype).cuda()
    dout = torch.randn(1, n, n, 128, generator=g).to(dtype).cuda()
    mask = torch.ones(1, n, dtype=torch.bool, device="cuda")
    mask[:, n - 3:] = False
    kw = {} if kind == "pairwise_transition" else {"mask": mask}
    got = {}
    for fused in (True, False):
        xg = x.clone().requires_grad_()
        for p in blk.parameters():
            p.grad = None
        y = blk(xg, add_residual=True, **kw) if fused else blk(xg, **kw) + xg
        y.backward(dout)
        got[fused] = [y.detach(), xg.grad] + [p.grad.clone() for p in blk.parameters()]
    t = tol_for(dtype)
    for a, b in zip(got[True][:2], got[False][:2]):
        torch.testing.assert_close(a.float(), b.float(), **t)
    for a, b in zip(got[True][2:], got[False][2:]):                  # parameter gradients do not see the sums
        torch.testing.assert_close(a.float(), b.float(), rtol=t["rtol"], atol=t["atol"] * n)


@pytest.mark.gpu
def test_add_residual_with_active_dropout_falls_back_to_the_separate_sum():
    blk = PairwiseBlock(dropout_row_prob=0.5, dropout_col_prob=0.5).tri_mult_outgoing.cuda().to(torch.bfloat16).train()
    x = torch.randn(1, 24, 24, 128, device="cuda", dtype=torch.bfloat16)
    torch.manual_seed(3)
    a = blk(x, add_residual=True)
    torch.manual_seed(3)
    b = blk(x) + x
    assert torch.equal(a, b)


@pytest.mark.gpu
@pytest.mark.parametrize("kind", ["tri_mult_outgoing", "tri_attn_ending", "pairwise_transition", "block"])
def test_fp32_residual_stream_under_autocast_stays_fp32(kind):
    """bf16 autocast with fp32 parameters and an fp32 pair tensor (the reference's bf16-mixed setup): `x + block(x)`
    promotes to fp32 there (megafold.py:742-747), so add_residual must return fp32 in training and in evaluation
    mode, hand back an fp32 input gradient, and agree with the separate sum bit for bit (it IS the separate sum)."""
    n = 24
    g = torch.Generator().manual_seed(5)
    full = PairwiseBlock(dropout_row_prob=0.0, dropout_col_prob=0.0).cuda()
    blk = full if kind == "block" else getattr(full, kind)
    with torch.no_grad():
        for p in blk.parameters():
            p.copy_(torch.randn(p.shape, generator=g) * 0.3)
    x = torch.randn(1, n, n, 128, generator=g).cuda()
    mask = torch.ones(1, n, dtype=torch.bool, device="cuda")
    mask[:, n - 3:] = False

    def call(xin, fused):
        if kind == "block":
            return blk(pairwise_repr=xin, mask=mask)
        kw = {} if kind == "pairwise_transition" else {"mask": mask}
        return blk(xin, add_residual=True, **kw) if fused else blk(xin, **kw) + xin

    for training in (True, False):
        blk.train(training)
        xg = x.clone().requires_grad_()
        with torch.autocast("cuda", dtype=torch.bfloat16):
            y = call(xg, True)
        assert y.dtype == torch.float32, (kind, training, y.dtype)
        y.float().square().mean().backward()
        assert xg.grad.dtype == torch.float32 and torch.isfinite(xg.grad).all()
        if kind != "block":
            x2 = x.clone().requires_grad_()
            with torch.autocast("cuda", dtype=torch.bfloat16):
                y2 = call(x2, False)
            y2.float().square().mean().backward()
            assert torch.equal(y, y2) and torch.equal(xg.grad, x2.grad)


@pytest.mark.gpu
@pytest.mark.parametrize("kind", ["pairwise_block", "attention_pair_bias", "msa_pair_weighted_averaging",
                                  "outer_product_mean"])
def test_blocks_replay_from_a_captured_graph(kind):
    """Forward and backward of a block captured into HIP graphs (torch.cuda.make_graphed_callables) and replayed:
    the library launches on the stream it is handed and neither allocates, clears memory with a memset node nor
    synchronises, so a capture holds kernels only.  Every replay, with eager work of the same module and
    synchronisations between the replays and with new input values each time, must reproduce the eager output, input
    gradients and parameter gradients bit for bit."""
    from megafold_amd.model.FusedAttentionPairBias import AttentionPairBias
    from megafold_amd.model.FusedMSAOps import MSAPairWeightedAveraging, OuterProductMean
    n, s = 72, 20
    g = torch.Generator().manual_seed(17)
    rnd = lambda *sh: torch.randn(*sh, generator=g).to(torch.bfloat16).cuda()
    mask = torch.ones(1, n, dtype=torch.bool, device="cuda")
    mask[:, n - 5:] = False

    class Wrapped(torch.nn.Module):          # graphed callables take tensors only: the mask rides along as a constant
        def __init__(self, inner, call):
            super().__init__()
            self.inner, self.call = inner, call

        def forward(self, *tensors):
            return self.call(self.inner, *tensors)

    if kind == "pairwise_block":
        mod = Wrapped(PairwiseBlock(dropout_row_prob=0.0, dropout_col_prob=0.0),
                      lambda m, pair: m(pairwise_repr=pair, mask=mask))
        shapes, oshape = [(1, n, n, 128)], (1, n, n, 128)
    elif kind == "attention_pair_bias":
        mod = Wrapped(AttentionPairBias(heads=16, dim_pairwise=128, dim=384, dim_head=64),
                      lambda m, single, pair: m(single, pairwise_repr=pair, mask=mask))
        shapes, oshape = [(1, n, 384), (1, n, n, 128)], (1, n, 384)
    elif kind == "msa_pair_weighted_averaging":
        mod = Wrapped(MSAPairWeightedAveraging(dim_msa=64, dim_pairwise=128, dim_head=32, heads=8),
                      lambda m, msa, pair: m(msa=msa, pairwise_repr=pair, mask=mask))
        shapes, oshape = [(1, s, n, 64), (1, n, n, 128)], (1, s, n, 64)
    else:
        mod = Wrapped(OuterProductMean(dim_msa=64, dim_pairwise=128, dim_hidden=32), lambda m, msa: m(msa, mask=mask))
        shapes, oshape = [(1, s, n, 64)], (1, n, n, 128)
    mod = mod.cuda().to(torch.bfloat16)
    with torch.no_grad():
        for p in mod.parameters():
            p.copy_((torch.randn(p.shape, generator=g) * 0.05).to(p.dtype))

    def fresh():
        return tuple(rnd(*sh).requires_grad_() for sh in shapes)

    def run(fn, args, dout):
        out = fn(*args)
        out.backward(dout)
        res = [out.detach().clone()] + [a.grad.clone() for a in args] + [p.grad.clone() for p in mod.parameters()]
        for t in list(args) + list(mod.parameters()):
            t.grad = None
        return res

    cases = [(fresh(), rnd(*oshape)) for _ in range(3)]
    want = [run(mod, a, d) for a, d in cases]
    graphed = torch.cuda.make_graphed_callables(mod, fresh(), num_warmup_iters=3)
    for rep in range(3):
        for i, (a, d) in enumerate(cases):
            got = run(graphed, a, d)
            torch.cuda.synchronize()
            for j, (x, y) in enumerate(zip(got, want[i])):
                assert torch.equal(x, y), "replay %d, inputs %d, tensor %d differs from the eager result" % (rep, i, j)
        eager = run(mod, *cases[rep])                        # the program's own eager work between the replays
        torch.cuda.synchronize()
        assert all(torch.equal(x, y) for x, y in zip(eager, want[rep]))
