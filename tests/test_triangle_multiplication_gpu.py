"""GPU parity of the fused triangle-multiplication block against the CPU oracle (output, input gradient and
every parameter gradient; both mixes, with and without mask, ragged n) and of the layout kernels against
plain tensor expressions.  16-bit runs against the float64 oracle on the same rounded inputs at
rtol = atol = 2e-2, fp32 at 1e-4 / 1e-5, both relative to each tensor's scale."""
import pytest
import torch
import torch.nn.functional as F

from conftest import param_grad_tol, stream_tol, tol_for
from megafold_amd.model.FusedTriangleMultiplication import (TriangleMultiplication, channels_first_to_last,
                                                            channels_last_to_first, trimul_pack_backward,
                                                            trimul_pack_forward)
from oracle import triangle_multiplication as otm

pytestmark = pytest.mark.gpu


def pair_mask(mask):
    return (mask[:, :, None] & mask[:, None, :]).unsqueeze(-1)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("b,n,dh,incoming,masked", [(1, 24, 128, False, 3), (2, 13, 64, True, 2), (1, 40, 64, True, 0)])
def test_pack_kernels(dtype, b, n, dh, incoming, masked):
    """mf_trimul_pack_fwd / _bwd: GLU + pair mask + move to channel-first operands, and its backward."""
    g = torch.Generator().manual_seed(n)
    ld = 5 * dh
    Y = torch.randn(b * n * n, ld, generator=g).to(dtype)
    mask = None
    if masked:
        mask = torch.ones(b, n, dtype=torch.bool)
        mask[:, n - masked:] = False
    y64 = Y.double().view(b, n, n, ld).requires_grad_(True)
    lr = F.glu(y64[..., :4 * dh], dim=-1)
    if mask is not None:
        lr = lr * pair_mask(mask)
    left, right = lr[..., :dh], lr[..., dh:]
    if incoming:      # P0[c][i][k] = right[k, i, c], P1[c][j][k] = left[k, j, c]
        want0, want1 = right.permute(0, 3, 2, 1), left.permute(0, 3, 2, 1)
    else:             # P0[c][i][k] = left[i, k, c],  P1[c][j][k] = right[j, k, c]
        want0, want1 = left.permute(0, 3, 1, 2), right.permute(0, 3, 1, 2)
    Yg = Y.cuda()
    P = trimul_pack_forward(Yg, mask.cuda() if mask is not None else None, b, n, dh, incoming)
    npad = P.shape[-1]
    assert npad % 8 == 0 and P.shape == (2, b * dh, npad, npad)
    tol = tol_for(dtype)
    got = P.cpu().double().view(2, b, dh, npad, npad)
    torch.testing.assert_close(got[0][..., :n, :n], want0.detach(), **tol)
    torch.testing.assert_close(got[1][..., :n, :n], want1.detach(), **tol)
    assert torch.all(got[..., n:] == 0) and torch.all(got[..., n:, :] == 0)      # padding is zero

    dP = torch.randn(2, b, dh, npad, npad, generator=g).to(dtype)
    loss = (want0 * dP[0][..., :n, :n].double()).sum() + (want1 * dP[1][..., :n, :n].double()).sum()
    (dy64,) = torch.autograd.grad(loss, y64)
    dY = torch.full((b * n * n, ld), 5.0, dtype=dtype, device="cuda")
    trimul_pack_backward(dP.cuda().view(2, b * dh, npad, npad), Yg, mask.cuda() if mask is not None else None, dY, b, n, dh, incoming)
    torch.testing.assert_close(dY[:, :4 * dh].cpu().double(), dy64.reshape(b * n * n, ld)[:, :4 * dh], **tol)
    assert torch.all(dY[:, 4 * dh:] == 5.0)                                     # other columns untouched


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("b,n,dh", [(1, 24, 128), (2, 13, 64), (1, 70, 128)])
def test_channel_layout_kernels_round_trip(dtype, b, n, dh):
    g = torch.Generator().manual_seed(n + dh)
    X = torch.randn(b * n * n, dh, generator=g).to(dtype).cuda()
    Pc = channels_last_to_first(X, b, n, dh)
    npad = Pc.shape[-1]
    want = X.view(b, n, n, dh).permute(0, 3, 1, 2)
    torch.testing.assert_close(Pc.view(b, dh, npad, npad)[..., :n, :n], want, rtol=0, atol=0)
    assert torch.all(Pc.view(b, dh, npad, npad)[..., n:] == 0)
    back = channels_first_to_last(Pc, b, n, dh)
    torch.testing.assert_close(back, X, rtol=0, atol=0)


def build(dim, mix, dtype, seed):
    m = TriangleMultiplication(dim=dim, mix=mix)
    g = torch.Generator().manual_seed(seed)
    with torch.no_grad():
        for name, p in m.named_parameters():
            if name.endswith("WEIGHT"):
                p.copy_(1 + 0.1 * torch.randn(p.shape, generator=g))
            elif name.endswith("BIAS") or name.endswith("linear_bias"):
                p.copy_(0.1 * torch.randn(p.shape, generator=g))
            else:
                p.copy_(torch.randn(p.shape, generator=g) * p.shape[0] ** -0.5)
    return m.to(dtype)


CASES = [
    # b, n, dim, masked, mix, dtype
    (1, 48, 128, 5, "outgoing", torch.bfloat16),
    (1, 48, 128, 5, "incoming", torch.bfloat16),
    (2, 37, 128, 0, "incoming", torch.bfloat16),       # ragged n (padded to 40), no mask, batch of two
    (1, 29, 64, 4, "outgoing", torch.float16),
    (1, 40, 128, 3, "incoming", torch.float32),
    (1, 21, 64, 2, "outgoing", torch.float32),
    (1, 26, 32, 3, "outgoing", torch.bfloat16),        # widths the layout kernels do not take: the composed path
    (2, 19, 96, 0, "incoming", torch.float32),
]


@pytest.mark.parametrize("b,n,dim,masked,mix,dtype", CASES)
def test_block_parity(b, n, dim, masked, mix, dtype):
    print("case", b, n, dim, masked, mix, dtype, flush=True)
    m = build(dim, mix, dtype, seed=n)
    g = torch.Generator().manual_seed(100 + n)
    x = torch.randn(b, n, n, dim, generator=g).to(dtype)
    dout = torch.randn(b, n, n, dim, generator=g).to(dtype)
    mask = None
    if masked:
        mask = torch.ones(b, n, dtype=torch.bool)
        mask[:, n - masked:] = False
        mask[0, 1] = False
    params = {k: v.detach().clone() for k, v in m.state_dict().items()}
    want_out, want_dx, want_dp = otm.triangle_multiplication_forward_backward(x, mask, params, dout, mix)

    m = m.cuda()
    xg = x.cuda().requires_grad_(True)
    out = m(xg, mask.cuda() if mask is not None else None)
    out.backward(dout.cuda())
    tol = tol_for(dtype)

    def close(name, got, want, t):
        assert not torch.isnan(got).any(), name
        torch.testing.assert_close(got.detach().cpu().double(), want, msg=lambda msg: "%s: %s" % (name, msg), **t)

    close("out", out, want_out, tol)              # element-wise at the stated bar
    close("dx", xg.grad, want_dx, stream_tol(dtype, want_dx))   # gradient of a length-n contraction
    ptol = param_grad_tol(dtype, b * n * n)       # sums over b*n*n rows
    for name, p in m.named_parameters():
        close(name, p.grad, want_dp[name], ptol)


@pytest.mark.parametrize("mix", ["outgoing", "incoming"])
def test_block_parity_at_the_benchmarked_size(mix):
    """[1, 384, 384, 128] bf16 with the last 38 positions masked (the timed shape): output, input gradient and
    all parameter gradients against the oracle evaluated in fp32 on the CPU, plus bitwise reproducibility."""
    print("full size", mix, flush=True)
    b, n, dim, dtype = 1, 384, 128, torch.bfloat16
    m = build(dim, mix, dtype, seed=5)
    g = torch.Generator().manual_seed(9)
    x = torch.randn(b, n, n, dim, generator=g).to(dtype)
    dout = torch.randn(b, n, n, dim, generator=g).to(dtype)
    mask = torch.ones(b, n, dtype=torch.bool)
    mask[:, n - 38:] = False
    params = {k: v.detach().clone() for k, v in m.state_dict().items()}
    torch.set_num_threads(16)
    want_out, want_dx, want_dp = otm.triangle_multiplication_forward_backward(x, mask, params, dout, mix, dtype=torch.float32)
    m = m.cuda()
    runs = []
    for _ in range(2):
        xg = x.cuda().requires_grad_(True)
        for p in m.parameters():
            p.grad = None
        out = m(xg, mask.cuda())
        out.backward(dout.cuda())
        runs.append([out.detach(), xg.grad] + [p.grad.clone() for p in m.parameters()])
    assert all(torch.equal(a_, b_) for a_, b_ in zip(*runs))
    # The contraction sums 346 products of 16-bit-rounded factors per output, which the block then
    # normalises: element-wise bars as everywhere, parameter gradients with the sqrt(rows) rule.
    tol, ptol = tol_for(dtype), param_grad_tol(dtype, b * n * n)
    torch.testing.assert_close(runs[0][0].cpu().float(), want_out, msg=lambda s_: "out: " + s_, **tol)
    torch.testing.assert_close(runs[0][1].cpu().float(), want_dx, msg=lambda s_: "dx: " + s_, **stream_tol(dtype, want_dx))
    for (name, p), got in zip(m.named_parameters(), runs[0][2:]):
        torch.testing.assert_close(got.cpu().float(), want_dp[name], msg=lambda s_, n_=name: n_ + ": " + s_,
                                   **param_grad_tol(dtype, b * n * n, want_dp[name]))


def test_block_under_autocast_with_fp32_master_weights():
    m = TriangleMultiplication(dim=128, mix="outgoing", dropout=0.25, dropout_type="row").cuda().eval()
    x = torch.randn(1, 32, 32, 128, device="cuda", requires_grad=True)
    with torch.autocast("cuda", dtype=torch.bfloat16):
        out = m(x)
    assert out.dtype == torch.bfloat16 and out.shape == x.shape
    out.float().square().mean().backward()
    assert x.grad.dtype == torch.float32 and torch.isfinite(x.grad).all()
    assert all(p.grad is not None and p.grad.dtype == torch.float32 and torch.isfinite(p.grad).all() for p in m.parameters())
    want = otm.triangle_multiplication_forward(x.detach().cpu(), None, {k: v.cpu() for k, v in m.state_dict().items()}, "outgoing")
    torch.testing.assert_close(out.detach().cpu().double(), want, rtol=2e-2, atol=2e-2)


@pytest.mark.parametrize("mix", ["outgoing", "incoming"])
def test_block_against_golden_fixture(mix):
    """fp32 run against the frozen oracle outputs (tests/golden/triangle_blocks_small.npz)."""
    import os
    import numpy as np
    from megafold_amd import workloads
    g = np.load(os.path.join(os.path.dirname(__file__), "golden", "triangle_blocks_small.npz"))
    w = workloads.triangle_multiplication_inputs(seed=13)
    m = TriangleMultiplication(dim=64, mix=mix)
    m.load_state_dict(w["params"])
    m = m.cuda()
    x = w["x"].cuda().requires_grad_(True)
    out = m(x, w["mask"].cuda())
    out.backward(w["dout"].cuda())
    got = {"out": out, "dx": x.grad, "dW1": m.combined.linear_weight.grad}
    for name, t in got.items():
        want = torch.from_numpy(g["mult_%s_%s" % (mix, name)])
        # out, dx element-wise at the fp32 bar; the weight gradients are sums over 144 rows
        atol = 1e-5 if name in ("out", "dx") else 1e-5 * 12
        torch.testing.assert_close(t.detach().cpu(), want, rtol=1e-4, atol=atol, msg=lambda m_, n=name: "%s: %s" % (n, m_))

