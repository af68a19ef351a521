"""GPU parity of the fused MSAPairWeightedAveraging and OuterProductMean modules against their CPU oracles:
output, input gradients and every parameter gradient, with and without masks.  16-bit runs are compared with
the float64 oracle on the same (rounded) inputs at rtol = atol = 2e-2; fp32 runs at 1e-4 / 1e-5 relative to
the size of each tensor."""
import pytest
import torch

from conftest import param_grad_tol, tol_for
from megafold_amd.model.FusedMSAOps import MSAPairWeightedAveraging, OuterProductMean
from oracle import msa_ops as om

pytestmark = pytest.mark.gpu


def randomise(m, dtype, seed):
    g = torch.Generator().manual_seed(seed)
    with torch.no_grad():
        for name, p in m.named_parameters():
            if name.endswith("WEIGHT"):
                p.copy_(1 + 0.1 * torch.randn(p.shape, generator=g))
            elif name.endswith(("bias", "BIAS")):
                p.copy_(0.1 * torch.randn(p.shape, generator=g))
            elif name.endswith("linear_weight"):
                p.copy_(torch.randn(p.shape, generator=g) * p.shape[0] ** -0.5)      # stored [K, N]
            else:
                p.copy_(torch.randn(p.shape, generator=g) * p.shape[1] ** -0.5)
    return m.to(dtype)


def close(name, got, want, t):
    assert not torch.isnan(got).any(), name
    torch.testing.assert_close(got.detach().cpu().to(want.dtype), want, msg=lambda msg: "%s: %s" % (name, msg), **t)


def key_mask(b, n, masked):
    if not masked:
        return None
    mask = torch.ones(b, n, dtype=torch.bool)
    mask[:, n - masked:] = False
    mask[0, 1] = False
    return mask


def run_pwa(b, s, n, dm, dp, heads, dh, masked, dtype, oracle_dtype=torch.float64):
    m = randomise(MSAPairWeightedAveraging(dim_msa=dm, dim_pairwise=dp, dim_head=dh, heads=heads), dtype, seed=n)
    g = torch.Generator().manual_seed(200 + n)
    msa = torch.randn(b, s, n, dm, generator=g).to(dtype)
    pairwise = torch.randn(b, n, n, dp, generator=g).to(dtype)
    dout = torch.randn(b, s, n, dm, generator=g).to(dtype)
    mask = key_mask(b, n, masked)
    params = {k: v.detach().clone() for k, v in m.state_dict().items()}
    want = om.msa_pair_weighted_averaging_forward_backward(msa, pairwise, params, dout, heads, dh, mask, dtype=oracle_dtype)
    m = m.cuda()
    mg, zg = msa.cuda().requires_grad_(True), pairwise.cuda().requires_grad_(True)
    out = m(msa=mg, pairwise_repr=zg, mask=mask.cuda() if masked else None)
    out.backward(dout.cuda())
    return m, (out.detach(), mg.grad, zg.grad), want


PWA_CASES = [
    # b, s, n, dm, dp, heads, dh, masked, dtype
    (1, 12, 48, 64, 128, 8, 32, 5, torch.bfloat16),          # the MSA module's shapes
    (2, 5, 37, 64, 128, 8, 32, 0, torch.bfloat16),           # ragged tiles, no mask, batch of two
    (1, 7, 77, 32, 64, 2, 16, 9, torch.float16),
    (1, 6, 40, 64, 128, 4, 32, 3, torch.float32),
    (1, 9, 200, 64, 128, 8, 32, 11, torch.bfloat16),         # 14 key tiles of 16: the middle instantiation of the kernel
    (1, 6, 70, 64, 128, 8, 32, 4, torch.float16),            # the dedicated kernels in fp16
]


@pytest.mark.parametrize("b,s,n,dm,dp,heads,dh,masked,dtype", PWA_CASES)
def test_pair_weighted_averaging_parity(b, s, n, dm, dp, heads, dh, masked, dtype):
    print("pwa case", b, s, n, dm, dp, heads, dh, masked, dtype, flush=True)
    m, (out, dmsa, dpair), (want_out, want_dm, want_dz, want_dp) = run_pwa(b, s, n, dm, dp, heads, dh, masked, dtype)
    tol = tol_for(dtype)
    close("out", out, want_out, tol)
    close("dmsa", dmsa, want_dm, tol)
    close("dpairwise", dpair, want_dz, tol)
    for name, p in m.named_parameters():
        rows = b * n * n if name.startswith("pairwise_repr_to_attn") else b * s * n
        close(name, p.grad, want_dp[name], param_grad_tol(dtype, rows, want_dp[name]))


def test_pair_weighted_averaging_at_the_msa_module_size():
    """[1, 128, 384, 64] MSA and [1, 384, 384, 128] pair representation in bf16, 8 heads of 32, last 38 positions
    masked, against the oracle in fp32 on the CPU."""
    b, s, n, dm, dp, heads, dh, dtype = 1, 128, 384, 64, 128, 8, 32, torch.bfloat16
    torch.set_num_threads(16)
    m, (out, dmsa, dpair), (want_out, want_dm, want_dz, want_dp) = run_pwa(b, s, n, dm, dp, heads, dh, 38, dtype,
                                                                          oracle_dtype=torch.float32)
    tol = tol_for(dtype)
    close("out", out, want_out, tol)
    close("dmsa", dmsa, want_dm, tol)
    close("dpairwise", dpair, want_dz, tol)
    for name, p in m.named_parameters():
        rows = b * n * n if name.startswith("pairwise_repr_to_attn") else b * s * n
        close(name, p.grad, want_dp[name], param_grad_tol(dtype, rows, want_dp[name]))


OPM_CASES = [
    # b, s, n, dm, dh, dp, pair mask, msa mask, dtype
    (1, 12, 48, 64, 32, 128, True, True, torch.bfloat16),    # the MSA module's shapes
    (2, 5, 37, 64, 32, 128, False, False, torch.bfloat16),
    (1, 7, 33, 32, 8, 64, True, False, torch.float16),
    (1, 6, 40, 64, 16, 128, True, True, torch.float32),
    (1, 9, 52, 64, 32, 128, True, True, torch.float16),      # the fused kernels in fp16
    (2, 20, 26, 64, 32, 128, True, False, torch.bfloat16),   # ragged position tiles in both directions, batch of two
]


@pytest.mark.parametrize("b,s,n,dm,dh,dp,use_mask,use_msa_mask,dtype", OPM_CASES)
def test_outer_product_mean_parity(b, s, n, dm, dh, dp, use_mask, use_msa_mask, dtype):
    print("opm case", b, s, n, dm, dh, dp, use_mask, use_msa_mask, dtype, flush=True)
    m = randomise(OuterProductMean(dim_msa=dm, dim_pairwise=dp, dim_hidden=dh), dtype, seed=n)
    g = torch.Generator().manual_seed(300 + n)
    msa = torch.randn(b, s, n, dm, generator=g).to(dtype)
    dout = torch.randn(b, n, n, dp, generator=g).to(dtype)
    mask = key_mask(b, n, 4) if use_mask else None
    msa_mask = None
    if use_msa_mask:
        msa_mask = torch.ones(b, s, dtype=torch.bool)
        msa_mask[:, s - 2:] = False
        msa_mask[0, 0] = False
    params = {k: v.detach().clone() for k, v in m.state_dict().items()}
    want_out, want_dm, want_dp = om.outer_product_mean_forward_backward(msa, params, dout, mask, msa_mask)
    m = m.cuda()
    mg = msa.cuda().requires_grad_(True)
    out = m(mg, mask=mask.cuda() if use_mask else None, msa_mask=msa_mask.cuda() if use_msa_mask else None)
    out.backward(dout.cuda())
    tol = tol_for(dtype)
    close("out", out, want_out, tol)
    close("dmsa", mg.grad, want_dm, param_grad_tol(dtype, n, want_dm))       # each element sums over n partner positions
    for name, p in m.named_parameters():
        rows = b * n * n if name.startswith("to_pairwise_repr") else b * s * n
        close(name, p.grad, want_dp[name], param_grad_tol(dtype, rows, want_dp[name]))


def test_outer_product_mean_at_the_msa_module_size():
    """[1, 128, 384, 64] MSA in bf16, hidden 32, last 38 positions and three MSA rows masked, against the oracle in fp32
    on the CPU; 125 kept rows (not a power of two), so a doubly rounded 1 / rows would show in the relative RMS error."""
    from conftest import rel_rms
    b, s, n, dm, dh, dp, dtype = 1, 128, 384, 64, 32, 128, torch.bfloat16
    torch.set_num_threads(16)
    m = randomise(OuterProductMean(dim_msa=dm, dim_pairwise=dp, dim_hidden=dh), dtype, seed=n)
    g = torch.Generator().manual_seed(300 + n)
    msa = torch.randn(b, s, n, dm, generator=g).to(dtype)
    dout = torch.randn(b, n, n, dp, generator=g).to(dtype)
    mask = key_mask(b, n, 38)
    msa_mask = torch.ones(b, s, dtype=torch.bool)
    msa_mask[:, s - 2:] = False
    msa_mask[0, 0] = False
    params = {k: v.detach().clone() for k, v in m.state_dict().items()}
    want_out, want_dm, want_dp = om.outer_product_mean_forward_backward(msa, params, dout, mask, msa_mask, dtype=torch.float32)
    m = m.cuda()
    mg = msa.cuda().requires_grad_(True)
    dmask, dmsa_mask = mask.cuda(), msa_mask.cuda()
    torch.cuda.synchronize()
    torch.cuda.reset_peak_memory_stats()
    base = torch.cuda.memory_allocated()
    out = m(mg, mask=dmask, msa_mask=dmsa_mask)
    torch.cuda.synchronize()
    # the forward never holds the [n, n, dh * dh] outer product (288 MiB here), neither while it runs nor for the
    # backward: its peak is the output (36 MiB), the projected MSA and the two operand matrices
    fwd_peak_mib = (torch.cuda.max_memory_allocated() - base) / 2 ** 20
    held_mib = (torch.cuda.memory_allocated() - base) / 2 ** 20
    print("outer product mean forward: peak %.0f MiB, held for backward %.0f MiB" % (fwd_peak_mib, held_mib), flush=True)
    assert fwd_peak_mib < 100 and held_mib < 80
    dd = dout.cuda()
    torch.cuda.synchronize()
    torch.cuda.reset_peak_memory_stats()
    base_b = torch.cuda.memory_allocated()
    out.backward(dd)
    torch.cuda.synchronize()
    # nor does the backward: its three kernels form the outer blocks and their gradient tile by tile (the two-GEMM form
    # held two 288 MiB tensors at its peak)
    bwd_peak_mib = (torch.cuda.max_memory_allocated() - base_b) / 2 ** 20
    print("outer product mean backward: peak %.0f MiB above what the forward left" % bwd_peak_mib, flush=True)
    assert bwd_peak_mib < 120
    close("out", out, want_out, tol_for(dtype))
    assert rel_rms(out, want_out) < 4e-3
    close("dmsa", mg.grad, want_dm, param_grad_tol(dtype, n, want_dm))
    assert rel_rms(mg.grad, want_dm) < 1e-2
    for name, p in m.named_parameters():
        rows = b * n * n if name.startswith("to_pairwise_repr") else b * s * n
        close(name, p.grad, want_dp[name], param_grad_tol(dtype, rows, want_dp[name]))


def test_msa_modules_under_autocast_with_fp32_master_weights():
    """fp32 parameters and inputs under bf16 autocast: bf16 outputs, fp32 gradients for inputs and parameters, values within
    the 16-bit bar of the oracle; dropout of the averaging module zeroes whole rows in training mode only."""
    b, s, n = 1, 6, 40
    g = torch.Generator().manual_seed(11)
    msa = torch.randn(b, s, n, 64, generator=g).cuda().requires_grad_()
    pair = torch.randn(b, n, n, 128, generator=g).cuda().requires_grad_()
    mask = key_mask(b, n, 4).cuda()
    pwa = randomise(MSAPairWeightedAveraging(dim_msa=64, dim_pairwise=128, dim_head=32, heads=8), torch.float32, 1).cuda()
    opm = randomise(OuterProductMean(dim_msa=64, dim_pairwise=128, dim_hidden=32), torch.float32, 2).cuda()
    with torch.autocast("cuda", dtype=torch.bfloat16):
        y1 = pwa(msa=msa, pairwise_repr=pair, mask=mask)
        y2 = opm(msa, mask=mask)
    assert y1.dtype == torch.bfloat16 and y2.dtype == torch.bfloat16
    (y1.float().square().mean() + y2.float().square().mean()).backward()
    assert msa.grad.dtype == torch.float32 and pair.grad.dtype == torch.float32
    for m in (pwa, opm):
        assert all(p.grad is not None and p.grad.dtype == torch.float32 and torch.isfinite(p.grad).all() for p in m.parameters())
    cpu = lambda m: {k: v.detach().cpu() for k, v in m.state_dict().items()}
    want1 = om.msa_pair_weighted_averaging_forward(msa.detach().cpu(), pair.detach().cpu(), cpu(pwa), 8, 32, mask.cpu())
    want2 = om.outer_product_mean_forward(msa.detach().cpu(), cpu(opm), mask.cpu(), None)
    torch.testing.assert_close(y1.detach().cpu().double(), want1, rtol=2e-2, atol=2e-2)
    torch.testing.assert_close(y2.detach().cpu().double(), want2, rtol=2e-2, atol=2e-2)
    drop = MSAPairWeightedAveraging(dim_msa=64, dim_pairwise=128, dim_head=32, heads=8, dropout=0.5, dropout_type="row").cuda().to(torch.bfloat16)
    x16, z16 = msa.detach().to(torch.bfloat16), pair.detach().to(torch.bfloat16)
    drop.train()
    yd = drop(msa=x16, pairwise_repr=z16, mask=mask)
    dropped = (yd == 0).all(dim=1)                 # "row" dropout zeroes whole [b, :, col, channel] lines
    assert dropped.any() and not dropped.all()
    drop.eval()
    assert not (drop(msa=x16, pairwise_repr=z16, mask=mask) == 0).all(dim=1).any()


@pytest.mark.gpu
@pytest.mark.parametrize("A,B,C,E,dtype", [(3, 32, 40, 32, torch.bfloat16), (2, 5, 7, 8, torch.float16),
                                           (1, 70, 33, 4, torch.float32), (4, 40, 32, 128, torch.bfloat16),
                                           (2, 33, 50, 24, torch.bfloat16), (2, 16, 16, 3, torch.float32)])
def test_permute_0213_matches_torch(A, B, C, E, dtype):
    """The layout move of the outer product and its inverse (the autograd backward) against torch.permute, bit for
    bit: whole tiles, ragged tiles, every supported row width, and a row width the kernel does not take (12 bytes:
    the wrapper falls back to PyTorch)."""
    from megafold_amd.model.FusedMSAOps.msa_ops import _Permute0213
    x = torch.randn(A, B, C, E, device="cuda").to(dtype).requires_grad_()
    y = _Permute0213.apply(x)
    assert y.is_contiguous() and torch.equal(y, x.detach().permute(0, 2, 1, 3))
    g = torch.randn(A, C, B, E, device="cuda").to(dtype)
    y.backward(g)
    assert torch.equal(x.grad, g.permute(0, 2, 1, 3))
