"""The allocation-free forward entry point (``mf_evoattn_fwd_noalloc``) against ``mf_evoattn_fwd``, through the
C ABI: same kernels, scratch in the library's fixed device array instead of a caller workspace.  Two calls
in a row, the second on a smaller problem (the array keeps the first call's contents), each compared bit for
bit with the workspace form, plus the size limit and the absence of allocations."""
import ctypes as C

import pytest
import torch

from megafold_amd import _lib, workloads
from megafold_amd.model.FusedEvoAttention import evoattention as ev

pytestmark = pytest.mark.gpu


def _both(shape, dtype, seed):
    B, N, S, H, D, nm = shape
    inp = {k: v.cuda() for k, v in workloads.evoattention_inputs(B, N, S, H, D, nm, dtype=dtype, seed=seed).items()}
    want_o, want_lse, _ = ev.evoattention_forward(inp["q"], inp["k"], inp["v"], inp["mask"], inp["bias"])
    got_o = torch.full_like(want_o, float("nan"))
    got_lse = torch.full_like(want_lse, float("nan"))
    torch.cuda.synchronize()
    # nothing may come from the caching allocator (not even a transient block that is freed again: the running
    # counts of allocations and segments must not move) nor from the driver (free device memory must not move)
    stats = torch.cuda.memory_stats()
    before = (torch.cuda.memory_allocated(), stats["allocation.all.allocated"], stats["segment.all.allocated"])
    free_before = torch.cuda.mem_get_info()[0]
    ev.evoattention_forward_noalloc(inp["q"], inp["k"], inp["v"], inp["mask"], inp["bias"], got_o, got_lse)
    torch.cuda.synchronize()
    stats = torch.cuda.memory_stats()
    assert (torch.cuda.memory_allocated(), stats["allocation.all.allocated"], stats["segment.all.allocated"]) == before
    assert torch.cuda.mem_get_info()[0] == free_before
    return (got_o, got_lse), (want_o, want_lse)


def test_noalloc_matches_workspace_form_twice():
    print("noalloc big then small", flush=True)
    # the entry point's first call on a device is its set-up: the runtime loads the library's device image, which
    # is when the fixed scratch array gets its memory; the calls after it must leave the device's free memory alone
    tiny = {k: v.cuda() for k, v in workloads.evoattention_inputs(1, 1, 32, 1, 8, 0, dtype=torch.bfloat16, seed=1).items()}
    ev.evoattention_forward_noalloc(tiny["q"], tiny["k"], tiny["v"], tiny["mask"], tiny["bias"],
                                    torch.empty_like(tiny["q"]), torch.empty(1, 1, 1, 32, device="cuda"))
    torch.cuda.synchronize()
    for shape, dtype, seed in (((1, 6, 200, 4, 32, 17), torch.bfloat16, 5), ((2, 2, 45, 2, 16, 3), torch.float32, 6)):
        got, want = _both(shape, dtype, seed)
        for g, w in zip(got, want):
            assert torch.equal(g, w)


def test_noalloc_rejects_oversized_problems():
    # B * H * ceil(S / 32)^2 = 16 * 17^2 = 4624 tiles of 4 KiB > 16 MiB: rejected before any launch
    B, N, S, H, D = 1, 1, 544, 16, 8
    q = torch.zeros(B, N, S, H, D, dtype=torch.bfloat16, device="cuda")
    bias = torch.zeros(B, 1, H, S, S, dtype=torch.bfloat16, device="cuda")
    mask = torch.zeros(B, N, 1, 1, S, device="cuda")
    o = torch.empty_like(q)
    lse = torch.empty(B, N, H, S, device="cuda")
    with pytest.raises(RuntimeError, match="scratch bytes"):
        ev.evoattention_forward_noalloc(q, q, q, mask, bias, o, lse)
    # the workspace form takes the same problem
    ev.evoattention_forward(q, q, q, mask, bias)
    torch.cuda.synchronize()
