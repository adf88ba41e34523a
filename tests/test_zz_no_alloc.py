"""GPU test of fused_mha_backward_noalloc, the backward entry point that allocates
nothing (its workspace is a static device array inside the library): called through
the C ABI, its gradients must equal fused_mha_backward's bit for bit (same kernels,
no atomics), on two calls in a row, the second with a smaller input, so that
whatever the first call left in the shared array must not matter."""
import math

import pytest
import torch

import abi
from oracle import attention_oracle as ao

pytestmark = pytest.mark.gpu

G_TOL = 1e-2


def _err(got, want):
    return (got.float().cpu() - want.half().float()).abs().max().item()


def test_noalloc_backward_matches_workspace_backward_twice():
    if not torch.cuda.is_available():
        pytest.fail("this test needs a GPU")
    lib = abi.load()
    cases = [(2, 4, 384, 128, True), (1, 3, 100, 128, True)]  # the second is smaller (and ragged)
    for B, H, N, D, causal in cases:
        scale = 1.0 / math.sqrt(D)
        q, k, v, do = ao.make_inputs(B, N, H, D, seed=N + H)
        print(f"noalloc B{B} H{H} N{N} D{D} causal={causal}", flush=True)
        qg, kg, vg, dog = (t.cuda() for t in (q, k, v, do))
        out, lse = abi.forward(lib, qg, kg, vg, scale, causal)
        want = abi.backward(lib, qg, kg, vg, out, dog, lse, scale, causal)[:3]
        grads = tuple(torch.full_like(qg, float("nan")) for _ in range(3))  # allocated before the call
        torch.cuda.synchronize()
        before = torch.cuda.memory_stats()["allocation.all.allocated"]
        got = abi.backward_noalloc(lib, qg, kg, vg, out, dog, lse, scale, causal, grads=grads)
        torch.cuda.synchronize()
        assert torch.cuda.memory_stats()["allocation.all.allocated"] == before  # nothing came from torch's allocator
        for a, b in zip(got, want):
            assert torch.equal(a, b)
        dq_ref, dk_ref, dv_ref = ao.attention_backward(q, k, v, do, scale, causal)
        assert _err(got[0], dq_ref) <= G_TOL and _err(got[1], dk_ref) <= G_TOL and _err(got[2], dv_ref) <= G_TOL
    # beyond the static array: a clear error, nothing launched
    p = qg.data_ptr()
    rc = lib.fused_mha_backward_noalloc(p, p, p, p, p, p, p, p, p, 4, 64, 8192, 8192, 128, 1.0, 1, None)
    assert rc == abi.ERR_SCRATCH_LIMIT
