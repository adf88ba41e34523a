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
        # the same kernels with a caller-supplied workspace of the same (minimum) size
        want = abi.backward(lib, qg, kg, vg, out, dog, lse, scale, causal, min_workspace=True)[:3]
        grads = tuple(torch.full_like(qg, float("nan")) for _ in range(3))  # allocated before the call
        torch.cuda.synchronize()
        before = torch.cuda.memory_stats()["allocation.all.allocated"]
        free_before = torch.cuda.mem_get_info()[0]
        got = abi.backward_noalloc(lib, qg, kg, vg, out, dog, lse, scale, causal, grads=grads)
        torch.cuda.synchronize()
        assert torch.cuda.memory_stats()["allocation.all.allocated"] == before  # nothing came from torch's allocator
        # and nothing from the HIP runtime behind its back: the device's free memory is what it was (the code
        # object is loaded already, abi.backward above ran the same kernels)
        assert torch.cuda.mem_get_info()[0] == free_before
        for a, b in zip(got, want):
            assert torch.equal(a, b)
        dq_ref, dk_ref, dv_ref = ao.attention_backward(q, k, v, do, scale, causal)
        assert _err(got[0], dq_ref) <= G_TOL and _err(got[1], dk_ref) <= G_TOL and _err(got[2], dv_ref) <= G_TOL
    # beyond the static array: a clear error, nothing launched
    p = qg.data_ptr()
    rc = lib.fused_mha_backward_noalloc(p, p, p, p, p, p, p, p, p, 4, 64, 8192, 8192, 128, 1.0, 1, None)
    assert rc == abi.ERR_SCRATCH_LIMIT


def test_noalloc_backward_under_graph_capture():
    """What the entry point is for: after one warm call outside capture (the first call on a device looks up the
    address of the static array), fused_mha_backward_noalloc can be captured into a HIP graph; every replay,
    with eager work between the replays, gives the eager result bit for bit."""
    if not torch.cuda.is_available():
        pytest.fail("this test needs a GPU")
    lib = abi.load()
    B, H, N, D, causal = 2, 4, 200, 64, True
    scale = 1.0 / math.sqrt(D)
    static = [torch.zeros(B, N, H, D, dtype=torch.float16, device="cuda") for _ in range(5)]
    sq, sk, sv, sdo, sout = static
    slse = torch.zeros(B, H, N, dtype=torch.float32, device="cuda")
    grads = tuple(torch.zeros_like(sq) for _ in range(3))

    def fill(seed):
        q, k, v, do = ao.make_inputs(B, N, H, D, seed=seed)
        for dst, src in zip((sq, sk, sv, sdo), (q, k, v, do)):
            dst.copy_(src.cuda())
        out, lse = abi.forward(lib, sq, sk, sv, scale, causal)
        sout.copy_(out)
        slse.copy_(lse)
        return q, k, v, do

    fill(1)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):  # the warm call, on a side stream as graph capture asks for
        abi.backward_noalloc(lib, sq, sk, sv, sout, sdo, slse, scale, causal, grads=grads)
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        abi.backward_noalloc(lib, sq, sk, sv, sout, sdo, slse, scale, causal, grads=grads)
    for seed in (2, 3, 4):
        q, k, v, do = fill(seed)
        for g in grads:
            g.fill_(float("nan"))
        graph.replay()
        torch.cuda.synchronize()
        replayed = [g.clone() for g in grads]
        eager = abi.backward(lib, sq, sk, sv, sout, sdo, slse, scale, causal, min_workspace=True)[:3]
        torch.cuda.synchronize()
        for a, b in zip(replayed, eager):
            assert torch.equal(a, b), f"replay with seed {seed} differs from the eager result"
        dq_ref = ao.attention_backward(q, k, v, do, scale, causal)[0]
        assert _err(replayed[0], dq_ref) <= G_TOL
