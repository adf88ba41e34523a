"""GPU parity tests: the HIP kernels, called through the Python API
(flash_attn_func -> extension -> C ABI) and through the C ABI directly (ctypes),
against the fp32 CPU oracle on the same seeded inputs.

Tolerances (max-abs, after rounding the oracle to fp16): O 2e-3, dQ/dK/dV 1e-2.
The reference's own check is allclose(atol=1e-2, rtol=0) on all four
(test.py:42-45)."""
import math

import pytest
import torch

import abi
from oracle import attention_oracle as ao

pytestmark = pytest.mark.gpu

O_TOL = 2e-3
G_TOL = 1e-2
LSE_TOL = 2e-3

CONFIGS = {  # name: B, H, N, D, causal, scale (None = D**-0.5), zero-dout tail rows, heads checked against the oracle
    "plumbing": (1, 4, 128, 64, False, None, 0, range(4)),
    "bert_base": (16, 12, 512, 64, False, None, 0, range(12)),
    "gpt_causal": (4, 16, 1024, 64, True, None, 0, range(16)),
    "llama7b_headline": (2, 32, 4096, 128, True, None, 0, range(32)),
    # one head costs the oracle a 1 GiB score matrix several times over: three heads, spread over the XCDs
    "long_context": (1, 16, 16384, 128, True, None, 32, (0, 7, 15)),
    # the reference's own test case (test.py:4-9): 80 slices, 10 per XCD
    "reference_test_py": (2, 40, 2048, 128, True, 0.1, 0, range(40)),
    # slice counts that are no multiple of the 8 XCDs
    "twelve_slices": (1, 12, 2048, 128, True, None, 0, range(12)),
    "twenty_slices_d64": (1, 20, 1536, 64, False, None, 0, range(20)),
    # a ragged length with a slice count that is a multiple of 8
    "ragged_sixteen_slices": (2, 8, 1000, 128, True, None, 0, range(8)),
}


@pytest.fixture(scope="module")
def lib():
    if not torch.cuda.is_available():
        pytest.fail("these tests need a GPU")
    return abi.load()


def _err(got, want):
    return (got.float().cpu() - want.half().float()).abs().max().item()


@pytest.mark.parametrize("name", list(CONFIGS))
def test_config_through_python_api(name):
    from flash_attn_v100 import flash_attn_func

    B, H, N, D, causal, scale, tail, heads = CONFIGS[name]
    heads = list(heads)
    torch.set_num_threads(16)
    q, k, v, do = ao.make_inputs(B, N, H, D, seed=20, zero_tail_rows=tail)
    scale = 1.0 / math.sqrt(D) if scale is None else scale
    print(f"config {name}: B{B} H{H} N{N} D{D} causal={causal}", flush=True)
    qg, kg, vg = (t.cuda().requires_grad_() for t in (q, k, v))
    out = flash_attn_func(qg, kg, vg, scale, causal)
    out.backward(do.cuda())
    torch.cuda.synchronize()
    assert out.shape == q.shape and out.dtype == torch.float16
    sl = lambda t: t[:, :, heads].contiguous()
    o_ref, _ = ao.attention_forward(sl(q), sl(k), sl(v), scale, causal)
    dq_ref, dk_ref, dv_ref = ao.attention_backward(sl(q), sl(k), sl(v), sl(do), scale, causal)
    rows = N - tail  # the padded rows' outputs are ignored by the loss
    errs = (_err(out[:, :rows, heads], o_ref[:, :rows]), _err(qg.grad[:, :, heads], dq_ref),
            _err(kg.grad[:, :, heads], dk_ref), _err(vg.grad[:, :, heads], dv_ref))
    print("  max-abs errors O %.2e dQ %.2e dK %.2e dV %.2e over heads %s" % (*errs, heads), flush=True)
    assert errs[0] <= O_TOL
    assert max(errs[1:]) <= G_TOL  # also the reference's own bound, allclose(atol=1e-2) (test.py:42-45)
    if tail:
        # zero dout on the padded rows + causal masking: their gradients are exactly zero
        for g in (qg.grad, kg.grad, vg.grad):
            assert g[:, rows:].abs().max().item() == 0.0
    # properties that hold at any size
    if causal:
        assert torch.equal(out[:, 0], vg[:, 0])  # row 0 sees only key 0
    assert torch.isfinite(out).all() and torch.isfinite(qg.grad).all()
    assert torch.isfinite(kg.grad).all() and torch.isfinite(vg.grad).all()


SMALL = [  # B, H, N, D, causal, scale
    (1, 1, 32, 64, True, 0.125), (1, 2, 32, 128, False, 0.1), (2, 3, 96, 64, True, 0.125),
    (1, 2, 160, 128, True, 0.0883883), (2, 2, 224, 64, False, 0.125), (1, 3, 288, 128, False, 0.0883883),
    (1, 2, 96, 64, True, -0.125), (1, 2, 128, 128, False, -0.05), (1, 2, 64, 64, True, 0.0),
    (3, 5, 352, 128, True, 0.2), (1, 1, 1056, 64, True, 0.125),
]


@pytest.mark.parametrize("B,H,N,D,causal,scale", SMALL)
def test_c_abi_small_shapes(lib, B, H, N, D, causal, scale):
    q, k, v, do = ao.make_inputs(B, N, H, D, seed=N + D)
    print(f"c-abi B{B} H{H} N{N} D{D} causal={causal} scale={scale}", flush=True)
    qg, kg, vg, dog = (t.cuda() for t in (q, k, v, do))
    out, lse = abi.forward(lib, qg, kg, vg, scale, causal)
    dq, dk, dv, delta = abi.backward(lib, qg, kg, vg, out, dog, lse, scale, causal)
    dq2, dk2, dv2, _ = abi.backward(lib, qg, kg, vg, out, dog, lse, scale, causal, split=True)
    torch.cuda.synchronize()
    o_ref, lse_ref = ao.attention_forward(q, k, v, scale, causal)
    dq_ref, dk_ref, dv_ref = ao.attention_backward(q, k, v, do, scale, causal)
    assert _err(out, o_ref) <= O_TOL
    assert (lse.cpu() - lse_ref).abs().max().item() <= LSE_TOL
    assert (delta.cpu() - ao.attention_delta(out.cpu(), do)).abs().max().item() <= 1e-3
    assert _err(dq, dq_ref) <= G_TOL and _err(dk, dk_ref) <= G_TOL and _err(dv, dv_ref) <= G_TOL
    # the per-pass entry points give bit-identical results
    assert torch.equal(dq, dq2) and torch.equal(dk, dk2) and torch.equal(dv, dv2)


RAGGED = [  # B, H, N, D, causal: lengths that are no multiple of 32 (the last tile is partial)
    (1, 2, 1, 64, True), (2, 2, 7, 128, False), (1, 3, 33, 64, True), (2, 2, 100, 128, True),
    (1, 2, 129, 64, False), (1, 2, 257, 128, True), (1, 1, 1000, 128, False), (1, 2, 1031, 64, True),
]


@pytest.mark.parametrize("B,H,N,D,causal", RAGGED)
def test_ragged_sequence_lengths(lib, B, H, N, D, causal):
    """No right-padding: any N is accepted and matches the oracle on the same N."""
    scale = 1.0 / math.sqrt(D)
    q, k, v, do = ao.make_inputs(B, N, H, D, seed=3 * N + D)
    print(f"ragged B{B} H{H} N{N} D{D} causal={causal}", flush=True)
    qg, kg, vg, dog = (t.cuda() for t in (q, k, v, do))
    out, lse = abi.forward(lib, qg, kg, vg, scale, causal)
    dq, dk, dv, delta = abi.backward(lib, qg, kg, vg, out, dog, lse, scale, causal)
    dq2, dk2, dv2, _ = abi.backward(lib, qg, kg, vg, out, dog, lse, scale, causal, split=True)
    torch.cuda.synchronize()
    o_ref, lse_ref = ao.attention_forward(q, k, v, scale, causal)
    dq_ref, dk_ref, dv_ref = ao.attention_backward(q, k, v, do, scale, causal)
    assert _err(out, o_ref) <= O_TOL
    assert (lse.cpu() - lse_ref).abs().max().item() <= LSE_TOL
    assert (delta.cpu() - ao.attention_delta(out.cpu(), do)).abs().max().item() <= 1e-3
    assert _err(dq, dq_ref) <= G_TOL and _err(dk, dk_ref) <= G_TOL and _err(dv, dv_ref) <= G_TOL
    assert torch.equal(dq, dq2) and torch.equal(dk, dk2) and torch.equal(dv, dv2)
    # the same rows inside a longer, right-padded sequence give the same output under
    # causal masking (the reference's way of handling such lengths, README.md:3)
    if causal:
        pad = (-N) % 32
        if pad:
            qp, kp, vp = (torch.cat([t, torch.zeros(B, pad, H, D, dtype=t.dtype)], 1).cuda() for t in (q, k, v))
            out_p, _ = abi.forward(lib, qp, kp, vp, scale, True)
            # (not bit for bit: when the running maximum is moved depends on all 32 rows of a wave)
            assert (out_p[:, :N].float() - out.float()).abs().max().item() <= 1e-3


def test_golden_fixtures_on_gpu(lib):
    import os
    import numpy as np

    data = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "attention_small.npz"))
    for name in sorted({key.split("/")[0] for key in data.files}):
        B, N, H, D, causal = (int(x) for x in data[f"{name}/meta"])
        scale = float(data[f"{name}/scale"][0])
        q, k, v, do = (torch.from_numpy(data[f"{name}/{t}"]).cuda() for t in ("q", "k", "v", "dout"))
        out, lse = abi.forward(lib, q, k, v, scale, bool(causal))
        dq, dk, dv, _ = abi.backward(lib, q, k, v, out, do, lse, scale, bool(causal))
        want = {t: torch.from_numpy(data[f"{name}/{t}"]) for t in ("out", "lse", "dq", "dk", "dv")}
        assert _err(out, want["out"]) <= O_TOL
        assert (lse.cpu() - want["lse"]).abs().max().item() <= LSE_TOL
        assert _err(dq, want["dq"]) <= G_TOL and _err(dk, want["dk"]) <= G_TOL and _err(dv, want["dv"]) <= G_TOL


def test_invariants_at_full_size(lib):
    """Size-independent properties at the headline shape B2 H32 N4096 D128."""
    B, H, N, D = 2, 32, 4096, 128
    scale = 1.0 / math.sqrt(D)
    q, k, v, do = (t.cuda() for t in ao.make_inputs(B, N, H, D, seed=5))
    out, lse = abi.forward(lib, q, k, v, scale, True)
    # deterministic: a second run is bit-identical, forward and backward (no atomics)
    out2, lse2 = abi.forward(lib, q, k, v, scale, True)
    assert torch.equal(out, out2) and torch.equal(lse, lse2)
    g1 = abi.backward(lib, q, k, v, out, do, lse, scale, True)
    g2 = abi.backward(lib, q, k, v, out, do, lse, scale, True)
    for a, b in zip(g1[:3], g2[:3]):
        assert torch.equal(a, b)
    # causal: O[:n] is independent of K/V[n:], bit for bit
    k2, v2 = k.clone(), v.clone()
    k2[:, 2048:] = 3.0
    v2[:, 2048:] = -3.0
    out3, _ = abi.forward(lib, q, k2, v2, scale, True)
    assert torch.equal(out3[:, :2048], out[:, :2048])
    # constant V gives constant O (rows of P sum to 1)
    vc = torch.full_like(v, 0.75)
    oc, _ = abi.forward(lib, q, k, vc, scale, False)
    assert (oc.float() - 0.75).abs().max().item() <= 1e-3
    # batch / head independence: running one (b, h) slice alone gives the same bits
    sl = lambda t: t[1:2, :, 7:8].contiguous()
    o1, l1 = abi.forward(lib, sl(q), sl(k), sl(v), scale, True)
    assert torch.equal(o1, out[1:2, :, 7:8]) and torch.equal(l1, lse[1:2, 7:8])
    # rows of dS sum to zero  =>  with K constant along the sequence, dQ = 0
    kc = torch.ones_like(k) * 0.5
    oc2, lc2 = abi.forward(lib, q, kc, v, scale, True)
    dqc, _, _, _ = abi.backward(lib, q, kc, v, oc2, do, lc2, scale, True)
    assert dqc.float().abs().max().item() <= 2e-2
    # linearity of the backward in dout: grads(2*dout) == 2*grads(dout) up to fp16 rounding
    g3 = abi.backward(lib, q, k, v, out, do * 2, lse, scale, True)
    for a, b in zip(g1[:3], g3[:3]):
        assert (a.float() * 2 - b.float()).abs().max().item() <= 2e-2


def test_non_dense_inputs_and_side_stream():
    from flash_attn_v100 import flash_attn_func

    B, H, N, D = 2, 4, 256, 64
    q, k, v, do = ao.make_inputs(B, N, H, D, seed=9)
    o_ref, _ = ao.attention_forward(q, k, v, None, True)
    dq_ref, dk_ref, dv_ref = ao.attention_backward(q, k, v, do, None, True)
    # (B, H, N, D)-backed views: last dim contiguous, the rest not dense
    mk = lambda t: t.permute(0, 2, 1, 3).contiguous().cuda().permute(0, 2, 1, 3).requires_grad_()
    qg, kg, vg = mk(q), mk(k), mk(v)
    assert not qg.is_contiguous()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        out = flash_attn_func(qg, kg, vg, causal=True)  # default scale D**-0.5
        out.backward(do.cuda())
    side.synchronize()
    assert _err(out, o_ref) <= O_TOL
    assert _err(qg.grad, dq_ref) <= G_TOL and _err(kg.grad, dk_ref) <= G_TOL and _err(vg.grad, dv_ref) <= G_TOL


def test_random_shapes_and_scales(lib):
    """Forty shapes drawn from a fixed seed: batch 1-3, 1-12 heads (slice counts that are and are not
    multiples of 8), lengths 1-1500 (tiny, ragged, whole tiles), both head sizes, both mask modes, four
    scales including a negative one and one that makes the softmax peaky.  The outputs are fp16, so the
    tolerance grows with the magnitude of the expected tensor (half an ulp of fp16 at 8 is 4e-3)."""
    import random

    rng = random.Random(2024)
    torch.set_num_threads(16)
    for case in range(40):
        B, H, D = rng.randint(1, 3), rng.choice([1, 2, 3, 5, 7, 8, 9, 12]), rng.choice([64, 128])
        N = rng.choice([rng.randint(1, 70), rng.randint(60, 400), rng.randint(400, 1500), 64 * rng.randint(1, 20)])
        causal = rng.random() < 0.6
        scale = rng.choice([1 / math.sqrt(D), 0.1, -0.07, 0.3])
        print(f"case {case}: B{B} H{H} N{N} D{D} causal={causal} scale={scale:.3f}", flush=True)
        q, k, v, do = ao.make_inputs(B, N, H, D, seed=case)
        qg, kg, vg, dog = (t.cuda() for t in (q, k, v, do))
        out, lse = abi.forward(lib, qg, kg, vg, scale, causal)
        dq, dk, dv, _ = abi.backward(lib, qg, kg, vg, out, dog, lse, scale, causal)
        torch.cuda.synchronize()
        o_ref, lse_ref = ao.attention_forward(q, k, v, scale, causal)
        refs = (o_ref,) + tuple(ao.attention_backward(q, k, v, do, scale, causal))
        assert (lse.cpu() - lse_ref).abs().max().item() <= LSE_TOL
        for name, got, want, tol in zip(("O", "dQ", "dK", "dV"), (out, dq, dk, dv), refs, (O_TOL, G_TOL, G_TOL, G_TOL)):
            assert _err(got, want) <= tol * max(1.0, want.abs().max().item()), (case, name)


@pytest.mark.parametrize("D,causal", [(64, True), (128, False), (128, True)])
def test_wide_score_ranges(lib, D, causal):
    """Scores whose running maximum keeps growing along the keys and rows dominated by
    one key: the lazily moved running maximum must still give the oracle's result."""
    B, H, N = 1, 2, 1024
    scale = 1.0 / math.sqrt(D)
    q, k, v, do = ao.make_inputs(B, N, H, D, seed=11 + D)
    ramp = torch.linspace(0.25, 6.0, N).view(1, N, 1, 1)
    k = (k.float() * ramp).half()                 # later keys score higher and higher
    k[:, 0] = (q[:, N // 2].float() * 2).half()   # key 0 is a sink for query N/2
    q[:, 5] = 0                                   # an all-zero query: uniform attention
    qg, kg, vg, dog = (t.cuda() for t in (q, k, v, do))
    out, lse = abi.forward(lib, qg, kg, vg, scale, causal)
    dq, dk, dv, _ = abi.backward(lib, qg, kg, vg, out, dog, lse, scale, causal)
    torch.cuda.synchronize()
    o_ref, lse_ref = ao.attention_forward(q, k, v, scale, causal)
    dq_ref, dk_ref, dv_ref = ao.attention_backward(q, k, v, do, scale, causal)
    assert torch.isfinite(out).all() and torch.isfinite(lse).all()
    assert _err(out, o_ref) <= O_TOL
    assert (lse.cpu() - lse_ref).abs().max().item() <= LSE_TOL
    # dQ scales with the keys here (values beyond 16): allow two fp16 steps at its largest magnitude
    dq_tol = max(G_TOL, 2 * 2.0 ** -10 * dq_ref.abs().max().item())
    assert _err(dq, dq_ref) <= dq_tol and _err(dk, dk_ref) <= G_TOL and _err(dv, dv_ref) <= G_TOL


def _strided_cases(B, N, H, D, seed):
    """The same values behind three layouts that are not dense (B, N, H, D)."""
    q, k, v, do = ao.make_inputs(B, N, H, D, seed=seed)
    packed = torch.stack([q, k, v], dim=2).cuda()                      # (B, N, 3, H, D): a fused QKV projection
    heads_first = [t.permute(0, 2, 1, 3).contiguous().cuda().permute(0, 2, 1, 3) for t in (q, k, v, do)]  # (B, H, N, D) storage
    wide = [torch.cat([t, t], dim=3).cuda()[..., :D] for t in (q, k, v, do)]   # rows twice as long as D
    return (q, k, v, do), {
        "packed_qkv": (packed[:, :, 0], packed[:, :, 1], packed[:, :, 2], do.cuda()),
        "heads_first": tuple(heads_first),
        "wide_rows": tuple(wide),
    }


@pytest.mark.parametrize("B,H,N,D,causal", [(2, 3, 200, 64, True), (1, 2, 320, 128, False), (2, 2, 96, 128, True)])
def test_strided_inputs_c_abi(lib, B, H, N, D, causal):
    """Strided q, k, v, dout give the same bits as their dense copies, without a copy."""
    scale = 1.0 / math.sqrt(D)
    (q, k, v, do), cases = _strided_cases(B, N, H, D, seed=N + D + 1)
    qd, kd, vd, dod = (t.cuda() for t in (q, k, v, do))
    out_d, lse_d = abi.forward(lib, qd, kd, vd, scale, causal)
    dq_d, dk_d, dv_d, _ = abi.backward(lib, qd, kd, vd, out_d, dod, lse_d, scale, causal)
    o_ref, _ = ao.attention_forward(q, k, v, scale, causal)
    assert _err(out_d, o_ref) <= O_TOL
    for name, (qs, ks, vs, gs) in cases.items():
        print(f"strided {name} B{B} H{H} N{N} D{D} causal={causal} q.stride={tuple(qs.stride())}", flush=True)
        assert not qs.is_contiguous() and torch.equal(qs, qd)
        out, lse = abi.forward_strided(lib, qs, ks, vs, scale, causal)
        dq, dk, dv = abi.backward_strided(lib, qs, ks, vs, out, gs, lse, scale, causal)
        torch.cuda.synchronize()
        assert torch.equal(out, out_d) and torch.equal(lse, lse_d), name
        assert torch.equal(dq, dq_d) and torch.equal(dk, dk_d) and torch.equal(dv, dv_d), name


def test_strided_inputs_python_api():
    """flash_attn_func on views of a packed QKV tensor: gradients flow back into the packed tensor."""
    from flash_attn_v100 import flash_attn_func

    B, H, N, D = 2, 4, 160, 64
    q, k, v, do = ao.make_inputs(B, N, H, D, seed=77)
    packed = torch.stack([q, k, v], dim=2).cuda().requires_grad_()
    out = flash_attn_func(packed[:, :, 0], packed[:, :, 1], packed[:, :, 2], None, True)
    out.backward(do.cuda())
    scale = 1.0 / math.sqrt(D)
    o_ref, _ = ao.attention_forward(q, k, v, scale, True)
    dq_ref, dk_ref, dv_ref = ao.attention_backward(q, k, v, do, scale, True)
    assert _err(out, o_ref) <= O_TOL
    g = packed.grad
    assert _err(g[:, :, 0], dq_ref) <= G_TOL and _err(g[:, :, 1], dk_ref) <= G_TOL and _err(g[:, :, 2], dv_ref) <= G_TOL
    # a layout whose rows are not on 16-byte boundaries falls back to a dense copy and still works
    odd = torch.zeros(B, N, H, D + 4, dtype=torch.float16, device="cuda")
    odd[..., :D] = q.cuda()
    out2 = flash_attn_func(odd[..., :D], k.cuda(), v.cuda(), None, True)
    assert torch.equal(out2, out.detach())


def test_hip_graph_capture_and_replay():
    """The extension only launches kernels on the current stream (no synchronisation, no memset),
    so forward + backward can be captured into a graph; every replay must equal the eager result."""
    from flash_attn_v100 import flash_attn_func

    B, H, N, D = 2, 4, 200, 64
    static = [torch.zeros(B, N, H, D, dtype=torch.float16, device="cuda") for _ in range(4)]
    sq, sk, sv, sdo = static
    sq.requires_grad_(), sk.requires_grad_(), sv.requires_grad_()

    def step():
        out = flash_attn_func(sq, sk, sv, None, True)
        gq, gk, gv = torch.autograd.grad(out, (sq, sk, sv), sdo)
        return out, gq, gk, gv

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):  # warm-up on a side stream, as graph capture asks for
        for _ in range(2):
            step()
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        captured = step()
    for seed in (1, 2, 3):
        q, k, v, do = ao.make_inputs(B, N, H, D, seed=seed)
        with torch.no_grad():
            for dst, src in zip(static, (q, k, v, do)):
                dst.copy_(src.cuda())
        graph.replay()
        torch.cuda.synchronize()
        replayed = [t.clone() for t in captured]
        eager = step()  # the program's own eager work between the replays
        torch.cuda.synchronize()
        for a, b in zip(replayed, eager):
            assert torch.equal(a, b), f"replay with seed {seed} differs from the eager result"
        o_ref, _ = ao.attention_forward(q, k, v, None, True)
        assert _err(replayed[0], o_ref) <= O_TOL


SPILL_CASES = [  # B, H, N, D, causal
    (1, 2, 64, 128, True), (2, 3, 333, 64, True), (1, 2, 70, 128, False), (1, 2, 40, 64, True),
    (1, 2, 1031, 128, True), (2, 4, 512, 64, False), (1, 20, 384, 128, True), (1, 9, 1500, 64, False),
]


@pytest.mark.parametrize("B,H,N,D,causal", SPILL_CASES)
def test_spill_and_recompute_backward_agree(lib, B, H, N, D, causal):
    """The backward has two paths, chosen by the size of the workspace: with room for the dS tiles the dK/dV pass
    spills them and the dQ pass is one GEMM; with the minimum workspace the dQ pass recomputes S and dP.  dK and
    dV come from the same arithmetic (bit-equal); dQ sums the same products tile by tile (equal to rounding);
    both match the oracle."""
    scale = 1.0 / math.sqrt(D)
    q, k, v, do = ao.make_inputs(B, N, H, D, seed=5 * N + D)
    print(f"spill/recompute B{B} H{H} N{N} D{D} causal={causal}", flush=True)
    assert lib.fused_mha_backward_workspace_bytes(B, H, N, D) > lib.fused_mha_backward_min_workspace_bytes(B, H, N, D)
    qg, kg, vg, dog = (t.cuda() for t in (q, k, v, do))
    out, lse = abi.forward(lib, qg, kg, vg, scale, causal)
    dq_s, dk_s, dv_s, _ = abi.backward(lib, qg, kg, vg, out, dog, lse, scale, causal)
    dq_p, dk_p, dv_p, _ = abi.backward(lib, qg, kg, vg, out, dog, lse, scale, causal, split=True)
    dq_r, dk_r, dv_r, _ = abi.backward(lib, qg, kg, vg, out, dog, lse, scale, causal, min_workspace=True)
    torch.cuda.synchronize()
    assert torch.equal(dk_s, dk_r) and torch.equal(dv_s, dv_r)
    assert torch.equal(dq_s, dq_p) and torch.equal(dk_s, dk_p) and torch.equal(dv_s, dv_p)  # per-pass entry points
    assert (dq_s.float() - dq_r.float()).abs().max().item() <= 2e-3
    dq_ref, dk_ref, dv_ref = ao.attention_backward(q, k, v, do, scale, causal)
    for got in (dq_s, dq_r):
        assert _err(got, dq_ref) <= G_TOL
    assert _err(dk_s, dk_ref) <= G_TOL and _err(dv_s, dv_ref) <= G_TOL
    assert torch.isfinite(dq_s).all()


TWO_PANEL_CASES = [  # B, H, N, D, causal: at least 1024 blocks of 256 queries
    (8, 32, 1024, 128, True), (7, 32, 1100, 64, True), (4, 64, 1000, 64, False), (7, 32, 1100, 128, False),
    (8, 32, 777, 128, True),
]


@pytest.mark.parametrize("B,H,N,D,causal", TWO_PANEL_CASES)
def test_spill_backward_with_many_blocks(lib, B, H, N, D, causal):
    """With enough blocks to go round, the dQ pass over the spilled dS takes 256 queries per block instead of 128
    (a K tile then serves twice as many queries).  Shapes that select it, with ragged ends, an odd number of
    128-query panels (the second half of the last block is then empty) and both maskings: dK and dV are bit-equal
    to the minimum-workspace path, dQ equal to rounding, and batch 0 matches the oracle."""
    scale = 1.0 / math.sqrt(D)
    q, k, v, do = ao.make_inputs(B, N, H, D, seed=3 * N + D)
    print(f"two-panel spill B{B} H{H} N{N} D{D} causal={causal}", flush=True)
    assert ((N + 255) // 256) * B * H >= 1024
    qg, kg, vg, dog = (t.cuda() for t in (q, k, v, do))
    out, lse = abi.forward(lib, qg, kg, vg, scale, causal)
    dq_s, dk_s, dv_s, _ = abi.backward(lib, qg, kg, vg, out, dog, lse, scale, causal)
    dq_r, dk_r, dv_r, _ = abi.backward(lib, qg, kg, vg, out, dog, lse, scale, causal, min_workspace=True)
    torch.cuda.synchronize()
    assert torch.equal(dk_s, dk_r) and torch.equal(dv_s, dv_r)
    assert (dq_s.float() - dq_r.float()).abs().max().item() <= 2e-3
    assert torch.isfinite(dq_s).all()
    dq_ref, dk_ref, dv_ref = ao.attention_backward(q[:1], k[:1], v[:1], do[:1], scale, causal)
    assert _err(dq_s[:1], dq_ref) <= G_TOL
    assert _err(dk_s[:1], dk_ref) <= G_TOL and _err(dv_s[:1], dv_ref) <= G_TOL


def _forward_oracle_in_row_chunks(q, k, v, scale, causal, chunk=2048):
    """attention_oracle.attention_forward for ONE (batch, head) slice, evaluated in chunks of query rows so that
    the score matrix in memory is chunk x N (fp32) instead of N x N; same formulas (test.py:13-26)."""
    N = q.shape[0]
    outs, lses = [], []
    for r0 in range(0, N, chunk):
        r1 = min(N, r0 + chunk)
        nk = r1 if causal else N  # keys past the chunk's last row are masked for all of its rows
        s = (q[r0:r1].float() @ k[:nk].float().t()) * scale
        if causal:
            rows = torch.arange(r0, r1).unsqueeze(1)
            s = s.masked_fill(torch.arange(nk).unsqueeze(0) > rows, float("-inf"))
        lses.append(torch.logsumexp(s, dim=-1))
        outs.append(torch.softmax(s, dim=-1) @ v[:nk].float())
    return torch.cat(outs), torch.cat(lses)


def test_long_context_forward_all_heads(lib):
    """B1 H16 N16384 D128 causal: O and lse of every head against the oracle (in row chunks: a whole head's score
    matrix would be 1 GiB), not only of the three heads whose backward is checked."""
    B, H, N, D, causal = 1, 16, 16384, 128, True
    scale = 1.0 / math.sqrt(D)
    torch.set_num_threads(16)
    q, k, v, _ = ao.make_inputs(B, N, H, D, seed=20, zero_tail_rows=32)
    out, lse = abi.forward(lib, q.cuda(), k.cuda(), v.cuda(), scale, causal)
    torch.cuda.synchronize()
    out, lse = out.cpu(), lse.cpu()
    # the chunked evaluation is the oracle's: same numbers on a head small enough for both
    o_small, l_small = _forward_oracle_in_row_chunks(q[0, :3000, 0], k[0, :3000, 0], v[0, :3000, 0], scale, causal, 512)
    o_ref, l_ref = ao.attention_forward(q[:, :3000, :1], k[:, :3000, :1], v[:, :3000, :1], scale, causal)
    assert (o_small - o_ref[0, :, 0]).abs().max().item() <= 1e-5 and (l_small - l_ref[0, 0]).abs().max().item() <= 1e-4
    for h in range(H):
        o_ref, l_ref = _forward_oracle_in_row_chunks(q[0, :, h], k[0, :, h], v[0, :, h], scale, causal)
        eo = (out[0, :, h].float() - o_ref.half().float()).abs().max().item()
        el = (lse[0, h] - l_ref).abs().max().item()
        print(f"long context head {h}: O {eo:.2e} lse {el:.2e}", flush=True)
        assert eo <= O_TOL and el <= LSE_TOL


def test_extension_takes_caller_supplied_outputs():
    """ext.fwd with out_ and ext.bwd with dq_, dk_, dv_ supplied by the caller (reference
    kernel/fused_mha_api.cpp:49-58, 125-153): the results land in those tensors, equal to the ones the extension
    allocates itself, and nothing depends on what the tensors held (NaN here; the reference needs dq zero-filled)."""
    import flash_attn_v100_cuda as ext

    B, H, N, D, causal = 2, 3, 300, 128, True
    scale = 1.0 / math.sqrt(D)
    q, k, v, do = ao.make_inputs(B, N, H, D, seed=91)
    qg, kg, vg, dog = (t.cuda() for t in (q, k, v, do))
    out0, lse0 = ext.fwd(qg, kg, vg, None, scale, causal)
    mine = torch.full_like(qg, float("nan"))
    out1, lse1 = ext.fwd(qg, kg, vg, mine, scale, causal)
    torch.cuda.synchronize()
    assert out1.data_ptr() == mine.data_ptr()
    assert torch.equal(mine, out0) and torch.equal(lse1, lse0)
    o_ref, _ = ao.attention_forward(q, k, v, scale, causal)
    assert _err(mine, o_ref) <= O_TOL
    with pytest.raises(RuntimeError, match="contiguous"):
        ext.fwd(qg, kg, vg, torch.empty(B, H, N, D, dtype=torch.float16, device="cuda").transpose(1, 2), scale, causal)
    with pytest.raises(RuntimeError):
        ext.fwd(qg, kg, vg, torch.empty(B, N, H, D, dtype=torch.float32, device="cuda"), scale, causal)

    dq0, dk0, dv0 = ext.bwd(dog, qg, kg, vg, out0, lse0, None, None, None, scale, causal)
    grads = [torch.full_like(qg, float("nan")) for _ in range(3)]
    dq1, dk1, dv1 = ext.bwd(dog, qg, kg, vg, out0, lse0, grads[0], grads[1], grads[2], scale, causal)
    torch.cuda.synchronize()
    assert [t.data_ptr() for t in (dq1, dk1, dv1)] == [t.data_ptr() for t in grads]
    assert torch.equal(grads[0], dq0) and torch.equal(grads[1], dk0) and torch.equal(grads[2], dv0)
    dq_ref, dk_ref, dv_ref = ao.attention_backward(q, k, v, do, scale, causal)
    assert _err(grads[0], dq_ref) <= G_TOL and _err(grads[1], dk_ref) <= G_TOL and _err(grads[2], dv_ref) <= G_TOL


def test_errors_on_gpu():
    from flash_attn_v100 import flash_attn_func

    bad = torch.zeros(1, 0, 2, 64, dtype=torch.float16, device="cuda")
    with pytest.raises(RuntimeError, match="seqlen must be positive"):
        flash_attn_func(bad, bad, bad)
    bad = torch.zeros(1, 64, 2, 32, dtype=torch.float16, device="cuda")
    with pytest.raises(RuntimeError, match="head dimension"):
        flash_attn_func(bad, bad, bad)
    ok = torch.zeros(1, 64, 2, 64, dtype=torch.float32, device="cuda")
    with pytest.raises(RuntimeError, match="fp16"):
        flash_attn_func(ok, ok, ok)
