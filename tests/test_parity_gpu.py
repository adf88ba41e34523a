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
