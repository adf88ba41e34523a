"""CPU tests that pin the oracle (oracle/attention_oracle.py) before anything is
compared against it: brute-force fp64 loops, autograd, gradcheck, closed forms,
invariants, and the committed fixtures."""
import math
import os

import numpy as np
import pytest
import torch

from oracle import attention_oracle as ao
from oracle.bruteforce import attention_bruteforce

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "attention_small.npz")

SMALL = [  # B, N, H, D, causal
    (1, 32, 1, 64, True), (1, 32, 2, 64, False), (2, 96, 2, 64, True),
    (1, 64, 1, 128, True), (1, 160, 2, 128, False),
]


@pytest.mark.parametrize("B,N,H,D,causal", SMALL)
def test_oracle_matches_bruteforce(B, N, H, D, causal):
    q, k, v, do = ao.make_inputs(B, N, H, D, seed=3)
    scale = D ** -0.5
    bo, bl, bdq, bdk, bdv = attention_bruteforce(q.numpy(), k.numpy(), v.numpy(), do.numpy(), scale, causal)
    o, lse = ao.attention_forward(q, k, v, scale, causal, dtype=torch.float64)
    dq, dk, dv = ao.attention_backward(q, k, v, do, scale, causal, dtype=torch.float64)
    for got, want in ((o, bo), (lse, bl), (dq, bdq), (dk, bdk), (dv, bdv)):
        np.testing.assert_allclose(got.numpy(), want, rtol=0, atol=1e-11)
    # and the fp32 evaluation used as the parity reference stays within fp32 noise of it
    o32, lse32 = ao.attention_forward(q, k, v, scale, causal)
    dq32, dk32, dv32 = ao.attention_backward(q, k, v, do, scale, causal)
    for got, want in ((o32, bo), (lse32, bl), (dq32, bdq), (dk32, bdk), (dv32, bdv)):
        np.testing.assert_allclose(got.numpy(), want, rtol=0, atol=2e-5)


def test_plumbing_config_on_cpu():
    """B=1 H=4 N=128 D=64 non-causal, fwd + bwd, entirely on the CPU: analytic
    backward == autograd of the forward == brute force."""
    q, k, v, do = ao.make_inputs(1, 128, 4, 64)
    scale = 1 / math.sqrt(64)
    o, _ = ao.attention_forward(q, k, v, scale, False)
    dq, dk, dv = ao.attention_backward(q, k, v, do, scale, False)
    o2, dq2, dk2, dv2 = ao.attention_autograd(q, k, v, do, scale, False)
    for a, b in ((o, o2), (dq, dq2), (dk, dk2), (dv, dv2)):
        assert (a - b).abs().max().item() < 5e-6
    bo, _, bdq, bdk, bdv = attention_bruteforce(q.numpy(), k.numpy(), v.numpy(), do.numpy(), scale, False)
    for a, b in ((o, bo), (dq, bdq), (dk, bdk), (dv, bdv)):
        assert np.abs(a.numpy() - b).max() < 2e-5


@pytest.mark.parametrize("causal", [False, True])
def test_analytic_backward_equals_autograd(causal):
    q, k, v, do = ao.make_inputs(2, 64, 3, 64, seed=7)
    dq, dk, dv = ao.attention_backward(q, k, v, do, 0.2, causal, dtype=torch.float64)
    _, dq2, dk2, dv2 = ao.attention_autograd(q, k, v, do, 0.2, causal, dtype=torch.float64)
    for a, b in ((dq, dq2), (dk, dk2), (dv, dv2)):
        assert (a - b).abs().max().item() < 1e-12


@pytest.mark.parametrize("causal", [False, True])
def test_gradcheck_fp64(causal):
    torch.manual_seed(0)
    q, k, v = (torch.randn(1, 8, 2, 4, dtype=torch.float64, requires_grad=True) for _ in range(3))

    def f(q, k, v):
        return ao.attention_forward(q, k, v, 0.5, causal, dtype=torch.float64)[0]

    assert torch.autograd.gradcheck(f, (q, k, v), eps=1e-6, atol=1e-6)


def test_golden_fixtures():
    data = np.load(GOLDEN)  # allow_pickle defaults to False
    names = sorted({key.split("/")[0] for key in data.files})
    assert len(names) == 4
    for name in names:
        B, N, H, D, causal = (int(x) for x in data[f"{name}/meta"])
        scale = float(data[f"{name}/scale"][0])
        q, k, v, do = (torch.from_numpy(data[f"{name}/{t}"]) for t in ("q", "k", "v", "dout"))
        assert q.shape == (B, N, H, D)
        o, lse = ao.attention_forward(q, k, v, scale, bool(causal))
        dq, dk, dv = ao.attention_backward(q, k, v, do, scale, bool(causal))
        for got, key in ((o, "out"), (lse, "lse"), (dq, "dq"), (dk, "dk"), (dv, "dv")):
            np.testing.assert_allclose(got.numpy(), data[f"{name}/{key}"], rtol=0, atol=2e-5)


def test_closed_forms_and_invariants():
    B, N, H, D = 1, 64, 2, 64
    q, k, v, do = ao.make_inputs(B, N, H, D, seed=11)
    scale = 0.125
    # softmax / logsumexp closed form, and LSE = max + ln(sum) of the two statistics
    # the reference stores (kernel/fused_mha_kernel.cu:173-178, 298-303)
    o, lse = ao.attention_forward(q, k, v, scale, True)
    s = torch.einsum("bihd,bjhd->bhij", q.float(), k.float()) * scale
    s = s.masked_fill(~torch.ones(N, N, dtype=torch.bool).tril(), float("-inf"))
    mx = s.max(-1).values
    sm = torch.exp(s - mx[..., None]).sum(-1)
    assert (lse - (mx + sm.log())).abs().max() < 1e-5
    assert (o - torch.einsum("bhij,bjhd->bihd", torch.softmax(s, -1), v.float())).abs().max() < 1e-5
    # causal row 0 sees only key 0
    assert torch.equal(o[:, 0], v[:, 0].float())
    assert (lse[:, :, 0] - scale * (q[:, 0].float() * k[:, 0].float()).sum(-1)).abs().max() < 1e-5
    # constant V gives constant O (rows of P sum to 1)
    vc = torch.full_like(v, 0.75)
    oc, _ = ao.attention_forward(q, k, vc, scale, False)
    assert (oc - 0.75).abs().max() < 1e-6
    # scale = 0: uniform P, causal O is the prefix mean of V
    o0, lse0 = ao.attention_forward(q, k, v, 0.0, True)
    prefix = v.float().cumsum(1) / torch.arange(1, N + 1).view(1, N, 1, 1)
    assert (o0 - prefix).abs().max() < 1e-5
    assert (lse0 - torch.log(torch.arange(1, N + 1).float())).abs().max() < 1e-5
    # causal: O[:n] does not depend on K/V[n:]
    k2, v2 = k.clone(), v.clone()
    k2[:, 40:] = 9.0
    v2[:, 40:] = -9.0
    o2, _ = ao.attention_forward(q, k2, v2, scale, True)
    assert torch.equal(o2[:, :40], o[:, :40])
    # non-causal: permuting keys/values together leaves O unchanged
    perm = torch.randperm(N, generator=torch.Generator().manual_seed(1))
    on, _ = ao.attention_forward(q, k, v, scale, False)
    op, _ = ao.attention_forward(q, k[:, perm], v[:, perm], scale, False)
    assert (on - op).abs().max() < 1e-5
    # heads are independent
    oh, _ = ao.attention_forward(q[:, :, 1:], k[:, :, 1:], v[:, :, 1:], scale, True)
    assert torch.equal(oh, o[:, :, 1:])
    # delta identity: rowsum(dO o O) == rowsum(P o dP)
    p = torch.softmax(s, -1)
    dp = torch.einsum("bihd,bjhd->bhij", do.float(), v.float())
    assert (ao.attention_delta(o, do) - (p * dp).sum(-1)).abs().max() < 1e-4
    # dout = 0 on a row gives dq = 0 on that row; under causal masking zero dout on the
    # tail rows gives zero dk, dv on those rows too
    do2 = do.clone()
    do2[:, N - 8:] = 0
    dq, dk, dv = ao.attention_backward(q, k, v, do2, scale, True)
    assert dq[:, N - 8:].abs().max() == 0 and dk[:, N - 8:].abs().max() == 0 and dv[:, N - 8:].abs().max() == 0


def test_flop_count():
    assert ao.flops(2, 32, 4096, 128, True, "fwd") == pytest.approx(274.878e9, rel=1e-5)
    assert ao.flops(2, 32, 4096, 128, True, "fwd_bwd") == pytest.approx(962.073e9, rel=1e-5)
    assert ao.flops(16, 12, 512, 64, False, "fwd") == pytest.approx(12.885e9, rel=1e-4)
