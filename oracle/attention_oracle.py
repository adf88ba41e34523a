"""fp32 CPU restatement of the reference attention math.  TEST INFRASTRUCTURE ONLY.

The product never imports this file; it exists so tests can check the HIP
kernels.  It restates, entirely in fp32 (or fp64 on request), the formula the
reference uses as its own correctness check:

    reference test.py:13-26
        p = (q @ k^T) * sm_scale          # per (batch, head)
        p[j > i] = -inf   (if causal)     # key j visible to query i iff j <= i
        p = softmax(p)
        out = p @ v
        out.backward(dout)  ->  dq, dk, dv

Differences from the reference script, on purpose: the two matmuls run in fp32
here (the script runs them in fp16 and only the softmax in fp32,
test.py:17,20-21) and P is not rounded to fp16 before P@V.

Layouts follow the reference: q, k, v, out, dout are (B, N, H, D)
(kernel/fused_mha_api.cpp:37-47), row statistics are (B, H, N)
(kernel/fused_mha_api.cpp:65-66).

How each function is pinned (none of them is "parity unpinned"):
  * attention_forward      - against torch.softmax/torch.logsumexp closed forms,
                             the fp64 brute-force C loops in attention_bruteforce.c,
                             and invariants (constant V, causal row 0, scale 0).
  * attention_backward     - analytic formulas (reference
                             kernel/fused_mha_kernel.cu:598-603, 653-656) checked
                             against torch autograd of attention_autograd, against
                             torch.autograd.gradcheck in fp64, and against the
                             brute-force C loops.
  * attention_delta        - identity delta_i = sum_j P_ij dP_ij.
The reference holds no golden vectors for this path (its only check,
test.py:42-45, draws inputs from the GPU RNG), so the fixtures under
tests/golden/ are produced by the brute-force C program from hand-listed inputs.
"""
import math

import torch


def make_inputs(batch, n, head, d, seed=20, dtype=torch.float16, zero_tail_rows=0):
    """Seeded N(0,1) q, k, v, dout, drawn on the CPU in fp32 in that order and
    rounded to fp16 (reference test.py:5-10 draws them in the same order).
    ``zero_tail_rows`` zeroes dout on the last rows (right-padding that the
    loss ignores)."""
    g = torch.Generator(device="cpu")
    g.manual_seed(seed)
    out = []
    for _ in range(4):
        out.append(torch.randn((batch, n, head, d), generator=g, dtype=torch.float32).to(dtype))
    if zero_tail_rows:
        out[3][:, n - zero_tail_rows:] = 0
    return tuple(out)


def _scores(qh, kh, scale, causal):
    # qh, kh: (N, D).  reference test.py:17-19
    s = (qh @ kh.t()) * scale
    if causal:
        n = s.shape[0]
        mask = torch.ones((n, n), dtype=torch.bool).tril_()
        s = s.masked_fill(~mask, float("-inf"))
    return s


def attention_forward(q, k, v, scale=None, causal=False, dtype=torch.float32):
    """Returns (out (B,N,H,D), lse (B,H,N)) in ``dtype``, looping over (b, h) so
    the N x N score matrix exists for one head at a time."""
    B, N, H, D = q.shape
    if scale is None:
        scale = D ** -0.5  # reference flash_attn_interface.py:67-68
    out = torch.empty((B, N, H, D), dtype=dtype)
    lse = torch.empty((B, H, N), dtype=dtype)
    for b in range(B):
        for h in range(H):
            s = _scores(q[b, :, h].to(dtype), k[b, :, h].to(dtype), scale, causal)
            l = torch.logsumexp(s, dim=-1)
            p = torch.exp(s - l[:, None])  # == softmax(s), reference test.py:20
            out[b, :, h] = p @ v[b, :, h].to(dtype)
            lse[b, h] = l
    return out, lse


def attention_delta(out, dout, dtype=torch.float32):
    """delta (B,H,N) = rowsum(dout * out); reference flash_attn_interface.py:43-44
    (there in fp16)."""
    return (out.to(dtype) * dout.to(dtype)).sum(-1).permute(0, 2, 1).contiguous()


def attention_backward(q, k, v, dout, scale=None, causal=False, dtype=torch.float32):
    """Analytic gradients (dq, dk, dv), each (B,N,H,D) in ``dtype``.

        P  = softmax(S)                       kernel/fused_mha_kernel.cu:598-603
        dV = P^T dO                           :618-629
        dP = dO V^T                           :631-644
        dS = P o (dP - rowsum(P o dP)) scale  :653-656
        dQ = dS K, dK = dS^T Q                :680-683, 697-712
    """
    B, N, H, D = q.shape
    if scale is None:
        scale = D ** -0.5
    dq = torch.empty((B, N, H, D), dtype=dtype)
    dk = torch.empty_like(dq)
    dv = torch.empty_like(dq)
    for b in range(B):
        for h in range(H):
            qh, kh, vh, gh = (t[b, :, h].to(dtype) for t in (q, k, v, dout))
            s = _scores(qh, kh, scale, causal)
            p = torch.softmax(s, dim=-1)
            dv[b, :, h] = p.t() @ gh
            dp = gh @ vh.t()
            ds = p * (dp - (p * dp).sum(-1, keepdim=True)) * scale
            dq[b, :, h] = ds @ kh
            dk[b, :, h] = ds.t() @ qh
    return dq, dk, dv


def attention_autograd(q, k, v, dout, scale=None, causal=False, dtype=torch.float32):
    """The reference script's own procedure (test.py:13-26): build the forward
    with differentiable torch ops, call backward(dout), read .grad.  Batched
    over (B, H); use for sizes where B*H*N*N elements fit in memory."""
    B, N, H, D = q.shape
    if scale is None:
        scale = D ** -0.5
    qq, kk, vv = (t.detach().to(dtype).requires_grad_() for t in (q, k, v))
    qt, kt, vt = qq.transpose(1, 2), kk.transpose(1, 2), vv.transpose(1, 2)
    p = torch.matmul(qt, kt.transpose(2, 3)) * scale
    if causal:
        m = torch.tril(torch.ones((N, N)))
        p = p.masked_fill(m == 0, float("-inf"))
    p = torch.softmax(p, dim=-1)
    out = torch.matmul(p, vt).transpose(1, 2)
    out.backward(dout.to(dtype))
    return out.detach(), qq.grad, kk.grad, vv.grad


def flops(batch, head, n, d, causal, mode="fwd"):
    """Algorithmic FLOPs: 4*B*H*N^2*D for the forward, halved when causal;
    backward = 2.5 x forward."""
    f = 4.0 * batch * head * n * n * d
    if causal:
        f *= 0.5
    return {"fwd": f, "bwd": 2.5 * f, "fwd_bwd": 3.5 * f}[mode]
