# The shape of this API (flash_attn_func over a torch.autograd.Function that calls
# a compiled fwd/bwd pair) follows flash_attn_interface.py of FlashAttention,
# Copyright (c) 2023, Tri Dao, through the reference's copy of that file.
"""Autograd front end, API-compatible with the reference's
flash_attn_v100/flash_attn_interface.py:1-110.

``flash_attn_func(q, k, v, softmax_scale=None, causal=False)`` takes fp16
tensors of shape (batch, seqlen, heads, head_size) and returns the attention
output in the same layout, just like the reference; seqlen need not be
right-padded to a multiple of 32 as the reference asks (any length works, a
padded one still does).  What differs is behind the extension boundary: the forward
saves one fp32 logsumexp per row instead of separate max and sum tensors, and
delta = rowsum(dout * out) is computed on the device in fp32 by the backward
launcher instead of by two fp16 PyTorch ops (reference :43-44).

The compiled extension is required: importing this module without it raises.
"""
import torch

# The kernels are imported after torch so that they bind to the HIP runtime
# torch has already loaded (same order as reference flash_attn_interface.py:8-9).
try:
    import flash_attn_v100_cuda as flash_attn_cuda
except ImportError as exc:  # fail loudly: there is no fallback path
    raise ImportError(
        "flash_attn_v100 needs its compiled extension flash_attn_v100_cuda "
        "(run `python setup.py build_ext --inplace` in flash-attention-v100_amd/): %s" % exc
    ) from exc


def _flash_attn_forward(q, k, v, softmax_scale, causal):
    maybe_contiguous = lambda x: x.contiguous() if x.stride(-1) != 1 else x
    q, k, v = [maybe_contiguous(x) for x in (q, k, v)]
    out, softmax_lse = flash_attn_cuda.fwd(q, k, v, None, softmax_scale, causal)
    return out, q, k, v, softmax_lse


def _flash_attn_backward(dout, q, k, v, out, softmax_lse, dq, dk, dv, softmax_scale, causal):
    maybe_contiguous = lambda x: x.contiguous() if x.stride(-1) != 1 else x
    # dq, dk, dv are allocated by us so they should already be contiguous
    dout, q, k, v, out = [maybe_contiguous(x) for x in (dout, q, k, v, out)]
    dq, dk, dv = flash_attn_cuda.bwd(dout, q, k, v, out, softmax_lse, dq, dk, dv, softmax_scale, causal)
    return dq, dk, dv


class FlashAttnFunc(torch.autograd.Function):
    @staticmethod
    def forward(ctx, q, k, v, softmax_scale, causal):
        if softmax_scale is None:
            softmax_scale = q.shape[-1] ** (-0.5)
        out, q, k, v, softmax_lse = _flash_attn_forward(q, k, v, softmax_scale, causal=causal)
        ctx.save_for_backward(q, k, v, out, softmax_lse)
        ctx.softmax_scale = softmax_scale
        ctx.causal = causal
        return out

    @staticmethod
    def backward(ctx, dout, *args):
        q, k, v, out, softmax_lse = ctx.saved_tensors
        # every element of dq, dk, dv is written by the kernels: no zero fill
        # (the reference needs zeros for its atomics, :84)
        # dense (B, N, H, D) whatever the strides of the saved inputs are
        dq, dk, dv = (torch.empty_like(x, memory_format=torch.contiguous_format) for x in (q, k, v))
        _flash_attn_backward(dout, q, k, v, out, softmax_lse, dq, dk, dv, ctx.softmax_scale, ctx.causal)
        return dq, dk, dv, None, None


def flash_attn_func(q, k, v, softmax_scale=None, causal=False):
    return FlashAttnFunc.apply(q, k, v, softmax_scale, causal)
