"""ctypes binding of the C ABI in include/fused_mha.h, for the tests.

torch is imported first so the library binds to the HIP runtime torch loaded.
The library must have been built beforehand (setup.py build_ext); nothing is
compiled from here."""
import ctypes
import os
import re

import torch  # noqa: F401  (load order matters)

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
LIB_PATH = os.path.join(ROOT, "flash-attention-v100_amd", "flash_attn_v100", "lib", "libfused_mha.so")
HEADER = os.path.join(ROOT, "include", "fused_mha.h")

OK = 0
(ERR_NULL_POINTER, ERR_BAD_SHAPE, ERR_BAD_HEAD_DIM, ERR_MISALIGNED, ERR_LAUNCH, ERR_BAD_SCALE, ERR_TOO_LARGE,
 ERR_BAD_STRIDE, ERR_SCRATCH_LIMIT, ERR_RUNTIME) = (-1, -2, -3, -4, -5, -6, -7, -8, -9, -10)
NOALLOC_MAX_ROWS = 1 << 20

_vp, _i, _f, _sz = ctypes.c_void_p, ctypes.c_int, ctypes.c_float, ctypes.c_size_t


class Strides(ctypes.Structure):
    """struct fused_mha_strides: element strides of a (batch, n, head, d) tensor."""
    _fields_ = [("batch", ctypes.c_longlong), ("seq", ctypes.c_longlong), ("head", ctypes.c_longlong)]

    @classmethod
    def of(cls, t):
        return cls(t.stride(0), t.stride(1), t.stride(2))


_sp = ctypes.POINTER(Strides)


def declared_symbols():
    """Function names the header declares."""
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(fused_mha_\w+)\s*\(", text)))


def load():
    if not os.path.exists(LIB_PATH):
        raise RuntimeError("libfused_mha.so is not built: run `python setup.py build_ext` in flash-attention-v100_amd/")
    lib = ctypes.CDLL(LIB_PATH)
    lib.fused_mha_forward.argtypes = [_vp] * 5 + [_i] * 5 + [_f, _i, _vp]
    lib.fused_mha_forward.restype = _i
    lib.fused_mha_backward_workspace_bytes.argtypes = [_i] * 4
    lib.fused_mha_backward_workspace_bytes.restype = _sz
    lib.fused_mha_backward_min_workspace_bytes.argtypes = [_i] * 4
    lib.fused_mha_backward_min_workspace_bytes.restype = _sz
    lib.fused_mha_backward.argtypes = [_vp] * 7 + [_sz] + [_vp] * 3 + [_i] * 5 + [_f, _i, _vp]
    lib.fused_mha_backward.restype = _i
    lib.fused_mha_backward_noalloc.argtypes = [_vp] * 9 + [_i] * 5 + [_f, _i, _vp]
    lib.fused_mha_backward_noalloc.restype = _i
    lib.fused_mha_backward_delta.argtypes = [_vp, _vp, _vp, _vp, _sz] + [_i] * 4 + [_vp]
    lib.fused_mha_backward_delta.restype = _i
    lib.fused_mha_backward_dq.argtypes = [_vp] * 6 + [_sz, _vp] + [_i] * 4 + [_f, _i, _vp]
    lib.fused_mha_backward_dq.restype = _i
    lib.fused_mha_backward_dkdv.argtypes = [_vp] * 6 + [_sz, _vp, _vp] + [_i] * 4 + [_f, _i, _vp]
    lib.fused_mha_backward_dkdv.restype = _i
    lib.fused_mha_forward_strided.argtypes = [_vp, _sp] * 3 + [_vp, _vp] + [_i] * 4 + [_f, _i, _vp]
    lib.fused_mha_forward_strided.restype = _i
    lib.fused_mha_backward_strided.argtypes = ([_vp, _sp] * 3 + [_vp, _vp, _sp, _vp, _vp, _sz] + [_vp] * 3 + [_i] * 4 +
                                               [_f, _i, _vp])
    lib.fused_mha_backward_strided.restype = _i
    lib.fused_mha_error_string.argtypes = [_i]
    lib.fused_mha_error_string.restype = ctypes.c_char_p
    return lib


def forward(lib, q, k, v, scale, causal, stream=None):
    """q, k, v: dense fp16 device tensors (B, N, H, D).  Returns (out, lse)."""
    B, N, H, D = q.shape
    out = torch.empty_like(q)
    lse = torch.empty((B, H, N), dtype=torch.float32, device=q.device)
    s = torch.cuda.current_stream().cuda_stream if stream is None else stream
    rc = lib.fused_mha_forward(q.data_ptr(), k.data_ptr(), v.data_ptr(), out.data_ptr(), lse.data_ptr(),
                               B, H, N, N, D, scale, int(causal), s)
    assert rc == OK, lib.fused_mha_error_string(rc)
    return out, lse


def backward(lib, q, k, v, out, dout, lse, scale, causal, stream=None, split=False, min_workspace=False):
    """min_workspace: pass only delta + lse2 (the dQ pass then recomputes S and dP) instead of the
    workspace with room for the dS tiles (the dK/dV pass spills dS, the dQ pass is one GEMM)."""
    B, N, H, D = q.shape
    nbytes = (lib.fused_mha_backward_min_workspace_bytes if min_workspace else
              lib.fused_mha_backward_workspace_bytes)(B, H, N, D)
    ws = torch.empty(nbytes, dtype=torch.uint8, device=q.device)
    dq, dk, dv = torch.empty_like(q), torch.empty_like(q), torch.empty_like(q)
    s = torch.cuda.current_stream().cuda_stream if stream is None else stream
    if split:
        rc = lib.fused_mha_backward_delta(out.data_ptr(), dout.data_ptr(), lse.data_ptr(), ws.data_ptr(), nbytes, B, H, N, D, s)
        assert rc == OK, lib.fused_mha_error_string(rc)
        rc = lib.fused_mha_backward_dkdv(q.data_ptr(), k.data_ptr(), v.data_ptr(), dout.data_ptr(), lse.data_ptr(),
                                         ws.data_ptr(), nbytes, dk.data_ptr(), dv.data_ptr(), B, H, N, D, scale,
                                         int(causal), s)
        assert rc == OK, lib.fused_mha_error_string(rc)
        rc = lib.fused_mha_backward_dq(q.data_ptr(), k.data_ptr(), v.data_ptr(), dout.data_ptr(), lse.data_ptr(),
                                       ws.data_ptr(), nbytes, dq.data_ptr(), B, H, N, D, scale, int(causal), s)
    else:
        rc = lib.fused_mha_backward(q.data_ptr(), k.data_ptr(), v.data_ptr(), out.data_ptr(), dout.data_ptr(),
                                    lse.data_ptr(), ws.data_ptr(), nbytes, dq.data_ptr(), dk.data_ptr(),
                                    dv.data_ptr(), B, H, N, N, D, scale, int(causal), s)
    assert rc == OK, lib.fused_mha_error_string(rc)
    return dq, dk, dv, ws.view(torch.float32)[:B * H * N].view(B, H, N)


def backward_noalloc(lib, q, k, v, out, dout, lse, scale, causal, grads=None):
    """fused_mha_backward_noalloc; `grads` = preallocated (dq, dk, dv) or None to allocate them here."""
    B, N, H, D = q.shape
    dq, dk, dv = grads if grads is not None else (torch.empty_like(q), torch.empty_like(q), torch.empty_like(q))
    s = torch.cuda.current_stream().cuda_stream
    rc = lib.fused_mha_backward_noalloc(q.data_ptr(), k.data_ptr(), v.data_ptr(), out.data_ptr(), dout.data_ptr(),
                                        lse.data_ptr(), dq.data_ptr(), dk.data_ptr(), dv.data_ptr(), B, H, N, N, D,
                                        scale, int(causal), s)
    assert rc == OK, lib.fused_mha_error_string(rc)
    return dq, dk, dv


def forward_strided(lib, q, k, v, scale, causal):
    """q, k, v: fp16 device tensors (B, N, H, D) with any qualifying strides.  Returns dense (out, lse)."""
    B, N, H, D = q.shape
    out = torch.empty((B, N, H, D), dtype=q.dtype, device=q.device)
    lse = torch.empty((B, H, N), dtype=torch.float32, device=q.device)
    s = torch.cuda.current_stream().cuda_stream
    rc = lib.fused_mha_forward_strided(q.data_ptr(), Strides.of(q), k.data_ptr(), Strides.of(k), v.data_ptr(),
                                       Strides.of(v), out.data_ptr(), lse.data_ptr(), B, H, N, D, scale, int(causal), s)
    assert rc == OK, lib.fused_mha_error_string(rc)
    return out, lse


def backward_strided(lib, q, k, v, out, dout, lse, scale, causal):
    """q, k, v, dout with any qualifying strides; out, lse dense.  Returns dense (dq, dk, dv)."""
    B, N, H, D = q.shape
    nbytes = lib.fused_mha_backward_workspace_bytes(B, H, N, D)
    ws = torch.empty(nbytes, dtype=torch.uint8, device=q.device)
    dq, dk, dv = (torch.empty((B, N, H, D), dtype=q.dtype, device=q.device) for _ in range(3))
    s = torch.cuda.current_stream().cuda_stream
    rc = lib.fused_mha_backward_strided(q.data_ptr(), Strides.of(q), k.data_ptr(), Strides.of(k), v.data_ptr(),
                                        Strides.of(v), out.data_ptr(), dout.data_ptr(), Strides.of(dout),
                                        lse.data_ptr(), ws.data_ptr(), nbytes, dq.data_ptr(), dk.data_ptr(),
                                        dv.data_ptr(), B, H, N, D, scale, int(causal), s)
    assert rc == OK, lib.fused_mha_error_string(rc)
    return dq, dk, dv
