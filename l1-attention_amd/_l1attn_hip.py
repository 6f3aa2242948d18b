"""ctypes binding of libl1attn_hip.so: the stand-in for the reference's pybind11 driver modules
l1attn_cuda_drv, l1attn_sparse_cuda_drv and l1attn_sparse_bidi_cuda_drv
(cuda/l1attn_cuda_drv.cpp:106-109, cuda/l1attn_sparse_cuda_drv.cpp:71-74,
cuda/l1attn_sparse_bidi_cuda_drv.cpp:77-80).

Same contract as those drivers: the callee allocates and returns new tensors, inputs are
borrowed and never mutated, and the input checks raise RuntimeError with the driver's wording
("q must be a CUDA tensor", "q must be contiguous").  PyTorch is used for device memory and
the current stream only; every computation happens in the HIP library.  There is no CPU or
eager fallback: a missing library raises at import of the first operator.
"""
import ctypes
import math
import os

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libl1attn_hip.so")
_lib = None

_ERR = {-1: "invalid argument", -2: "workspace missing or too small",
        -3: "size out of range", -4: "edge list index outside [0, n_tok)"}

_c_p = ctypes.c_void_p
_c_i64 = ctypes.c_int64
_c_sz = ctypes.c_size_t


def lib():
    """Load the HIP library; raise (never fall back) when it is not built."""
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            raise RuntimeError(
                "libl1attn_hip.so is not built: run `python %s`" % os.path.join(_HERE, "build.py"))
        L = ctypes.CDLL(_LIB_PATH)
        L.l1attn_version.restype = ctypes.c_int
        L.l1attn_dense_bwd_workspace_bytes.restype = _c_sz
        L.l1attn_dense_bwd_workspace_bytes.argtypes = [_c_i64] * 4
        for sfx in ("f32", "f64"):
            f = getattr(L, "l1attn_dense_fwd_" + sfx)
            f.restype = ctypes.c_int
            f.argtypes = [_c_p, _c_p, _c_p, _c_i64, _c_i64, _c_i64, _c_i64, _c_p]
            f = getattr(L, "l1attn_dense_bwd_" + sfx)
            f.restype = ctypes.c_int
            f.argtypes = [_c_p] * 5 + [_c_i64] * 4 + [_c_p, _c_sz, _c_p]
        _lib = L
    return _lib


def check(rc, what):
    if rc == 0:
        return
    if rc < 0:
        raise RuntimeError("%s: %s (code %d)" % (what, _ERR.get(rc, "error"), rc))
    raise RuntimeError("%s: HIP error %d" % (what, rc))


def check_input(x, name):
    # CHECK_INPUT of the reference drivers (cuda/l1attn_cuda_drv.cpp:38-40)
    if not x.is_cuda:
        raise RuntimeError("%s must be a CUDA tensor" % name)
    if not x.is_contiguous():
        raise RuntimeError("%s must be contiguous" % name)


def sfx_of(x, name="q"):
    if x.dtype == torch.float32:
        return "f32"
    if x.dtype == torch.float64:
        return "f64"
    raise RuntimeError("%s: only float32 and float64 are implemented, got %s" % (name, x.dtype))


def stream_of(x):
    return _c_p(torch.cuda.current_stream(x.device).cuda_stream)


def ptr(x):
    return _c_p(x.data_ptr())


# ------------------------------------------------------------------------------------ dense

def dense_forward(q, k):
    """l1attn_cuda_drv.forward(q, k) -> [attn]  (cuda/l1attn_cuda_drv.cpp:42-65)."""
    check_input(q, "q")
    check_input(k, "k")
    if q.dim() != 4 or q.shape != k.shape or q.dtype != k.dtype or q.device != k.device:
        raise RuntimeError("q and k must be [batch, n_ctx, n_heads, width] tensors of one shape, dtype and device")
    B, T, H, W = q.shape
    sfx = sfx_of(q)
    attn = torch.empty((B, T, T, H), dtype=q.dtype, device=q.device)
    with torch.cuda.device(q.device):
        rc = getattr(lib(), "l1attn_dense_fwd_" + sfx)(ptr(q), ptr(k), ptr(attn), B, T, H, W, stream_of(q))
    check(rc, "l1attn_dense_fwd_" + sfx)
    return [attn]


def dense_backward(d_attn, q, k):
    """l1attn_cuda_drv.backward(d_attn, q, k) -> [d_q, d_k]  (cuda/l1attn_cuda_drv.cpp:67-104)."""
    check_input(d_attn, "d_attn")
    check_input(q, "q")
    check_input(k, "k")
    B, T, H, W = q.shape
    if tuple(d_attn.shape) != (B, T, T, H) or d_attn.dtype != q.dtype:
        raise RuntimeError("d_attn must be [batch, n_ctx, n_ctx, n_heads] with the dtype of q")
    sfx = sfx_of(q)
    dq = torch.empty_like(q)
    dk = torch.empty_like(k)
    L = lib()
    with torch.cuda.device(q.device):
        ws_bytes = L.l1attn_dense_bwd_workspace_bytes(B, T, H, W) if sfx == "f32" else 0
        ws = torch.empty(ws_bytes, dtype=torch.uint8, device=q.device) if ws_bytes else None
        rc = getattr(L, "l1attn_dense_bwd_" + sfx)(
            ptr(d_attn), ptr(q), ptr(k), ptr(dq), ptr(dk), B, T, H, W,
            ptr(ws) if ws is not None else None, ws_bytes, stream_of(q))
    check(rc, "l1attn_dense_bwd_" + sfx)
    return [dq, dk]
