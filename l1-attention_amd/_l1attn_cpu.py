"""ctypes binding of libl1attn_cpu.so: the stand-in for the reference's three CPU extension modules
l1attn_drv_cpp, l1attn_sparse_drv and l1attn_sparse_bidi_drv (cpp/setup.py:4-16; cpp/l1attn_drv.cpp:100-103,
cpp/l1attn_sparse_drv.cpp:192-195, cpp/l1attn_sparse_bidi_drv.cpp:214-217).

Same contract as those modules: the callee allocates and returns new tensors, inputs are borrowed and never
mutated.  For tensors in host memory only; float32 and float64 (the reference's CPU extension reads
float64 only, cpp/l1attn_drv.cpp:5).  Nothing on the GPU path imports this module, and this module never
touches a GPU tensor: it raises for one.
"""
import ctypes
import os

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libl1attn_cpu.so")
_lib = None

_ERR = {-1: "invalid argument", -4: "coo holds a token outside [0, n_tok) or a slot outside [0, dst_mxlen)"}
_c_p, _c_i64, _c_i = ctypes.c_void_p, ctypes.c_int64, ctypes.c_int


def lib():
    """Load the CPU library; raise when it is not built."""
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            raise RuntimeError("libl1attn_cpu.so is not built: run `python %s`" % os.path.join(_HERE, "build.py"))
        L = ctypes.CDLL(_LIB_PATH)
        L.l1attn_cpu_version.restype = _c_i
        L.l1attn_cpu_set_threads.restype = _c_i
        L.l1attn_cpu_set_threads.argtypes = [_c_i]
        L.l1attn_cpu_expand_coo.restype = _c_i
        L.l1attn_cpu_expand_coo.argtypes = [_c_p, _c_i, _c_i64, _c_i64, _c_p, _c_p]
        for sfx in ("f32", "f64"):
            for name, nptr, nint in (("dense_fwd", 3, 4), ("dense_bwd", 5, 4)):
                f = getattr(L, "l1attn_cpu_%s_%s" % (name, sfx))
                f.restype = _c_i
                f.argtypes = [_c_p] * nptr + [_c_i64] * nint
            for name, npre, npost in (("sparse_fwd", 4, 2), ("sparse_bidi_fwd", 5, 2),
                                      ("sparse_bwd", 5, 4), ("sparse_bidi_bwd", 6, 5)):
                f = getattr(L, "l1attn_cpu_%s_%s" % (name, sfx))
                f.restype = _c_i
                # tensors, coo + its stride, more tensors, B T H W Wv E dst_mxlen, use_softmax
                f.argtypes = [_c_p] * npre + [_c_i64] + [_c_p] * npost + [_c_i64] * 7 + [_c_i]
                if name.endswith("_fwd"):
                    f.argtypes = f.argtypes + [_c_i]  # attn_zeroed
            f = getattr(L, "l1attn_cpu_fused_fwd_" + sfx)
            f.restype = _c_i
            f.argtypes = [_c_p] * 5 + [_c_i64] * 5
            f = getattr(L, "l1attn_cpu_fused_bwd_" + sfx)
            f.restype = _c_i
            f.argtypes = [_c_p] * 9 + [_c_i64] * 5
        _lib = L
    return _lib


def set_threads(n):
    """Threads used by the CPU operators (0: the OpenMP default); returns the previous setting."""
    return int(lib().l1attn_cpu_set_threads(int(n)))


def _check(rc, what):
    if rc != 0:
        raise RuntimeError("%s: %s (code %d)" % (what, _ERR.get(rc, "error"), rc))


def _check_input(x, name):
    if x.device.type != "cpu":
        raise RuntimeError("%s must be a CPU tensor" % name)
    if not x.is_contiguous():
        raise RuntimeError("%s must be contiguous" % name)


def _sfx(x, name="q"):
    if x.dtype == torch.float32:
        return "f32"
    if x.dtype == torch.float64:
        return "f64"
    raise RuntimeError("%s: only float32 and float64 are implemented, got %s" % (name, x.dtype))


def _p(x):
    return _c_p(x.data_ptr())


def _dense_shapes(q, k):
    if q.dim() != 4 or q.shape != k.shape or q.dtype != k.dtype:
        raise RuntimeError("q and k must be [batch, n_ctx, n_heads, width] tensors of one shape and dtype")
    return q.shape


def dense_forward(q, k):
    """l1attn_drv_cpp.forward(q, k) -> [attn]  (cpp/l1attn_drv.cpp:13-55)."""
    _check_input(q, "q")
    _check_input(k, "k")
    B, T, H, W = _dense_shapes(q, k)
    sfx = _sfx(q)
    attn = torch.empty((B, T, T, H), dtype=q.dtype)
    _check(getattr(lib(), "l1attn_cpu_dense_fwd_" + sfx)(_p(q), _p(k), _p(attn), B, T, H, W), "l1attn_cpu_dense_fwd_" + sfx)
    return [attn]


def dense_backward(d_attn, q, k):
    """l1attn_drv_cpp.backward(d_attn, q, k) -> [d_q, d_k]  (cpp/l1attn_drv.cpp:57-98)."""
    for x, n in ((d_attn, "d_attn"), (q, "q"), (k, "k")):
        _check_input(x, n)
    B, T, H, W = _dense_shapes(q, k)
    if tuple(d_attn.shape) != (B, T, T, H) or d_attn.dtype != q.dtype:
        raise RuntimeError("d_attn must be [batch, n_ctx, n_ctx, n_heads] with the dtype of q")
    sfx = _sfx(q)
    dq, dk = torch.empty_like(q), torch.empty_like(k)
    _check(getattr(lib(), "l1attn_cpu_dense_bwd_" + sfx)(_p(d_attn), _p(q), _p(k), _p(dq), _p(dk), B, T, H, W),
           "l1attn_cpu_dense_bwd_" + sfx)
    return [dq, dk]


def expand_coo(co):
    """expandCoo (cpp/l1attn_sparse_cpp.py:61-106): co [cl,2] integer [dst,src] rows ->
    (coo int32 [cl,4] on the CPU, dst_mxlen, src_mxlen)."""
    if co.dim() != 2 or co.shape[1] < 2:
        raise RuntimeError("co must be [cl, 2] rows of [dst, src]")
    if co.dtype not in (torch.int8, torch.uint8, torch.int16, torch.int32, torch.int64):
        raise RuntimeError("co must hold integers, got %s" % co.dtype)
    if co.device.type != "cpu":
        raise RuntimeError("co must be a CPU tensor")
    c = co if co.dtype in (torch.int32, torch.int64) else co.to(torch.int64)
    c = c.contiguous()
    E = c.shape[0]
    coo = torch.zeros((E, 4), dtype=torch.int32)
    mx = (ctypes.c_int32 * 2)()
    _check(lib().l1attn_cpu_expand_coo(_p(c), 64 if c.dtype == torch.int64 else 32, c.shape[1], E, _p(coo), mx),
           "l1attn_cpu_expand_coo")
    return coo, int(mx[0]), int(mx[1])


def _sparse_shapes(v, q, k, coo):
    if q.dim() != 4 or q.shape != k.shape or v.dim() != 4 or v.shape[:3] != q.shape[:3]:
        raise RuntimeError("v, q, k must be [batch, n_tok, n_heads, width] tensors with equal leading dims")
    if not (v.dtype == q.dtype == k.dtype):
        raise RuntimeError("v, q, k must share a dtype")
    if coo.dtype != torch.int32 or coo.dim() != 2 or coo.shape[1] < 3:
        raise RuntimeError("coo must be an int32 [cl, >=3] tensor (the output of expandCoo)")
    B, T, H, W = q.shape
    return B, T, H, W, v.shape[3], coo.shape[0]


def _zero_pages(shape, dtype):
    """A zero tensor whose pages the allocator has not touched yet (numpy's zeros is calloc): the padded
    edge-weight tensor is mostly empty slots on skewed graphs, and the library writes the slots of edges only."""
    import numpy as np
    return torch.from_numpy(np.zeros(shape, dtype=np.float32 if dtype == torch.float32 else np.float64))


def _same_as(x, like, name, like_name):
    if x.shape != like.shape or x.dtype != like.dtype:
        raise RuntimeError("%s must have the shape and dtype of %s" % (name, like_name))


def sparse_forward(v, q, k, coo, dst_mxlen, use_softmax):
    """l1attn_sparse_drv.forward(v,q,k,coo,dst_mxlen,use_softmax) -> [vo, attn]  (cpp/l1attn_sparse_drv.cpp:13-91);
    attn is the padded [batch, n_tok, dst_mxlen, n_heads] tensor of edge weights, as there."""
    for x, n in ((v, "v"), (q, "q"), (k, "k"), (coo, "coo")):
        _check_input(x, n)
    B, T, H, W, Wv, E = _sparse_shapes(v, q, k, coo)
    M = int(dst_mxlen)
    sfx = _sfx(q)
    vo = torch.empty_like(v)
    attn = _zero_pages((B, T, M, H), q.dtype)
    _check(getattr(lib(), "l1attn_cpu_sparse_fwd_" + sfx)(
        _p(v), _p(q), _p(k), _p(coo), coo.shape[1], _p(vo), _p(attn), B, T, H, W, Wv, E, M, int(bool(use_softmax)), 1),
        "l1attn_cpu_sparse_fwd_" + sfx)
    return [vo, attn]


def sparse_backward(dvo, v, q, k, coo, attn, dst_mxlen, use_softmax):
    """l1attn_sparse_drv.backward(dvo,v,q,k,coo,attn,dst_mxlen,use_softmax) -> [dv,dq,dk]
    (cpp/l1attn_sparse_drv.cpp:93-190)."""
    for x, n in ((dvo, "dvo"), (v, "v"), (q, "q"), (k, "k"), (coo, "coo"), (attn, "attn")):
        _check_input(x, n)
    B, T, H, W, Wv, E = _sparse_shapes(v, q, k, coo)
    M = int(dst_mxlen)
    _same_as(dvo, v, "dvo", "v")
    if tuple(attn.shape) != (B, T, M, H) or attn.dtype != q.dtype:
        raise RuntimeError("attn must be the [batch, n_tok, dst_mxlen, n_heads] tensor the forward returned")
    sfx = _sfx(q)
    dv, dq, dk = torch.empty_like(v), torch.empty_like(q), torch.empty_like(k)
    _check(getattr(lib(), "l1attn_cpu_sparse_bwd_" + sfx)(
        _p(dvo), _p(v), _p(q), _p(k), _p(coo), coo.shape[1], _p(attn), _p(dv), _p(dq), _p(dk),
        B, T, H, W, Wv, E, M, int(bool(use_softmax))), "l1attn_cpu_sparse_bwd_" + sfx)
    return [dv, dq, dk]


def bidi_forward(vf, vb, q, k, coo, dst_mxlen, use_softmax):
    """l1attn_sparse_bidi_drv.forward -> [vo, attn]  (cpp/l1attn_sparse_bidi_drv.cpp:15-100)."""
    for x, n in ((vf, "vf"), (vb, "vb"), (q, "q"), (k, "k"), (coo, "coo")):
        _check_input(x, n)
    B, T, H, W, Wv, E = _sparse_shapes(vf, q, k, coo)
    _same_as(vb, vf, "vb", "vf")
    M = int(dst_mxlen)
    sfx = _sfx(q)
    vo = torch.empty_like(vf)
    attn = _zero_pages((B, T, M, H), q.dtype)
    _check(getattr(lib(), "l1attn_cpu_sparse_bidi_fwd_" + sfx)(
        _p(vf), _p(vb), _p(q), _p(k), _p(coo), coo.shape[1], _p(vo), _p(attn), B, T, H, W, Wv, E, M,
        int(bool(use_softmax)), 1), "l1attn_cpu_sparse_bidi_fwd_" + sfx)
    return [vo, attn]


def bidi_backward(dvo, vf, vb, q, k, coo, attn, dst_mxlen, use_softmax):
    """l1attn_sparse_bidi_drv.backward -> [dvf,dvb,dq,dk]  (cpp/l1attn_sparse_bidi_drv.cpp:102-212)."""
    for x, n in ((dvo, "dvo"), (vf, "vf"), (vb, "vb"), (q, "q"), (k, "k"), (coo, "coo"), (attn, "attn")):
        _check_input(x, n)
    B, T, H, W, Wv, E = _sparse_shapes(vf, q, k, coo)
    _same_as(vb, vf, "vb", "vf")
    _same_as(dvo, vf, "dvo", "vf")
    M = int(dst_mxlen)
    if tuple(attn.shape) != (B, T, M, H) or attn.dtype != q.dtype:
        raise RuntimeError("attn must be the [batch, n_tok, dst_mxlen, n_heads] tensor the forward returned")
    sfx = _sfx(q)
    dvf, dvb, dq, dk = torch.empty_like(vf), torch.empty_like(vb), torch.empty_like(q), torch.empty_like(k)
    _check(getattr(lib(), "l1attn_cpu_sparse_bidi_bwd_" + sfx)(
        _p(dvo), _p(vf), _p(vb), _p(q), _p(k), _p(coo), coo.shape[1], _p(attn), _p(dvf), _p(dvb), _p(dq), _p(dk),
        B, T, H, W, Wv, E, M, int(bool(use_softmax))), "l1attn_cpu_sparse_bidi_bwd_" + sfx)
    return [dvf, dvb, dq, dk]


def fused_forward(q, k, v):
    """Fused operator, forward -> [vo, lse]: softmax over src of the L1 logits with the no-op zero logit, times v,
    without the [B,T,T,H] logits (example-setfind/setfind.py:128-136 in one call)."""
    for x, n in ((q, "q"), (k, "k"), (v, "v")):
        _check_input(x, n)
    B, T, H, W = _dense_shapes(q, k)
    if v.dim() != 4 or v.shape[:3] != q.shape[:3] or v.dtype != q.dtype:
        raise RuntimeError("v must be [batch, n_ctx, n_heads, value width] with the dtype of q")
    sfx = _sfx(q)
    vo = torch.empty_like(v)
    lse = torch.empty((B, T, H), dtype=q.dtype)
    _check(getattr(lib(), "l1attn_cpu_fused_fwd_" + sfx)(_p(q), _p(k), _p(v), _p(vo), _p(lse), B, T, H, W, v.shape[3]),
           "l1attn_cpu_fused_fwd_" + sfx)
    return [vo, lse]


def fused_backward(dvo, q, k, v, vo, lse):
    """Backward of fused_forward -> [dq, dk, dv]."""
    for x, n in ((dvo, "dvo"), (q, "q"), (k, "k"), (v, "v"), (vo, "vo"), (lse, "lse")):
        _check_input(x, n)
    B, T, H, W = _dense_shapes(q, k)
    _same_as(dvo, v, "dvo", "v")
    _same_as(vo, v, "vo", "v")
    if v.dtype != q.dtype or tuple(lse.shape) != (B, T, H) or lse.dtype != q.dtype:
        raise RuntimeError("v must have the dtype of q, and lse must be the [batch, n_ctx, n_heads] tensor the forward returned")
    sfx = _sfx(q)
    dq, dk, dv = torch.empty_like(q), torch.empty_like(k), torch.empty_like(v)
    _check(getattr(lib(), "l1attn_cpu_fused_bwd_" + sfx)(
        _p(dvo), _p(q), _p(k), _p(v), _p(vo), _p(lse), _p(dq), _p(dk), _p(dv), B, T, H, W, v.shape[3]),
        "l1attn_cpu_fused_bwd_" + sfx)
    return [dq, dk, dv]
