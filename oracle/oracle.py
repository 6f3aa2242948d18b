"""TEST INFRASTRUCTURE -- ctypes front end of the CPU oracle (oracle/liboracle.so).

Only tests, the smoke check and the benchmark's CPU-baseline leg import this
module.  Every function takes and returns CPU torch tensors (float32 or float64,
contiguous) and follows the reference function named in its docstring.
`ref_modules()` returns the reference's own compiled cpp/ extension when
oracle/_ref was built (make -C oracle), else None.
"""
import ctypes
import importlib.util
import os
import subprocess
import sysconfig

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB = None


def build(force=False):
    """Compile liboracle.so (and oracle/_ref when the reference tree is present)."""
    args = ["make", "-C", _HERE]
    if force:
        args.append("-B")
    subprocess.run(args, check=True, stdout=subprocess.DEVNULL)


def lib():
    global _LIB
    if _LIB is None:
        path = os.path.join(_HERE, "liboracle.so")
        if not os.path.exists(path):
            build()
        _LIB = ctypes.CDLL(path)
        _LIB.oracle_expand_coo.restype = ctypes.c_int
        _LIB.oracle_max_threads.restype = ctypes.c_int
    return _LIB


def set_threads(n):
    lib().oracle_set_threads(ctypes.c_int(int(n)))


def max_threads():
    return int(lib().oracle_max_threads())


def _sfx(t):
    if t.dtype == torch.float64:
        return "_f64"
    if t.dtype == torch.float32:
        return "_f32"
    raise TypeError("oracle supports float32/float64, got %s" % t.dtype)


def _p(t):
    assert t.device.type == "cpu" and t.is_contiguous()
    return ctypes.c_void_p(t.data_ptr())


def _L(x):
    return ctypes.c_long(int(x))


def dense_fwd(q, k):
    """cpp/l1attn_drv.cpp:13-55 -> attn [B,S,T,H]."""
    B, T, H, W = q.shape
    q, k = q.contiguous(), k.contiguous()
    attn = torch.empty(B, T, T, H, dtype=q.dtype)
    getattr(lib(), "oracle_dense_fwd" + _sfx(q))(_p(q), _p(k), _p(attn), _L(B), _L(T), _L(H), _L(W))
    return attn


def dense_bwd(d_attn, q, k):
    """cpp/l1attn_drv.cpp:57-98 -> (dq, dk)."""
    B, T, H, W = q.shape
    d_attn, q, k = d_attn.contiguous(), q.contiguous(), k.contiguous()
    dq, dk = torch.empty_like(q), torch.empty_like(k)
    getattr(lib(), "oracle_dense_bwd" + _sfx(q))(
        _p(d_attn), _p(q), _p(k), _p(dq), _p(dk), _L(B), _L(T), _L(H), _L(W))
    return dq, dk


def fused_fwd(q, k, v):
    """The composition the reference's model code builds on the dense operator
    (example-setfind/setfind.py:128-136; python/l1attn_sparse.py:488-506, testsparse.py:50-62):
    logits from dense_fwd (cpp/l1attn_drv.cpp:13-55), a row of zero logits appended along src,
    softmax over src, the no-op row dropped, einsum 'bsdh,bshw->bdhw' with v.
    -> (vo [B,T,H,Wv], lse [B,T,H] = log of the softmax denominator)."""
    B, T, H, W = q.shape
    a = dense_fwd(q, k)
    a = torch.cat((a, torch.zeros(B, 1, T, H, dtype=a.dtype)), 1)
    p = torch.softmax(a, 1)[:, :T]
    return torch.einsum("bsdh,bshw->bdhw", p, v), torch.logsumexp(a, 1)


def fused_bwd(dvo, q, k, v):
    """Backward of fused_fwd along the reference's own pieces: the softmax and einsum steps of
    example-setfind/setfind.py:128-136 differentiated by hand (softmax over src with the no-op row:
    dA = P * (dP - sum_s P * dP), the no-op row's share dropped with the row), then dq, dk from the reference's
    dense backward loop (cpp/l1attn_drv.cpp:57-98).  -> (dq, dk, dv)."""
    B, T, H, W = q.shape
    a = dense_fwd(q, k)
    a = torch.cat((a, torch.zeros(B, 1, T, H, dtype=a.dtype)), 1)
    p = torch.softmax(a, 1)[:, :T]                                   # [B,S,T,H]
    dp = torch.einsum("bdhw,bshw->bsdh", dvo, v)
    d_attn = p * (dp - (p * dp).sum(1, keepdim=True))
    dq, dk = dense_bwd(d_attn.contiguous(), q, k)
    return dq, dk, torch.einsum("bsdh,bdhw->bshw", p, dvo)


def _coo32(coo):
    coo = coo.to(torch.int32).contiguous()
    assert coo.dim() == 2 and coo.shape[1] >= 3
    return coo


def sparse_fwd(v, q, k, coo, dst_mxlen, use_softmax=True):
    """cpp/l1attn_sparse_drv.cpp:13-91 -> (vo, attn[B,T,dst_mxlen,H])."""
    B, T, H, W = q.shape
    v, q, k, coo = v.contiguous(), q.contiguous(), k.contiguous(), _coo32(coo)
    vo = torch.empty_like(q)
    attn = torch.empty(B, T, dst_mxlen, H, dtype=q.dtype)
    getattr(lib(), "oracle_sparse_fwd" + _sfx(q))(
        _p(v), _p(q), _p(k), _p(coo), _L(coo.shape[1]), _p(vo), _p(attn),
        _L(B), _L(T), _L(H), _L(W), _L(coo.shape[0]), _L(dst_mxlen), ctypes.c_int(bool(use_softmax)))
    return vo, attn


def sparse_bwd(dvo, v, q, k, coo, attn, dst_mxlen, use_softmax=True, jac_mode=0):
    """cpp/l1attn_sparse_drv.cpp:93-190 -> (dv, dq, dk).  jac_mode 1 = O(mx) closed form."""
    B, T, H, W = q.shape
    dvo, v, q, k, coo, attn = (dvo.contiguous(), v.contiguous(), q.contiguous(), k.contiguous(),
                               _coo32(coo), attn.contiguous())
    dv, dq, dk = torch.empty_like(q), torch.empty_like(q), torch.empty_like(q)
    scratch = torch.empty(2 * attn.numel(), dtype=q.dtype)
    getattr(lib(), "oracle_sparse_bwd" + _sfx(q))(
        _p(dvo), _p(v), _p(q), _p(k), _p(coo), _L(coo.shape[1]), _p(attn),
        _p(dv), _p(dq), _p(dk), _p(scratch),
        _L(B), _L(T), _L(H), _L(W), _L(coo.shape[0]), _L(dst_mxlen),
        ctypes.c_int(bool(use_softmax)), ctypes.c_int(int(jac_mode)))
    return dv, dq, dk


def bidi_fwd(vf, vb, q, k, coo, dst_mxlen, use_softmax=True):
    """cpp/l1attn_sparse_bidi_drv.cpp:15-101 -> (vo, attn)."""
    B, T, H, W = q.shape
    vf, vb, q, k, coo = vf.contiguous(), vb.contiguous(), q.contiguous(), k.contiguous(), _coo32(coo)
    vo = torch.empty_like(q)
    attn = torch.empty(B, T, dst_mxlen, H, dtype=q.dtype)
    getattr(lib(), "oracle_bidi_fwd" + _sfx(q))(
        _p(vf), _p(vb), _p(q), _p(k), _p(coo), _L(coo.shape[1]), _p(vo), _p(attn),
        _L(B), _L(T), _L(H), _L(W), _L(coo.shape[0]), _L(dst_mxlen), ctypes.c_int(bool(use_softmax)))
    return vo, attn


def bidi_bwd(dvo, vf, vb, q, k, coo, attn, dst_mxlen, use_softmax=True, jac_mode=0):
    """cpp/l1attn_sparse_bidi_drv.cpp:103-212 -> (dvf, dvb, dq, dk)."""
    B, T, H, W = q.shape
    dvo, vf, vb, q, k, coo, attn = (dvo.contiguous(), vf.contiguous(), vb.contiguous(), q.contiguous(),
                                    k.contiguous(), _coo32(coo), attn.contiguous())
    outs = [torch.empty_like(q) for _ in range(4)]
    scratch = torch.empty(2 * attn.numel(), dtype=q.dtype)
    getattr(lib(), "oracle_bidi_bwd" + _sfx(q))(
        _p(dvo), _p(vf), _p(vb), _p(q), _p(k), _p(coo), _L(coo.shape[1]), _p(attn),
        _p(outs[0]), _p(outs[1]), _p(outs[2]), _p(outs[3]), _p(scratch),
        _L(B), _L(T), _L(H), _L(W), _L(coo.shape[0]), _L(dst_mxlen),
        ctypes.c_int(bool(use_softmax)), ctypes.c_int(int(jac_mode)))
    return tuple(outs)


def expand_coo(co):
    """python/l1attn_sparse.py:382-427 -> (coo int32 [E,4], dst_mxlen, src_mxlen)."""
    co64 = co.to(torch.int64).contiguous().cpu()
    E = co64.shape[0]
    coo = torch.zeros(E, 4, dtype=torch.int32)
    mx = (ctypes.c_int * 2)()
    rc = lib().oracle_expand_coo(_p(co64), _L(E), _p(coo), mx)
    if rc != 0:
        raise ValueError("oracle_expand_coo: negative index")
    return coo, int(mx[0]), int(mx[1])


def ref_modules():
    """The reference's compiled cpp/ pybind modules (cpp/setup.py:9-11) from oracle/_ref,
    as a dict name -> module, or None when oracle/_ref was not built."""
    sfx = sysconfig.get_config_var("EXT_SUFFIX")
    mods = {}
    for name in ("l1attn_drv_cpp", "l1attn_sparse_drv", "l1attn_sparse_bidi_drv"):
        path = os.path.join(_HERE, "_ref", name + sfx)
        if not os.path.exists(path):
            return None
        spec = importlib.util.spec_from_file_location(name, path)
        mod = importlib.util.module_from_spec(spec)
        spec.loader.exec_module(mod)
        mods[name] = mod
    return mods
