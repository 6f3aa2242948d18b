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

# Code paths whose kernels have not passed their GPU tests yet.  A public operator never reaches them unless the
# caller asks by name: enable_experimental("rows16") or L1ATTN_EXPERIMENTAL=rows16,fused,fixed in the environment.
#   rows16  float16 / bfloat16 rows in the sparse operators
#   fused   l1attn_cuda.L1AttnFused (dense_fused_forward / dense_fused_backward)
#   fixed   dense_forward_fixed (fixed-point float32 forward)
#   bwd_pipe    set_dense_backward_form(loop_form=1 or 2): pipelined step loops of the long-sequence dense backward
#   rank_merge  set_dense_backward_form(rank_sort=1): column ranks from the library's own merge sort
EXPERIMENTAL = ("rows16", "fused", "fixed", "bwd_pipe", "rank_merge")
_enabled = set(n for n in os.environ.get("L1ATTN_EXPERIMENTAL", "").replace(" ", "").split(",") if n)


def enable_experimental(*names):
    """Opt in to code paths that are built but not yet validated on a GPU; returns the enabled set."""
    for n in names:
        if n not in EXPERIMENTAL:
            raise ValueError("unknown experimental path %r (known: %s)" % (n, ", ".join(EXPERIMENTAL)))
        _enabled.add(n)
    return frozenset(_enabled)


def _require_experimental(name, what):
    if name not in _enabled:
        raise RuntimeError(
            "%s is experimental: its kernels have not passed their GPU tests yet.  Opt in with "
            "_l1attn_hip.enable_experimental(%r) or L1ATTN_EXPERIMENTAL=%s" % (what, name, name))


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
        L.l1attn_probe_valu.restype = ctypes.c_int
        L.l1attn_probe_valu.argtypes = [_c_p, _c_i64, _c_i64, _c_p]
        L.l1attn_probe_valu_op.restype = ctypes.c_int
        L.l1attn_probe_valu_op.argtypes = [_c_p, _c_i64, _c_i64, ctypes.c_int, _c_p]
        L.l1attn_dense_fwd_workspace_bytes.restype = _c_sz
        L.l1attn_dense_fwd_workspace_bytes.argtypes = [_c_i64] * 4
        L.l1attn_dense_fwd_ws_f32.restype = ctypes.c_int
        L.l1attn_dense_fwd_ws_f32.argtypes = [_c_p, _c_p, _c_p, _c_i64, _c_i64, _c_i64, _c_i64, _c_p, _c_sz, _c_p]
        L.l1attn_dense_fwd_fixed_workspace_bytes.restype = _c_sz
        L.l1attn_dense_fwd_fixed_workspace_bytes.argtypes = [_c_i64] * 4
        L.l1attn_dense_fwd_fixed_f32.restype = ctypes.c_int
        L.l1attn_dense_fwd_fixed_f32.argtypes = [_c_p, _c_p, _c_p, _c_i64, _c_i64, _c_i64, _c_i64, _c_p, _c_sz, _c_p]
        L.l1attn_dense_bwd_workspace_bytes.restype = _c_sz
        L.l1attn_dense_bwd_workspace_bytes.argtypes = [_c_i64] * 4
        L.l1attn_dense_bwd_plan_info.restype = ctypes.c_int
        L.l1attn_dense_bwd_plan_info.argtypes = [_c_i64] * 4 + [_c_p]
        L.l1attn_dense_bwd_plan_info_ex.restype = ctypes.c_int
        L.l1attn_dense_bwd_plan_info_ex.argtypes = [_c_i64] * 4 + [ctypes.c_int, _c_p]
        L.l1attn_dense_bwd_ex_f32.restype = ctypes.c_int
        L.l1attn_dense_bwd_ex_f32.argtypes = [_c_p] * 5 + [_c_i64] * 4 + [ctypes.c_int] * 3 + [_c_p, _c_sz, _c_p]
        for sfx in ("f32", "f64"):
            f = getattr(L, "l1attn_dense_fwd_" + sfx)
            f.restype = ctypes.c_int
            f.argtypes = [_c_p, _c_p, _c_p, _c_i64, _c_i64, _c_i64, _c_i64, _c_p]
            f = getattr(L, "l1attn_dense_bwd_" + sfx)
            f.restype = ctypes.c_int
            f.argtypes = [_c_p] * 5 + [_c_i64] * 4 + [_c_p, _c_sz, _c_p]
        _c_i = ctypes.c_int
        for sfx in ("f32", "f64"):
            f = getattr(L, "l1attn_fused_fwd_" + sfx)
            f.restype = _c_i
            f.argtypes = [_c_p] * 5 + [_c_i64] * 5 + [_c_p]
            if sfx == "f32":
                L.l1attn_fused_fwd_pipe_f32.restype = _c_i
                L.l1attn_fused_fwd_pipe_f32.argtypes = f.argtypes
            f = getattr(L, "l1attn_fused_bwd_stage_" + sfx)
            f.restype = _c_i
            f.argtypes = [_c_p] * 8 + [_c_i64] * 5 + [_c_p]
            if sfx == "f32":
                L.l1attn_fused_bwd_stage_pipe_f32.restype = _c_i
                L.l1attn_fused_bwd_stage_pipe_f32.argtypes = f.argtypes
        L.l1attn_dense_column_ranks_f32.restype = _c_i
        L.l1attn_dense_column_ranks_f32.argtypes = [_c_p] * 4 + [_c_i64] * 4 + [_c_p]
        L.l1attn_dense_column_ranks_merge_f32.restype = _c_i
        L.l1attn_dense_column_ranks_merge_f32.argtypes = [_c_p] * 4 + [_c_i64] * 4 + [_c_p]
        L.l1attn_expand_coo_workspace_bytes.restype = _c_sz
        L.l1attn_expand_coo_workspace_bytes.argtypes = [_c_i64]
        L.l1attn_expand_coo.restype = _c_i
        L.l1attn_expand_coo.argtypes = [_c_p, _c_i, _c_i64, _c_i64, _c_p, _c_p, _c_p, _c_sz, _c_p]
        for n in ("l1attn_sparse_plan_bytes", "l1attn_sparse_plan_workspace_bytes"):
            getattr(L, n).restype = _c_sz
            getattr(L, n).argtypes = [_c_i64, _c_i64]
        L.l1attn_sparse_plan_build.restype = _c_i
        L.l1attn_sparse_plan_build.argtypes = [_c_p, _c_i64, _c_i64, _c_i64, _c_p, _c_sz, _c_p, _c_sz, _c_p]
        L.l1attn_sparse_plan_check.restype = _c_i
        L.l1attn_sparse_plan_check.argtypes = [_c_p, _c_i64, _c_i64, _c_p, _c_p]
        dims = [_c_i64] * 6 + [_c_i, _c_p]
        for sfx in ("f32", "f64"):
            for name, nptr in (("l1attn_sparse_fwd_", 6), ("l1attn_sparse_bwd_", 10),
                               ("l1attn_sparse_bidi_fwd_", 7), ("l1attn_sparse_bidi_bwd_", 12)):
                f = getattr(L, name + sfx)
                f.restype = _c_i
                f.argtypes = [_c_p] * nptr + dims
        for sfx in ("f16", "bf16"):  # 16-bit rows, fp32 sums and edge weights
            for name, nptr in (("l1attn_sparse_fwd_", 6), ("l1attn_sparse_bidi_fwd_", 7),
                               ("l1attn_sparse_bwd_", 10), ("l1attn_sparse_bidi_bwd_", 12)):
                f = getattr(L, name + sfx)
                f.restype = _c_i
                f.argtypes = [_c_p] * nptr + dims
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


def sfx_fwd_sparse(x, name="q"):
    """Entry-point suffix and edge-weight dtype of the sparse operators.  They also take 16-bit rows
    (the reference dispatches Half in its forwards: cuda/l1attn_sparse_cuda_kernel.cu:405-435, :684-714);
    the weights of a 16-bit call are fp32."""
    if x.dtype in (torch.float16, torch.bfloat16):
        _require_experimental("rows16", "float16/bfloat16 rows in the sparse operators")
        return ("f16" if x.dtype == torch.float16 else "bf16"), torch.float32
    return sfx_of(x, name), x.dtype


def sfx_bwd_sparse(x):
    """Entry-point suffix of the sparse backwards.  The reference's exist for float32 and float64 only
    (AT_DISPATCH_FLOATING_TYPES, cuda/l1attn_sparse_cuda_kernel.cu:483-519, :765-803); the 16-bit ones here are
    an addition: gradients in the rows' type, sums and edge weights in fp32."""
    return sfx_fwd_sparse(x)[0]


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
    L = lib()
    with torch.cuda.device(q.device):
        ws_bytes = L.l1attn_dense_fwd_workspace_bytes(B, T, H, W) if sfx == "f32" else 0
        if ws_bytes:
            ws = torch.empty(ws_bytes, dtype=torch.uint8, device=q.device)
            rc = L.l1attn_dense_fwd_ws_f32(ptr(q), ptr(k), ptr(attn), B, T, H, W, ptr(ws), ws_bytes, stream_of(q))
        else:
            rc = getattr(L, "l1attn_dense_fwd_" + sfx)(ptr(q), ptr(k), ptr(attn), B, T, H, W, stream_of(q))
    check(rc, "l1attn_dense_fwd_" + sfx)
    return [attn]


def dense_forward_fixed(q, k):
    """Experimental float32 forward on fixed point (one v_sad_u32 per pair-element; inputs rounded to a
    per-head grid of 2^-24 of the head's largest magnitude).  Same contract as dense_forward; widths 32 and
    64 only.  Not used by L1AttnFn."""
    _require_experimental("fixed", "the fixed-point forward")
    check_input(q, "q")
    check_input(k, "k")
    if q.dim() != 4 or q.shape != k.shape or q.dtype != torch.float32 or k.dtype != torch.float32 or q.device != k.device:
        raise RuntimeError("q and k must be float32 [batch, n_ctx, n_heads, width] tensors of one shape and device")
    B, T, H, W = q.shape
    attn = torch.empty((B, T, T, H), dtype=q.dtype, device=q.device)
    L = lib()
    with torch.cuda.device(q.device):
        ws_bytes = L.l1attn_dense_fwd_fixed_workspace_bytes(B, T, H, W)
        ws = torch.empty(max(ws_bytes, 16), dtype=torch.uint8, device=q.device)
        rc = L.l1attn_dense_fwd_fixed_f32(ptr(q), ptr(k), ptr(attn), B, T, H, W, ptr(ws), ws_bytes, stream_of(q))
    check(rc, "l1attn_dense_fwd_fixed_f32")
    return [attn]


_dense_bwd_form = (0, 0)  # (loop_form, rank_sort) of l1attn_dense_bwd_ex_f32; (0, 0) is l1attn_dense_bwd_f32
_assume_sign_range = False


def assume_sign_range(flag=True):
    """flag=True: from now on the caller vouches that q and k handed to the float32 dense backward hold magnitudes
    below 2^63 and no non-zero magnitude below 2^-41 (ordinary activations do); the tiled backward then leaves out its
    range check, which saves a read of q and k per call (about 20/T of the call: it matters below a few hundred
    tokens).  Outside the vouched range sign(q-k) is replaced by clamp((q-k)*2^64, -1, 1).  Returns the previous
    setting; the default, False, is exact for every input."""
    global _assume_sign_range
    old, _assume_sign_range = _assume_sign_range, bool(flag)
    return old


def set_dense_backward_form(loop_form=0, rank_sort=0):
    """Which form of the float32 long-sequence backward dense_backward() runs from now on; returns the previous
    (loop_form, rank_sort).  (0, 0) is the default entry point.  loop_form 1 / 2 (pipelined step loops) need
    enable_experimental("bwd_pipe"), rank_sort 1 (merge sort for the column ranks) needs "rank_merge": those
    kernels have not passed their GPU tests yet.  All forms give bit-identical gradients."""
    global _dense_bwd_form
    if loop_form not in (0, 1, 2) or rank_sort not in (0, 1):
        raise ValueError("loop_form must be 0, 1 or 2 and rank_sort 0 or 1, got %r, %r" % (loop_form, rank_sort))
    if loop_form:
        _require_experimental("bwd_pipe", "the pipelined step loop of the dense backward")
    if rank_sort:
        _require_experimental("rank_merge", "the merge sort for the dense backward's column ranks")
    old, _dense_bwd_form = _dense_bwd_form, (int(loop_form), int(rank_sort))
    if _dense_bwd_form != (0, 0) and _dense_bwd_form != old:
        import warnings
        warnings.warn("l1attn: the float32 dense backward now runs loop_form=%d, rank_sort=%d "
                      "(l1attn_dense_bwd_ex_f32), kernels that have not passed their GPU tests yet" % _dense_bwd_form,
                      RuntimeWarning, stacklevel=2)
    return old


def dense_backward_plan(B, T, H, W, loop_form=None):
    """l1attn_dense_bwd_plan_info_ex as a list of 16 ints, for the form dense_backward() currently runs."""
    info = (ctypes.c_int64 * 16)()
    form = _dense_bwd_form[0] if loop_form is None else int(loop_form)
    check(lib().l1attn_dense_bwd_plan_info_ex(B, T, H, W, form, info), "l1attn_dense_bwd_plan_info_ex")
    return list(info)


def dense_backward(d_attn, q, k):
    """l1attn_cuda_drv.backward(d_attn, q, k) -> [d_q, d_k]  (cuda/l1attn_cuda_drv.cpp:67-104)."""
    check_input(d_attn, "d_attn")
    check_input(q, "q")
    check_input(k, "k")
    if q.dim() != 4 or q.shape != k.shape or q.dtype != k.dtype or q.device != k.device:
        raise RuntimeError("q and k must be [batch, n_ctx, n_heads, width] tensors of one shape, dtype and device")
    B, T, H, W = q.shape
    if tuple(d_attn.shape) != (B, T, T, H) or d_attn.dtype != q.dtype or d_attn.device != q.device:
        raise RuntimeError("d_attn must be [batch, n_ctx, n_ctx, n_heads] with the dtype and device of q")
    sfx = sfx_of(q)
    dq = torch.empty_like(q)
    dk = torch.empty_like(k)
    L = lib()
    with torch.cuda.device(q.device):
        ws_bytes = L.l1attn_dense_bwd_workspace_bytes(B, T, H, W) if sfx == "f32" else 0
        ws = torch.empty(ws_bytes, dtype=torch.uint8, device=q.device) if ws_bytes else None
        wsp = ptr(ws) if ws is not None else None
        if sfx == "f32" and (_dense_bwd_form != (0, 0) or _assume_sign_range):
            rc = L.l1attn_dense_bwd_ex_f32(ptr(d_attn), ptr(q), ptr(k), ptr(dq), ptr(dk), B, T, H, W,
                                           _dense_bwd_form[0], _dense_bwd_form[1], int(_assume_sign_range),
                                           wsp, ws_bytes, stream_of(q))
        else:
            rc = getattr(L, "l1attn_dense_bwd_" + sfx)(
                ptr(d_attn), ptr(q), ptr(k), ptr(dq), ptr(dk), B, T, H, W, wsp, ws_bytes, stream_of(q))
    check(rc, "l1attn_dense_bwd_" + sfx)
    return [dq, dk]


def dense_fused_forward(q, k, v, want_lse=False, pipelined=False):
    """Fused forward: vo[b,t,h,:] = sum_s p[s] * v[b,s,h,:] with p the softmax over src of the L1 logits
    and a no-op zero logit (1 + sum in the denominator), without materialising the [B,T,T,H] logits.
    What example-setfind/setfind.py:128-136 composes from L1Attn, softmax and einsum.
    Returns [vo, lse]; lse [B,T,H] = log(1 + sum_s exp(a)) if want_lse else None.
    pipelined (float32 only): the entry whose kernels stream k and v through a software pipeline of scalar loads;
    same results bit for bit."""
    _require_experimental("fused", "the fused L1 attention operator")
    for x, n in ((q, "q"), (k, "k"), (v, "v")):
        check_input(x, n)
    if q.dim() != 4 or q.shape != k.shape or v.dim() != 4 or v.shape[:3] != q.shape[:3]:
        raise RuntimeError("q, k, v must be [batch, n_ctx, n_heads, width] tensors with equal leading dims")
    if not (v.dtype == q.dtype == k.dtype) or not (v.device == q.device == k.device):
        raise RuntimeError("q, k, v must share dtype and device")
    B, T, H, W = q.shape
    Wv = v.shape[3]
    sfx = sfx_of(q)
    vo = torch.empty_like(v)
    lse = torch.empty((B, T, H), dtype=q.dtype, device=q.device) if want_lse else None
    with torch.cuda.device(q.device):
        name = "l1attn_fused_fwd_pipe_f32" if (pipelined and sfx == "f32") else "l1attn_fused_fwd_" + sfx
        rc = getattr(lib(), name)(
            ptr(q), ptr(k), ptr(v), ptr(vo), ptr(lse) if lse is not None else None, B, T, H, W, Wv, stream_of(q))
    check(rc, name)
    return [vo, lse]


_fused_da_bytes = 1 << 30


def set_fused_workspace_bytes(n):
    """Most bytes the fused backward may hold as logit gradients at a time (default 1 GiB); returns the previous
    setting.  The batch is worked through in slabs of as many entries as fit, never fewer than one."""
    global _fused_da_bytes
    if int(n) < 0:
        raise ValueError("a byte count, got %r" % (n,))
    old, _fused_da_bytes = _fused_da_bytes, int(n)
    return old


def fused_backward_slab(B, T, H, itemsize):
    """Batch entries per slab of the fused backward: as many [T,T,H] blocks of logit gradients as fit the
    workspace bound, at least one, at most B."""
    per_entry = T * T * H * itemsize
    return max(1, min(B, _fused_da_bytes // per_entry if per_entry else B))


def dense_fused_backward(dvo, q, k, v, vo, lse, pipelined=False):
    """Backward of dense_fused_forward -> [dq, dk, dv].  pipelined: the first stage through
    l1attn_fused_bwd_stage_pipe_f32 (float32 only; same results bit for bit).  Stage one writes dA (the gradient of the logits, from
    dvo and the forward's vo and lse) and dv; dq and dk are the dense backward of dA.  Batch entries are
    independent, so the batch goes through in slabs that share one dA buffer of [slab,T,T,H] (stream order
    keeps a slab's readers ahead of the next slab's writer): the whole [B,T,T,H] tensor never exists, 1 GiB in place
    of 8 GiB at B=8, T=4096, H=16 in float32.  A single batch entry beyond the bound still takes its [T,T,H]."""
    _require_experimental("fused", "the fused L1 attention operator")
    for x, n in ((dvo, "dvo"), (q, "q"), (k, "k"), (v, "v"), (vo, "vo"), (lse, "lse")):
        check_input(x, n)
    if q.dim() != 4 or q.shape != k.shape or v.dim() != 4 or v.shape[:3] != q.shape[:3]:
        raise RuntimeError("q, k, v must be [batch, n_ctx, n_heads, width] tensors with equal leading dims")
    _same_as(k, q, "k", "q")
    _same_as(dvo, v, "dvo", "v")
    _same_as(vo, v, "vo", "v")
    B, T, H, W = q.shape
    if v.dtype != q.dtype or v.device != q.device or tuple(lse.shape) != (B, T, H) or lse.dtype != q.dtype \
            or lse.device != q.device:
        raise RuntimeError("v must have the dtype and device of q, and lse must be the [batch, n_ctx, n_heads] "
                           "tensor the forward returned")
    sfx = sfx_of(q)
    stage = "l1attn_fused_bwd_stage_pipe_f32" if (pipelined and sfx == "f32") else "l1attn_fused_bwd_stage_" + sfx
    slab = fused_backward_slab(B, T, H, q.element_size())
    dA = torch.empty((slab, T, T, H), dtype=q.dtype, device=q.device)
    dv = torch.empty_like(v)
    if slab >= B:
        with torch.cuda.device(q.device):
            rc = getattr(lib(), stage)(
                ptr(dvo), ptr(q), ptr(k), ptr(v), ptr(vo), ptr(lse), ptr(dA), ptr(dv), B, T, H, W, v.shape[3],
                stream_of(q))
        check(rc, stage)
        dq, dk = dense_backward(dA, q, k)
        return [dq, dk, dv]
    dq, dk = torch.empty_like(q), torch.empty_like(k)
    for b0 in range(0, B, slab):
        b1 = min(B, b0 + slab)  # (a slice of leading batch entries of a contiguous tensor is contiguous)
        with torch.cuda.device(q.device):
            rc = getattr(lib(), stage)(
                ptr(dvo[b0:b1]), ptr(q[b0:b1]), ptr(k[b0:b1]), ptr(v[b0:b1]), ptr(vo[b0:b1]), ptr(lse[b0:b1]), ptr(dA),
                ptr(dv[b0:b1]), b1 - b0, T, H, W, v.shape[3], stream_of(q))
        check(rc, stage)
        dq[b0:b1], dk[b0:b1] = dense_backward(dA[:b1 - b0], q[b0:b1], k[b0:b1])
    return [dq, dk, dv]


# ------------------------------------------------------------------------------- edge lists

def expand_coo(co):
    """GPU expandCoo: co [E,2] integer [dst,src] rows -> (coo int32 [E,4] on co.device, dst_mxlen,
    src_mxlen).  python/l1attn_sparse.py:382-427.  A CPU `co` is copied to the current GPU and the
    result copied back, as the reference returns `coo` on co.device."""
    if co.dim() != 2 or co.shape[1] < 2:
        raise RuntimeError("co must be [cl, 2] rows of [dst, src]")
    if co.dtype not in (torch.int8, torch.uint8, torch.int16, torch.int32, torch.int64):
        raise RuntimeError("co must hold integers, got %s" % co.dtype)
    dev = co.device if co.is_cuda else torch.device("cuda", torch.cuda.current_device())
    cod = co.to(dev)
    if cod.dtype not in (torch.int32, torch.int64):
        cod = cod.to(torch.int64)
    cod = cod.contiguous()
    E = cod.shape[0]
    coo = torch.zeros((E, 4), dtype=torch.int32, device=dev)
    mx = (ctypes.c_int32 * 2)()
    L = lib()
    with torch.cuda.device(dev):
        ws_bytes = L.l1attn_expand_coo_workspace_bytes(E)
        ws = torch.empty(ws_bytes, dtype=torch.uint8, device=dev)
        rc = L.l1attn_expand_coo(ptr(cod), 64 if cod.dtype == torch.int64 else 32, cod.shape[1], E,
                                 ptr(coo), mx, ptr(ws), ws_bytes, stream_of(cod))
    check(rc, "l1attn_expand_coo")
    if not co.is_cuda:
        coo = coo.cpu()
    return coo, int(mx[0]), int(mx[1])


class Plan(object):
    """dst- and src-sorted views of one edge list on one device (opaque device buffer)."""
    __slots__ = ("buf", "E", "T", "max_dst_deg", "max_src_deg")


def build_plan(coo, n_tok):
    """Plan for coo [E, >=2] int32 (device) over n_tok tokens.  Raises on an index outside [0, n_tok)."""
    E = coo.shape[0]
    L = lib()
    plan = Plan()
    with torch.cuda.device(coo.device):
        nbytes = L.l1attn_sparse_plan_bytes(E, n_tok)
        plan.buf = torch.empty(nbytes, dtype=torch.uint8, device=coo.device)
        ws_bytes = L.l1attn_sparse_plan_workspace_bytes(E, n_tok)
        ws = torch.empty(ws_bytes, dtype=torch.uint8, device=coo.device)
        st = stream_of(coo)
        rc = L.l1attn_sparse_plan_build(ptr(coo), coo.shape[1], E, n_tok, ptr(plan.buf), nbytes,
                                        ptr(ws), ws_bytes, st)
        check(rc, "l1attn_sparse_plan_build")
        hdr = (ctypes.c_int32 * 16)()
        rc = L.l1attn_sparse_plan_check(ptr(plan.buf), E, n_tok, hdr, st)
    check(rc, "l1attn_sparse_plan_check")
    plan.E, plan.T = E, n_tok
    plan.max_dst_deg, plan.max_src_deg = int(hdr[4]), int(hdr[5])
    return plan


def plan_for(coo, n_tok):
    """The plan of `coo`, cached on the tensor object and invalidated by in-place writes to it."""
    check_input(coo, "coo")
    if coo.dtype != torch.int32 or coo.dim() != 2 or coo.shape[1] < 2:
        raise RuntimeError("coo must be an int32 [cl, >=2] tensor (the output of expandCoo)")
    cached = getattr(coo, "_l1attn_plan", None)
    key = (coo._version, coo.data_ptr(), tuple(coo.shape), int(n_tok))
    if cached is not None and cached[0] == key:
        return cached[1]
    plan = build_plan(coo, int(n_tok))
    try:
        coo._l1attn_plan = (key, plan)
    except AttributeError:
        pass
    return plan


# ----------------------------------------------------------------------------------- sparse

def _sparse_shapes(v, q, k):
    if q.dim() != 4 or q.shape != k.shape or v.dim() != 4 or v.shape[:3] != q.shape[:3]:
        raise RuntimeError("v, q, k must be [batch, n_tok, n_heads, width] tensors with equal leading dims")
    if not (v.dtype == q.dtype == k.dtype) or not (v.device == q.device == k.device):
        raise RuntimeError("v, q, k must share dtype and device")
    B, T, H, W = q.shape
    return B, T, H, W, v.shape[3]


def _same_as(x, like, name, like_name):
    if x.shape != like.shape or x.dtype != like.dtype or x.device != like.device:
        raise RuntimeError("%s must have the shape, dtype and device of %s" % (name, like_name))


def _edge_tensors(coo, P, q, E, B, H):
    """coo (and the saved edge weights P, if given) must live on q's device; P is [batch, edges, heads]."""
    if coo.device != q.device:
        raise RuntimeError("coo must be on the device of q")
    p_dtype = torch.float32 if q.dtype in (torch.float16, torch.bfloat16) else q.dtype
    if P is not None and (tuple(P.shape) != (B, E, H) or P.dtype != p_dtype or P.device != q.device):
        raise RuntimeError("attn must be the [batch, edges, heads] tensor the forward returned")


def sparse_forward(v, q, k, coo, dst_mxlen, use_softmax, plan=None):
    """l1attn_sparse_cuda_drv.forward(v,q,k,coo,dst_mxlen,use_softmax) -> [vo, attn]
    (cuda/l1attn_sparse_cuda_drv.cpp:32-46).  The second tensor is the edge-weight tensor P [B,E,H]
    in plan slot order (the reference's padded attn is internal to its backward).  dst_mxlen is
    accepted for signature compatibility; segment lengths come from the plan."""
    for x, n in ((v, "v"), (q, "q"), (k, "k"), (coo, "coo")):
        check_input(x, n)
    B, T, H, W, Wv = _sparse_shapes(v, q, k)
    _edge_tensors(coo, None, q, 0, B, H)
    if plan is None:
        plan = plan_for(coo, T)
    E = plan.E
    sfx, p_dtype = sfx_fwd_sparse(q)
    vo = torch.empty_like(v)
    P = torch.empty((B, E, H), dtype=p_dtype, device=q.device)
    with torch.cuda.device(q.device):
        rc = getattr(lib(), "l1attn_sparse_fwd_" + sfx)(
            ptr(v), ptr(q), ptr(k), ptr(plan.buf), ptr(vo), ptr(P), B, T, H, W, Wv, E,
            int(bool(use_softmax)), stream_of(q))
    check(rc, "l1attn_sparse_fwd_" + sfx)
    return [vo, P]


def sparse_backward(dvo, v, q, k, coo, P, dst_mxlen, use_softmax, plan=None):
    """l1attn_sparse_cuda_drv.backward(dvo,v,q,k,coo,attn,dst_mxlen,use_softmax) -> [dv,dq,dk]
    (cuda/l1attn_sparse_cuda_drv.cpp:48-69)."""
    for x, n in ((dvo, "dvo"), (v, "v"), (q, "q"), (k, "k"), (coo, "coo"), (P, "attn")):
        check_input(x, n)
    B, T, H, W, Wv = _sparse_shapes(v, q, k)
    sfx = sfx_bwd_sparse(q)
    _same_as(dvo, v, "dvo", "v")
    if plan is None:
        plan = plan_for(coo, T)
    E = plan.E
    _edge_tensors(coo, P, q, E, B, H)
    dv, dq, dk = torch.empty_like(v), torch.empty_like(q), torch.empty_like(k)
    DA = torch.empty_like(P)
    with torch.cuda.device(q.device):
        rc = getattr(lib(), "l1attn_sparse_bwd_" + sfx)(
            ptr(dvo), ptr(v), ptr(q), ptr(k), ptr(plan.buf), ptr(P), ptr(dv), ptr(dq), ptr(dk), ptr(DA),
            B, T, H, W, Wv, E, int(bool(use_softmax)), stream_of(q))
    check(rc, "l1attn_sparse_bwd_" + sfx)
    return [dv, dq, dk]


def bidi_forward(vf, vb, q, k, coo, dst_mxlen, use_softmax, plan=None):
    """l1attn_sparse_bidi_cuda_drv.forward -> [vo, attn] (cuda/l1attn_sparse_bidi_cuda_drv.cpp:34-50)."""
    for x, n in ((vf, "vf"), (vb, "vb"), (q, "q"), (k, "k"), (coo, "coo")):
        check_input(x, n)
    B, T, H, W, Wv = _sparse_shapes(vf, q, k)
    _same_as(vb, vf, "vb", "vf")
    _edge_tensors(coo, None, q, 0, B, H)
    if plan is None:
        plan = plan_for(coo, T)
    E = plan.E
    sfx, p_dtype = sfx_fwd_sparse(q)
    vo = torch.empty_like(vf)
    P = torch.empty((B, E, H), dtype=p_dtype, device=q.device)
    with torch.cuda.device(q.device):
        rc = getattr(lib(), "l1attn_sparse_bidi_fwd_" + sfx)(
            ptr(vf), ptr(vb), ptr(q), ptr(k), ptr(plan.buf), ptr(vo), ptr(P), B, T, H, W, Wv, E,
            int(bool(use_softmax)), stream_of(q))
    check(rc, "l1attn_sparse_bidi_fwd_" + sfx)
    return [vo, P]


def bidi_backward(dvo, vf, vb, q, k, coo, P, dst_mxlen, use_softmax, plan=None):
    """l1attn_sparse_bidi_cuda_drv.backward -> [dvf,dvb,dq,dk] (cuda/l1attn_sparse_bidi_cuda_drv.cpp:52-75)."""
    for x, n in ((dvo, "dvo"), (vf, "vf"), (vb, "vb"), (q, "q"), (k, "k"), (coo, "coo"), (P, "attn")):
        check_input(x, n)
    B, T, H, W, Wv = _sparse_shapes(vf, q, k)
    sfx = sfx_bwd_sparse(q)
    _same_as(vb, vf, "vb", "vf")
    _same_as(dvo, vf, "dvo", "vf")
    if plan is None:
        plan = plan_for(coo, T)
    E = plan.E
    _edge_tensors(coo, P, q, E, B, H)
    dvf, dvb, dq, dk = torch.empty_like(vf), torch.empty_like(vb), torch.empty_like(q), torch.empty_like(k)
    DA = torch.empty_like(P)
    with torch.cuda.device(q.device):
        rc = getattr(lib(), "l1attn_sparse_bidi_bwd_" + sfx)(
            ptr(dvo), ptr(vf), ptr(vb), ptr(q), ptr(k), ptr(plan.buf), ptr(P),
            ptr(dvf), ptr(dvb), ptr(dq), ptr(dk), ptr(DA),
            B, T, H, W, Wv, E, int(bool(use_softmax)), stream_of(q))
    check(rc, "l1attn_sparse_bidi_bwd_" + sfx)
    return [dvf, dvb, dq, dk]
