"""Stand-in for the reference's native module of the same name (pybind11, cuda/l1attn_sparse_cuda_drv.cpp:71-74):

    l1attn_sparse_cuda_drv.forward(v, q, k, coo, dst_mxlen, use_softmax)                -> [vo, attn]     (:32-46)
    l1attn_sparse_cuda_drv.backward(dvo, v, q, k, coo, attn, dst_mxlen, use_softmax)    -> [dv, dq, dk]   (:48-69)

Same names, argument order, list returns, ownership and CHECK_INPUT errors, so the reference's own
cuda/l1attn_sparse_cuda.py runs on this module unchanged.  `attn` is opaque to that caller (saved in forward,
handed back in backward): here it is the edge-weight tensor [batch, edges, heads] in dst-sorted order, not the
reference's padded [batch, n_tok, dst_mxlen, heads].  The dst- and src-sorted views of `coo` are built on the
first call with a given coo tensor and cached on it.
"""
import _l1attn_hip as _drv


def forward(v, q, k, coo, dst_mxlen, use_softmax):
    """L1AttnSparse forward (HIP)"""
    return _drv.sparse_forward(v, q, k, coo, int(dst_mxlen), bool(use_softmax))


def backward(dvo, v, q, k, coo, attn, dst_mxlen, use_softmax):
    """L1AttnSparse backward (HIP)"""
    return _drv.sparse_backward(dvo, v, q, k, coo, attn, int(dst_mxlen), bool(use_softmax))
