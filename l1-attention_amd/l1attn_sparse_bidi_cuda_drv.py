"""Stand-in for the reference's native module of the same name (pybind11,
cuda/l1attn_sparse_bidi_cuda_drv.cpp:77-80):

    l1attn_sparse_bidi_cuda_drv.forward(vf, vb, q, k, coo, dst_mxlen, use_softmax)              -> [vo, attn]   (:34-50)
    l1attn_sparse_bidi_cuda_drv.backward(dvo, vf, vb, q, k, coo, attn, dst_mxlen, use_softmax)  -> [dvf, dvb, dq, dk]  (:52-75)

Same names, argument order, list returns, ownership and CHECK_INPUT errors, so the reference's own
cuda/l1attn_sparse_bidi_cuda.py runs on this module unchanged.  `attn` is opaque to that caller: here it is the
edge-weight tensor [batch, edges, heads] in dst-sorted order.
"""
import _l1attn_hip as _drv


def forward(vf, vb, q, k, coo, dst_mxlen, use_softmax):
    """L1AttnSparseBidi forward (HIP)"""
    return _drv.bidi_forward(vf, vb, q, k, coo, int(dst_mxlen), bool(use_softmax))


def backward(dvo, vf, vb, q, k, coo, attn, dst_mxlen, use_softmax):
    """L1AttnSparseBidi backward (HIP)"""
    return _drv.bidi_backward(dvo, vf, vb, q, k, coo, attn, int(dst_mxlen), bool(use_softmax))
