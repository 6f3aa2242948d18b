"""Stand-in for the reference's native CPU module of the same name (pybind11,
cpp/l1attn_sparse_bidi_drv.cpp:214-217): forward(vf, vb, q, k, coo, dst_mxlen, use_softmax) -> [vo, attn],
backward(dvo, vf, vb, q, k, coo, attn, dst_mxlen, use_softmax) -> [dvf, dvb, dq, dk], on host tensors."""
import _l1attn_cpu as _drv


def forward(vf, vb, q, k, coo, dst_mxlen, use_softmax):
    """L1AttnSparseBidi forward"""
    return _drv.bidi_forward(vf, vb, q, k, coo, int(dst_mxlen), bool(use_softmax))


def backward(dvo, vf, vb, q, k, coo, attn, dst_mxlen, use_softmax):
    """L1AttnSparseBidi backward"""
    return _drv.bidi_backward(dvo, vf, vb, q, k, coo, attn, int(dst_mxlen), bool(use_softmax))
