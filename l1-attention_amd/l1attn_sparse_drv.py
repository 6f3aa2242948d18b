"""Stand-in for the reference's native CPU module of the same name (pybind11, cpp/l1attn_sparse_drv.cpp:192-195):
forward(v, q, k, coo, dst_mxlen, use_softmax) -> [vo, attn],
backward(dvo, v, q, k, coo, attn, dst_mxlen, use_softmax) -> [dv, dq, dk], on host tensors, float32 or float64."""
import _l1attn_cpu as _drv


def forward(v, q, k, coo, dst_mxlen, use_softmax):
    """L1AttnSparse forward"""
    return _drv.sparse_forward(v, q, k, coo, int(dst_mxlen), bool(use_softmax))


def backward(dvo, v, q, k, coo, attn, dst_mxlen, use_softmax):
    """L1AttnSparse backward"""
    return _drv.sparse_backward(dvo, v, q, k, coo, attn, int(dst_mxlen), bool(use_softmax))
