"""Stand-in for the reference's native CPU module of the same name (pybind11, cpp/l1attn_drv.cpp:100-103):
forward(q, k) -> [attn], backward(d_attn, q, k) -> [d_q, d_k], on host tensors, float32 or float64."""
import _l1attn_cpu as _drv


def forward(q, k):
    """L1Attn forward"""
    return _drv.dense_forward(q, k)


def backward(d_attn, q, k):
    """L1Attn backward"""
    return _drv.dense_backward(d_attn, q, k)
