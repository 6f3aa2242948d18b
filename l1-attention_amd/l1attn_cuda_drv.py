"""Stand-in for the reference's native module of the same name (pybind11, cuda/l1attn_cuda_drv.cpp:106-109):

    l1attn_cuda_drv.forward(q, k)            -> [attn]        (cuda/l1attn_cuda_drv.cpp:42-65)
    l1attn_cuda_drv.backward(d_attn, q, k)   -> [d_q, d_k]    (cuda/l1attn_cuda_drv.cpp:67-104)

Same names, argument order, list returns, ownership (the callee allocates, inputs are borrowed) and
CHECK_INPUT errors, so the reference's own cuda/l1attn_cuda.py runs on this module unchanged.  The work is
done by the gfx950 HIP library through its C ABI; there is no CPU path behind these functions.
"""
import _l1attn_hip as _drv


def forward(q, k):
    """L1Attn forward (HIP)"""
    return _drv.dense_forward(q, k)


def backward(d_attn, q, k):
    """L1Attn backward (HIP)"""
    return _drv.dense_backward(d_attn, q, k)
