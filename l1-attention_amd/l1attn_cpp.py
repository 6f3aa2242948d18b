"""Drop-in for the reference's CPU module of the same name (cpp/l1attn_cpp.py:12-34): dense L1 attention
logits with autograd on host tensors, computed by libl1attn_cpu.so (OpenMP, float32 and float64).

    a = l1attn_cpp.L1Attn()(q, k)   # q,k [batch, n_ctx, n_heads, width] -> a [batch, src, dst, heads]
"""
from torch import nn
from torch.autograd import Function

import _l1attn_cpu as _drv


class L1AttnFn(Function):
    @staticmethod
    def forward(ctx, q, k):
        q = q.contiguous()
        k = k.contiguous()
        attn = _drv.dense_forward(q, k)
        ctx.save_for_backward(q, k)
        return attn[0]

    @staticmethod
    def backward(ctx, d_attn):
        q, k = ctx.saved_tensors[:2]
        d_q, d_k = _drv.dense_backward(d_attn.contiguous(), q, k)
        return d_q, d_k


class L1Attn(nn.Module):
    def __init__(self):
        super(L1Attn, self).__init__()

    def forward(self, q, k):
        return L1AttnFn.apply(q, k)
