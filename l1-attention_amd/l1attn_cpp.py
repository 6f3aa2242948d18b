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


class L1AttnFusedFn(Function):
    """The host twin of l1attn_cuda.L1AttnFusedFn: softmax over the src tokens of the L1 logits with the no-op zero
    logit, times v, without the [B,T,T,H] logits.  Equals
    einsum('bsdh,bshw->bdhw', softmax(cat(L1Attn()(q,k), zeros), 1)[:, :-1], v), the composition of
    example-setfind/setfind.py:128-136; the reference has no such function (README.md:21 asks for it)."""
    @staticmethod
    def forward(ctx, q, k, v):
        q, k, v = q.contiguous(), k.contiguous(), v.contiguous()
        vo, lse = _drv.fused_forward(q, k, v)
        ctx.save_for_backward(q, k, v, vo, lse)
        return vo

    @staticmethod
    def backward(ctx, d_vo):
        q, k, v, vo, lse = ctx.saved_tensors[:5]
        d_q, d_k, d_v = _drv.fused_backward(d_vo.contiguous(), q, k, v, vo, lse)
        return d_q, d_k, d_v


class L1AttnFused(nn.Module):
    """pipelined: accepted for symmetry with l1attn_cuda.L1AttnFused (a choice between GPU kernels with equal
    results); it has no meaning on the host."""
    def __init__(self, pipelined=False):
        super(L1AttnFused, self).__init__()

    def forward(self, q, k, v):
        return L1AttnFusedFn.apply(q, k, v)
