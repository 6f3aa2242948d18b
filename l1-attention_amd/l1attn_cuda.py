"""Drop-in for the reference module of the same name (cuda/l1attn_cuda.py:7-32): dense L1
attention logits with autograd, computed by the gfx950 HIP library.

    m = l1attn_cuda.L1Attn()
    a = m(q, k)              # q,k [batch, n_ctx, n_heads, width] -> a [batch, src, dst, heads]
    a_sm = F.softmax(a, 1)   # softmax over the SRC dimension (dim 1)
    vo = torch.einsum('bsdh,bshw->bdhw', a_sm, v)

a[b,s,t,h] = -1/sqrt(width) * sum_w |q[b,t,h,w] - k[b,s,h,w]|.
"""
import torch
from torch import nn
from torch.autograd import Function

import _l1attn_hip as _drv


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
        # the reference driver rejects a non-contiguous d_attn (cuda/l1attn_cuda_drv.cpp:71);
        # autograd may hand one over (e.g. an expanded gradient), so it is packed here instead
        d_q, d_k = _drv.dense_backward(d_attn.contiguous(), q, k)
        return d_q, d_k


class L1Attn(nn.Module):
    def __init__(self):
        super(L1Attn, self).__init__()

    def forward(self, q, k):
        return L1AttnFn.apply(q, k)


class L1AttnFusedFn(Function):
    """L1 attention with the value sum fused in: softmax over the src tokens of the L1 logits with the no-op
    zero logit, times v, without the [B,T,T,H] logits.  Equals
    einsum('bsdh,bshw->bdhw', softmax(cat(L1Attn()(q,k), zeros), 1)[:, :-1], v), the composition of
    example-setfind/setfind.py:128-136.  The reference has no such function (README.md:21 asks for it).
    The backward holds one [B,T,T,H] tensor (the gradient of the logits) where the composition holds four."""
    @staticmethod
    def forward(ctx, q, k, v, *pipelined):
        # apply(q, k, v) or apply(q, k, v, pipelined): the flag picks the software-pipelined kernels (same results)
        q, k, v = q.contiguous(), k.contiguous(), v.contiguous()
        ctx.pipelined, ctx.n_flags = bool(pipelined and pipelined[0]), len(pipelined)
        vo, lse = _drv.dense_fused_forward(q, k, v, want_lse=True, pipelined=ctx.pipelined)
        ctx.save_for_backward(q, k, v, vo, lse)
        return vo

    @staticmethod
    def backward(ctx, d_vo):
        q, k, v, vo, lse = ctx.saved_tensors[:5]
        d_q, d_k, d_v = _drv.dense_fused_backward(d_vo.contiguous(), q, k, v, vo, lse, pipelined=ctx.pipelined)
        return (d_q, d_k, d_v) + (None,) * ctx.n_flags


class L1AttnFused(nn.Module):
    """pipelined: the kernels that stream the wave-uniform rows through a software pipeline of scalar loads, where
    they exist (float32, widths 32 and 64); same results bit for bit."""
    def __init__(self, pipelined=False):
        super(L1AttnFused, self).__init__()
        self.pipelined = bool(pipelined)

    def forward(self, q, k, v):
        return L1AttnFusedFn.apply(q, k, v, self.pipelined)
