"""Drop-in for the reference's CPU module of the same name (cpp/l1attn_sparse_bidi_cpp.py:10-57):
bidirectional sparse L1 attention with autograd on host tensors, computed by libl1attn_cpu.so.

    vo = l1attn_sparse_bidi_cpp.L1AttnSparseBidi()(vf, vb, q, k, coo, dst_mxlen)   # use_softmax defaults to True

The reference's module wrapper takes (q, k) only and cannot be called (cpp/l1attn_sparse_bidi_cpp.py:56-57);
here it takes the operator's arguments.  expandCoo is re-exported from l1attn_sparse_cpp for symmetry with the
GPU module (the reference's bidirectional CPU module has none; its CUDA twin carries its own copy,
cuda/l1attn_sparse_bidi_cuda.py:59-104).
"""
from torch import nn
from torch.autograd import Function

import _l1attn_cpu as _drv
from l1attn_sparse_cpp import expandCoo  # noqa: F401


class L1AttnSparseBidiFn(Function):
    @staticmethod
    def forward(ctx, vf, vb, q, k, coo, dst_mxlen, use_softmax=True):
        vf = vf.contiguous()
        vb = vb.contiguous()
        q = q.contiguous()
        k = k.contiguous()
        coo = coo.contiguous()
        vo, attn = _drv.bidi_forward(vf, vb, q, k, coo, dst_mxlen, use_softmax)
        ctx.save_for_backward(vf, vb, q, k, coo, attn)
        ctx.dst_mxlen = int(dst_mxlen)
        ctx.use_softmax = bool(use_softmax)
        return vo

    @staticmethod
    def backward(ctx, dvo):
        vf, vb, q, k, coo, attn = ctx.saved_tensors[:6]
        d_vf, d_vb, d_q, d_k = _drv.bidi_backward(dvo.contiguous(), vf, vb, q, k, coo, attn, ctx.dst_mxlen,
                                                  ctx.use_softmax)
        return d_vf, d_vb, d_q, d_k, None, None, None


class L1AttnSparseBidi(nn.Module):
    def __init__(self):
        super(L1AttnSparseBidi, self).__init__()

    def forward(self, vf, vb, q, k, coo, dst_mxlen, use_softmax=True):
        return L1AttnSparseBidiFn.apply(vf, vb, q, k, coo, dst_mxlen, use_softmax)
