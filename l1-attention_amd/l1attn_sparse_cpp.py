"""Drop-in for the reference's CPU module of the same name (cpp/l1attn_sparse_cpp.py:11-106): sparse
(edge-list) L1 attention with autograd and expandCoo on host tensors, computed by libl1attn_cpu.so.

    coo, dst_mxlen, src_mxlen = l1attn_sparse_cpp.expandCoo(co)
    vo = l1attn_sparse_cpp.L1AttnSparse()(v, q, k, coo, dst_mxlen)          # use_softmax defaults to True

The reference's module wrapper takes (q, k) only and cannot be called (cpp/l1attn_sparse_cpp.py:57-58; its
tests go through L1AttnSparseFn.apply); here it takes the operator's arguments.
"""
from torch import nn
from torch.autograd import Function

import _l1attn_cpu as _drv


class L1AttnSparseFn(Function):
    @staticmethod
    def forward(ctx, v, q, k, coo, dst_mxlen, use_softmax=True):
        v = v.contiguous()
        q = q.contiguous()
        k = k.contiguous()
        coo = coo.contiguous()
        vo, attn = _drv.sparse_forward(v, q, k, coo, dst_mxlen, use_softmax)
        ctx.save_for_backward(v, q, k, coo, attn)
        ctx.dst_mxlen = int(dst_mxlen)
        ctx.use_softmax = bool(use_softmax)
        return vo

    @staticmethod
    def backward(ctx, dvo):
        v, q, k, coo, attn = ctx.saved_tensors[:5]
        d_v, d_q, d_k = _drv.sparse_backward(dvo.contiguous(), v, q, k, coo, attn, ctx.dst_mxlen, ctx.use_softmax)
        return d_v, d_q, d_k, None, None, None


class L1AttnSparse(nn.Module):
    def __init__(self):
        super(L1AttnSparse, self).__init__()

    def forward(self, v, q, k, coo, dst_mxlen, use_softmax=True):
        return L1AttnSparseFn.apply(v, q, k, coo, dst_mxlen, use_softmax)


def expandCoo(co, warn=True):
    '''
    take a coordinate vector 'co' consisting of [dst,src] pairs; returns
    coo (int32 [cl,4] = [dst, src, dst_cnt, src_cnt]), dst_mxlen, src_mxlen
    (cpp/l1attn_sparse_cpp.py:61-106; the loop runs in the CPU library)
    '''
    coo, dst_mxlen, src_mxlen = _drv.expand_coo(co)
    if warn and coo.shape[0] > 0:
        # as this copy of the reference: one warning per unwritten dst and per unread src below the largest (:97-102)
        import torch
        for col, msg in ((0, 'Warning: degenerate sparse head - {} not written'),
                         (1, 'Warning degenerate sparse head - {} not read')):
            kmax = int(coo[:, col].max())
            if kmax > 0:
                seen = torch.zeros(kmax + 1, dtype=torch.bool)
                idx = coo[:, col].long()
                seen[idx[idx >= 0]] = True
                for i in torch.nonzero(~seen[:kmax]).flatten().tolist():
                    print(msg.format(i))
    return coo, dst_mxlen, src_mxlen
