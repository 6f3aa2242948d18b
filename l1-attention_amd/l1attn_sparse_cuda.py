"""Drop-in for the reference module of the same name (cuda/l1attn_sparse_cuda.py:8-101): sparse
(edge-list) L1 attention with autograd and expandCoo, computed by the gfx950 HIP library.

    coo, dst_mxlen, src_mxlen = l1attn_sparse_cuda.expandCoo(co)     # co [cl,2] = [dst,src] rows
    m = l1attn_sparse_cuda.L1AttnSparse()
    vo = m(v, q, k, coo.to(device), dst_mxlen)                       # use_softmax defaults to True

The reference's README calls the module with five arguments (README.md:93) while its wrapper
requires six (cuda/l1attn_sparse_cuda.py:54); both forms are accepted here.
float32 and float64 as in the reference; float16 and bfloat16 tensors are accepted too (rows and
gradients in that type, sums and edge weights in fp32; the reference dispatches Half in its forward only).
"""
import torch
from torch import nn
from torch.autograd import Function

import _l1attn_hip as _drv


class L1AttnSparseFn(Function):
    @staticmethod
    def forward(ctx, v, q, k, coo, dst_mxlen, use_softmax=True):
        v = v.contiguous()
        q = q.contiguous()
        k = k.contiguous()
        plan = _drv.plan_for(coo, q.shape[1])
        vo, attn = _drv.sparse_forward(v, q, k, coo, dst_mxlen, use_softmax, plan)
        ctx.save_for_backward(v, q, k, coo, attn)
        ctx.plan = plan
        ctx.dst_mxlen = int(dst_mxlen)
        ctx.use_softmax = bool(use_softmax)
        return vo

    @staticmethod
    def backward(ctx, dvo):
        dvo = dvo.contiguous()  # "not always" contiguous (cuda/l1attn_sparse_cuda.py:40-41)
        v, q, k, coo, attn = ctx.saved_tensors[:5]
        d_v, d_q, d_k = _drv.sparse_backward(dvo, v, q, k, coo, attn, ctx.dst_mxlen, ctx.use_softmax, ctx.plan)
        return d_v, d_q, d_k, None, None, None


class L1AttnSparse(nn.Module):
    def __init__(self):
        super(L1AttnSparse, self).__init__()

    def forward(self, v, q, k, coo, dst_mxlen, use_softmax=True):
        return L1AttnSparseFn.apply(v, q, k, coo, dst_mxlen, use_softmax)


def expandCoo(co, warn=True):
    '''
    take a coordinate vector 'co' consisting of [dst,src] pairs
    - add a third column: the index of the edge among the edges of its dst (softmax slot)
    - add a fourth column: the index of the edge among the edges of its src (backward pass)
    returns coo (int32 [cl,4] on co.device), dst_mxlen, src_mxlen
    (cuda/l1attn_sparse_cuda.py:58-101; the ranks are computed on the GPU)
    '''
    coo, dst_mxlen, src_mxlen = _drv.expand_coo(co)
    if warn and coo.shape[0] > 0:
        # this copy of the reference warns for tokens below the largest dst that are neither
        # read nor written (cuda/l1attn_sparse_cuda.py:92-98)
        dst_max = int(coo[:, 0].max())
        if dst_max > 0:
            seen = torch.zeros(dst_max + 1, dtype=torch.bool, device=coo.device)
            seen[coo[:, 0].long()] = True
            src = coo[:, 1].long()
            seen[src[src <= dst_max]] = True
            for i in torch.nonzero(~seen[:dst_max]).flatten().tolist():
                print(f'Warning: sparse head - {i} neither read nor written')
    return coo, dst_mxlen, src_mxlen
