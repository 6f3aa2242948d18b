"""Drop-in for the reference module of the same name (cuda/l1attn_sparse_bidi_cuda.py:8-104):
bidirectional sparse L1 attention with autograd and expandCoo, computed by the gfx950 HIP library.

    vo = L1AttnSparseBidi()(vf, vb, q, k, coo, dst_mxlen)      # use_softmax defaults to True
    vo[b,dst] += p*vf[b,src]   and   vo[b,src] += p*vb[b,dst]
"""
import torch
from torch import nn
from torch.autograd import Function

import _l1attn_hip as _drv


class L1AttnSparseBidiFn(Function):
    @staticmethod
    def forward(ctx, vf, vb, q, k, coo, dst_mxlen, use_softmax=True):
        vf = vf.contiguous()
        vb = vb.contiguous()
        q = q.contiguous()
        k = k.contiguous()
        plan = _drv.plan_for(coo, q.shape[1])
        vo, attn = _drv.bidi_forward(vf, vb, q, k, coo, dst_mxlen, use_softmax, plan)
        ctx.save_for_backward(vf, vb, q, k, coo, attn)
        ctx.plan = plan
        ctx.dst_mxlen = int(dst_mxlen)
        ctx.use_softmax = bool(use_softmax)
        return vo

    @staticmethod
    def backward(ctx, dvo):
        dvo = dvo.contiguous()
        vf, vb, q, k, coo, attn = ctx.saved_tensors[:6]
        d_vf, d_vb, d_q, d_k = _drv.bidi_backward(dvo, vf, vb, q, k, coo, attn, ctx.dst_mxlen,
                                                  ctx.use_softmax, ctx.plan)
        return d_vf, d_vb, d_q, d_k, None, None, None


class L1AttnSparseBidi(nn.Module):
    def __init__(self):
        super(L1AttnSparseBidi, self).__init__()

    def forward(self, vf, vb, q, k, coo, dst_mxlen, use_softmax=True):
        return L1AttnSparseBidiFn.apply(vf, vb, q, k, coo, dst_mxlen, use_softmax)


def expandCoo(co, warn=True):
    '''
    take a coordinate vector 'co' consisting of [dst,src] pairs; returns
    coo (int32 [cl,4] = [dst, src, dst_cnt, src_cnt] on co.device), dst_mxlen, src_mxlen
    (cuda/l1attn_sparse_bidi_cuda.py:59-104; the ranks are computed on the GPU)
    '''
    coo, dst_mxlen, src_mxlen = _drv.expand_coo(co)
    if warn and coo.shape[0] > 0:
        # this copy warns separately for unwritten dst and unread src indices (:96-101)
        for col, msg in ((0, 'Warning: degenerate sparse head - {} not written'),
                         (1, 'Warning degenerate sparse head - {} not read')):
            kmax = int(coo[:, col].max())
            if kmax > 0:
                seen = torch.zeros(kmax + 1, dtype=torch.bool, device=coo.device)
                seen[coo[:, col].long()] = True
                for i in torch.nonzero(~seen[:kmax]).flatten().tolist():
                    print(msg.format(i))
    return coo, dst_mxlen, src_mxlen
