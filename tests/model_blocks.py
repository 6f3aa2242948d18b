"""The two call patterns with which the reference's model code embeds the dense operator, as plain functions
of (inputs, weights, operator), shared by the CPU and GPU tests:

  * setfind_block: example-setfind/setfind.py:98-138 -- q and v from linear layers, k a per-head gated broadcast
    view of x, both padded with zero tokens to a multiple of 16, one logit row overwritten in place with the
    no-op 0, softmax over src, 'bsdh,bshw->bdhw' with v, sum over heads.
  * split_block: example/model.py:46-59 with its stale [b,h,t,s] indexing brought to the operator's
    [b,src,dst,h] -- q, k, v are the three torch.split views of one projection (non-contiguous: the last-but-one
    stride is three heads wide), the diagonal of the logits is zeroed in place, softmax over src, value
    contraction, heads concatenated.

`l1a(q, k)` is the operator under test or tests/closed_forms.dense_attn.
"""
import math

import torch


def setfind_block(x, wq, wv, wk, l1a, n_head):
    batch, ntok, d_model = x.shape
    q = (x @ wq).reshape(batch, ntok, n_head, d_model)
    v = (x @ wv).reshape(batch, ntok, n_head, d_model)
    k = x.unsqueeze(2).expand(-1, -1, n_head, -1) * wk.unsqueeze(0).unsqueeze(0)
    padn = ((ntok + 15) // 16) * 16 - ntok
    assert padn > 0  # room for the no-op row, as setfind.py:125 asserts
    zeros = torch.zeros(batch, padn, n_head, d_model, dtype=x.dtype, device=x.device)
    a = l1a(torch.cat((q, zeros), 1), torch.cat((k, zeros), 1))
    a = a[:, :ntok + 1, :ntok, :]
    a[:, ntok, :, :] = 0.0  # in place on a view of the operator's output, as setfind.py:130
    a = torch.softmax(a, 1)[:, :ntok, :ntok, :]
    return torch.einsum("bsdh,bshw->bdhw", a, v).sum(2)


def setfind_leaves(batch, ntok, d_model, n_head, dtype, device, seed=99):
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(batch, ntok, d_model, generator=g)
    wq = torch.randn(d_model, n_head * d_model, generator=g) / math.sqrt(d_model)
    wv = torch.randn(d_model, n_head * d_model, generator=g) / math.sqrt(d_model)
    wk = torch.randn(n_head, d_model, generator=g)
    return [t.to(dtype).to(device).requires_grad_() for t in (x, wq, wv, wk)]


def split_block(x, w_qkv, b_qkv, l1a, n_head):
    bs, n_ctx, width = x.shape
    attn_ch = width // n_head
    qkv = (x @ w_qkv + b_qkv).view(bs, n_ctx, n_head, -1)   # [bs, ctx, heads, 3 * attn_ch]
    q, k, v = torch.split(qkv, attn_ch, dim=-1)             # three strided views
    assert not q.is_contiguous() and not k.is_contiguous()
    weight = l1a(q, k)                                      # [b, src, dst, h]
    i = torch.arange(0, n_ctx, device=x.device)
    weight[:, i, i, :] = 0.0                                # the diagonal, in place on the operator's output
    weight = torch.softmax(weight, dim=1)                   # over src
    return x + torch.einsum("bsth,bshc->bthc", weight, v).reshape(bs, n_ctx, -1)


def split_leaves(bs, n_ctx, width, dtype, device, seed=77):
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(bs, n_ctx, width, generator=g)
    w = torch.randn(width, 3 * width, generator=g) / math.sqrt(width)
    b = torch.randn(3 * width, generator=g) * 0.1
    return [t.to(dtype).to(device).requires_grad_() for t in (x, w, b)]
