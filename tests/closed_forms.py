"""Vectorised fp64 statements of the hot path's mathematics, written independently of
the oracle's loops (broadcast / index_add_ instead of nested loops) and differentiable
by torch autograd.  Used to pin the oracle and as the fp64 yardstick for mid-size GPU
parity tests (sizes the loop oracle would take too long on)."""
import math

import torch


def dense_attn(q, k):
    """A[b,s,t,h] = -1/sqrt(W) * sum_w |q[b,t,h,w] - k[b,s,h,w]|  (src index first)."""
    W = q.shape[-1]
    return -(q[:, None, :, :, :] - k[:, :, None, :, :]).abs().sum(-1) / math.sqrt(W)


def dense_then_value(q, k, v, noop=True):
    """softmax over src with an extra zero logit (the '+1' in the denominator), then
    'bsdh,bshw->bdhw' -- what sparse attention over the full cartesian edge list equals."""
    a = dense_attn(q, k)
    if noop:
        e = a.exp()
        p = e / (1.0 + e.sum(1, keepdim=True))
    else:
        p = a.exp()
    return torch.einsum("bsdh,bshw->bdhw", p, v)


def edge_probs(q, k, coo, use_softmax=True):
    B, T, H, W = q.shape
    dst, src = coo[:, 0].long(), coo[:, 1].long()
    a = -(q[:, dst] - k[:, src]).abs().sum(-1) / math.sqrt(W)  # [B,E,H]
    e = a.exp()
    if use_softmax:
        den = torch.ones(B, T, H, dtype=q.dtype, device=q.device).index_add(1, dst, e)
        return e / den[:, dst]
    return e


def sparse_value(v, q, k, coo, use_softmax=True):
    dst, src = coo[:, 0].long(), coo[:, 1].long()
    p = edge_probs(q, k, coo, use_softmax)
    out = torch.zeros(v.shape, dtype=v.dtype, device=v.device)
    return out.index_add(1, dst, p[..., None] * v[:, src])


def bidi_value(vf, vb, q, k, coo, use_softmax=True):
    dst, src = coo[:, 0].long(), coo[:, 1].long()
    p = edge_probs(q, k, coo, use_softmax)
    out = torch.zeros(vf.shape, dtype=vf.dtype, device=vf.device)
    out = out.index_add(1, dst, p[..., None] * vf[:, src])
    return out.index_add(1, src, p[..., None] * vb[:, dst])


def expand_coo_bruteforce(co):
    """O(E^2): rank of row i among earlier rows with the same key."""
    co = co.long()
    E = co.shape[0]
    out = torch.zeros(E, 4, dtype=torch.int32)
    for i in range(E):
        out[i, 0] = co[i, 0]
        out[i, 1] = co[i, 1]
        out[i, 2] = int((co[:i, 0] == co[i, 0]).sum())
        out[i, 3] = int((co[:i, 1] == co[i, 1]).sum())
    dmx = int(out[:, 2].max()) + 1 if E else 1
    smx = int(out[:, 3].max()) + 1 if E else 1
    return out, dmx, smx


def rel_err(x, ref):
    """max|x-ref| / max|ref| : the tolerance metric for fp32 results against fp64."""
    denom = ref.abs().max().item()
    if denom == 0:
        return (x.double() - ref.double()).abs().max().item()
    return (x.double() - ref.double()).abs().max().item() / denom
