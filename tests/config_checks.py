"""Parity checks of the benchmark configurations at a size given by the caller, written against the operator
API only (L1Attn()(q,k); L1AttnSparse()(v,q,k,coo,dst_mxlen); L1AttnSparseBidi()(vf,vb,q,k,coo,dst_mxlen);
expandCoo), so that the same function checks the GPU operators at the configurations' full sizes (GPU tests) and
the CPU operator package at reduced sizes (CPU tests; that run also proves the check itself).

Yardstick: the float64 closed forms of tests/closed_forms.py with torch autograd on the same float32-valued
inputs, evaluated on `dev`.  Metric: max|x - ref| / max|ref| per tensor.
"""
import torch

import closed_forms as cf
import workloads

FWD_TOL, BWD_TOL = 1e-5, 1e-4


def dense_with_downstream(l1attn_mod, dev, B, T, H, W, seed=1001):
    """Second baseline configuration: logits, then softmax over src and 'bsdh,bshw->bdhw' with v, gradients from a
    random output gradient back to q and k.  The operator runs on the whole batch at once; the float64 yardstick
    goes batch by batch (its [1,S,T,H,W] intermediate is T*T*H*W*8 bytes: 4 GiB at T=1024, H=8, W=64).
    Returns the worst errors (logits, output, dq, dk)."""
    q, k, v = (x.to(dev) for x in workloads.dense_inputs(B, T, H, W, seed=seed, with_v=True))
    qd, kd = q.clone().requires_grad_(), k.clone().requires_grad_()
    a = l1attn_mod.L1Attn()(qd, kd)
    vo = torch.einsum("bsdh,bshw->bdhw", torch.softmax(a, 1), v)
    dvo = torch.randn(vo.shape, generator=torch.Generator().manual_seed(seed + 1)).to(dev)
    vo.backward(dvo)
    worst = [0.0, 0.0, 0.0, 0.0]
    for b in range(B):
        q64 = q[b:b + 1].double().requires_grad_()
        k64 = k[b:b + 1].double().requires_grad_()
        a64 = cf.dense_attn(q64, k64)
        vo64 = torch.einsum("bsdh,bshw->bdhw", torch.softmax(a64, 1), v[b:b + 1].double())
        vo64.backward(dvo[b:b + 1].double())
        errs = (cf.rel_err(a[b:b + 1].detach(), a64.detach()), cf.rel_err(vo[b:b + 1].detach(), vo64.detach()),
                cf.rel_err(qd.grad[b:b + 1], q64.grad), cf.rel_err(kd.grad[b:b + 1], k64.grad))
        worst = [max(x, y) for x, y in zip(worst, errs)]
        del q64, k64, a64, vo64
    return worst


def sparse_uniform_graph(sp_mod, dev, B, T, H, W, max_deg=64, seed=1004):
    """Fourth baseline configuration: every dst gets 1..max_deg distinct src tokens, rows shuffled, through
    expandCoo and the one-directional operator, forward and all three gradients.  The float64 yardstick gathers
    [B,E,H,W] rows: B*E*H*W*8 bytes per intermediate (1.1 GB at the full size, E = 133 k), a handful of them alive
    under autograd.  Returns (E, [errors of vo, dv, dq, dk])."""
    co = workloads.uniform_degree_graph(T, max_deg, seed=seed)
    coo, dmx, smx = sp_mod.expandCoo(co.to(dev), warn=False)
    assert dmx <= max_deg and coo.shape == (co.shape[0], 4)
    v, _, q, k = (x.to(dev) for x in workloads.sparse_inputs(B, T, H, W, seed=seed, n=4))
    dvo = torch.randn(B, T, H, W, generator=torch.Generator().manual_seed(seed + 1)).to(dev)
    leaves = [x.clone().requires_grad_() for x in (v, q, k)]
    vo = sp_mod.L1AttnSparse()(*leaves, coo, dmx)
    got = (vo.detach(),) + torch.autograd.grad(vo, leaves, dvo)
    ref_leaves = [x.double().requires_grad_() for x in (v, q, k)]
    rvo = cf.sparse_value(*ref_leaves, coo, True)
    ref = (rvo.detach(),) + torch.autograd.grad(rvo, ref_leaves, dvo.double())
    return co.shape[0], [cf.rel_err(x, y) for x, y in zip(got, ref)]


def bidi_powerlaw_graph(bi_mod, dev, B, T, H, W, seed=1005):
    """Fifth baseline configuration: Zipf degrees clipped to [1, 2048] plus self loops, bidirectional operator,
    forward and all four gradients.  Yardstick memory: B*E*H*W*8 bytes per gathered intermediate (2.2 GB at the
    full size, E = 1.08 M).  Returns (E, longest dst segment, [errors of vo, dvf, dvb, dq, dk])."""
    co = workloads.powerlaw_graph(T, seed=seed)
    coo, dmx, smx = bi_mod.expandCoo(co.to(dev), warn=False)
    vf, vb, q, k = (x.to(dev) for x in workloads.sparse_inputs(B, T, H, W, seed=seed, n=4))
    dvo = torch.randn(B, T, H, W, generator=torch.Generator().manual_seed(seed + 1)).to(dev)
    leaves = [x.clone().requires_grad_() for x in (vf, vb, q, k)]
    vo = bi_mod.L1AttnSparseBidi()(*leaves, coo, dmx)
    got = (vo.detach(),) + torch.autograd.grad(vo, leaves, dvo)
    ref_leaves = [x.double().requires_grad_() for x in (vf, vb, q, k)]
    rvo = cf.bidi_value(*ref_leaves, coo, True)
    ref = (rvo.detach(),) + torch.autograd.grad(rvo, ref_leaves, dvo.double())
    return co.shape[0], dmx, [cf.rel_err(x, y) for x, y in zip(got, ref)]


def dense_sampled_rows(drv, dev, B, T, H, W, layernorm, rows, seed=1003):
    """Third baseline configuration at a size where no full float64 yardstick fits: sampled (batch, row) pairs of
    the logits, dq and dk against the defining sums in float64, the checksum sum_t dq = -sum_s dk over everything,
    and bitwise repeatability of the backward.  `drv` is a driver binding with dense_forward(q, k) -> [attn] and
    dense_backward(d_attn, q, k) -> [dq, dk] (the reference's native interface, cuda/l1attn_cuda_drv.cpp:106-109).
    layernorm: inputs scaled to zero mean and unit variance per token and head, the configuration's second input set.
    Returns the worst errors (logits, dq, dk, checksum relative to the largest column sum)."""
    import math
    g = torch.Generator(device=dev).manual_seed(seed)
    q = torch.randn(B, T, H, W, generator=g, device=dev)
    k = torch.randn(B, T, H, W, generator=g, device=dev)
    if layernorm:
        q = torch.nn.functional.layer_norm(q, (W,))
        k = torch.nn.functional.layer_norm(k, (W,))
    da = torch.empty(B, T, T, H, device=dev)
    for b in range(B):  # one batch at a time: 1 GiB each at the full size
        da[b].normal_(generator=g)
    a = drv.dense_forward(q, k)[0]
    dq, dk = drv.dense_backward(da, q, k)
    dq2, dk2 = drv.dense_backward(da, q, k)
    assert torch.equal(dq, dq2) and torch.equal(dk, dk2)
    scale = -1.0 / math.sqrt(W)
    worst = [0.0, 0.0, 0.0]
    for b, r in rows:
        diff = q[b, r].double()[None] - k[b].double()                      # [S,H,W]: row r as dst token
        ra = scale * diff.abs().sum(-1)
        rdq = scale * (torch.sign(diff) * da[b, :, r, :, None].double()).sum(0)
        diff = q[b].double() - k[b, r].double()[None]                      # [T,H,W]: row r as src token
        rdk = -scale * (torch.sign(diff) * da[b, r, :, :, None].double()).sum(0)
        errs = (cf.rel_err(a[b, :, r, :], ra), cf.rel_err(dq[b, r], rdq), cf.rel_err(dk[b, r], rdk))
        worst = [max(x, y) for x, y in zip(worst, errs)]
    sq, sk = dq.double().sum(1), dk.double().sum(1)
    return worst + [float((sq + sk).abs().max()) / float(sq.abs().max())]
