"""Property tests of the CPU operator package against the oracle on random shapes and edge lists (hypothesis),
float64 so that the comparison is at rounding level, plus properties the mathematics fixes whatever the data:
the dense gradients cancel in total, the sparse operator ignores the order of the rows, and a bidirectional call
with a zero reverse value equals the one-directional operator."""
import pytest
import torch
from hypothesis import given, settings, strategies as st

import closed_forms as cf
from oracle import oracle

TOL = 1e-11
shapes = st.tuples(st.integers(1, 3), st.integers(1, 24), st.integers(1, 5), st.integers(1, 40))


@settings(max_examples=40, deadline=None)
@given(shape=shapes, seed=st.integers(0, 2 ** 31 - 1))
def test_dense_random_shapes(shape, seed):
    import _l1attn_cpu as drv
    B, T, H, W = shape
    g = torch.Generator().manual_seed(seed)
    q, k = (torch.randn(B, T, H, W, generator=g, dtype=torch.float64) for _ in range(2))
    q = torch.round(q * 4) / 4 if seed % 3 == 0 else q            # every third case: a coarse grid, many exact ties
    k = torch.round(k * 4) / 4 if seed % 3 == 0 else k
    da = torch.randn(B, T, T, H, generator=g, dtype=torch.float64)
    a = drv.dense_forward(q, k)[0]
    dq, dk = drv.dense_backward(da, q, k)
    assert cf.rel_err(a, oracle.dense_fwd(q, k)) <= TOL
    rdq, rdk = oracle.dense_bwd(da, q, k)
    assert cf.rel_err(dq, rdq) <= TOL and cf.rel_err(dk, rdk) <= TOL
    # every pair-element enters dq and dk with opposite signs, per (batch, head, column)
    assert float((dq.sum(1) + dk.sum(1)).abs().max()) <= 1e-9 * (1.0 + float(rdq.abs().sum()))


@settings(max_examples=40, deadline=None)
@given(shape=shapes, n_edges=st.integers(0, 120), seed=st.integers(0, 2 ** 31 - 1), sm=st.booleans())
def test_sparse_and_bidi_random_graphs(shape, n_edges, seed, sm):
    import _l1attn_cpu as drv
    B, T, H, W = shape
    g = torch.Generator().manual_seed(seed)
    co = torch.stack((torch.randint(0, T, (n_edges,), generator=g), torch.randint(0, T, (n_edges,), generator=g)), 1)
    coo, dmx, smx = drv.expand_coo(co)
    ocoo, odmx, osmx = oracle.expand_coo(co)
    assert torch.equal(coo, ocoo) and (dmx, smx) == (odmx, osmx)
    vf, vb, q, k, dvo = (torch.randn(B, T, H, W, generator=g, dtype=torch.float64) for _ in range(5))
    vo, attn = drv.sparse_forward(vf, q, k, coo, dmx, sm)
    rvo, rattn = oracle.sparse_fwd(vf, q, k, coo, dmx, sm)
    assert cf.rel_err(vo, rvo) <= TOL and cf.rel_err(attn, rattn) <= TOL
    for x, y in zip(drv.sparse_backward(dvo, vf, q, k, coo, attn, dmx, sm),
                    oracle.sparse_bwd(dvo, vf, q, k, coo, rattn, dmx, sm, 1)):
        assert cf.rel_err(x, y) <= TOL
    bvo, battn = drv.bidi_forward(vf, vb, q, k, coo, dmx, sm)
    rbvo, rbattn = oracle.bidi_fwd(vf, vb, q, k, coo, dmx, sm)
    assert cf.rel_err(bvo, rbvo) <= TOL
    for x, y in zip(drv.bidi_backward(dvo, vf, vb, q, k, coo, battn, dmx, sm),
                    oracle.bidi_bwd(dvo, vf, vb, q, k, coo, rbattn, dmx, sm, 1)):
        assert cf.rel_err(x, y) <= TOL
    # a zero reverse value makes the bidirectional operator the one-directional one
    zvo, _ = drv.bidi_forward(vf, torch.zeros_like(vb), q, k, coo, dmx, sm)
    assert cf.rel_err(zvo, vo) <= TOL
    # the order of the rows does not matter (the slots do change, the result does not)
    if n_edges > 1:
        perm = torch.randperm(n_edges, generator=g)
        pcoo, pdmx, _ = drv.expand_coo(co[perm])
        pvo, _ = drv.sparse_forward(vf, q, k, pcoo, pdmx, sm)
        assert cf.rel_err(pvo, vo) <= TOL
