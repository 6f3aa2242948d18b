"""Pins the CPU oracle (oracle/liboracle.so) before anything is compared with it.

Sources of truth, none of which is the oracle's own formula:
  * hand-computed answers for the reference's hand-made fixtures
    (testdense.py:20-35, python/l1attn_sparse.py:450-484 and :522-576, README.md:89);
  * golden vectors written by the reference's compiled CPU extension
    (tests/golden/ref_cpp_golden.npz, see tests/golden/make_golden.py);
  * independent vectorised closed forms + torch autograd + finite differences;
  * the invariants of check_sparse.py: full edge list == dense attention with the no-op
    logit, row-permutation invariance, edge dropping;
  * O(E^2) brute force for expandCoo.
"""
import math
import os

import numpy as np
import pytest
import torch

import closed_forms as cf
from oracle import oracle

GOLD = os.path.join(os.path.dirname(__file__), "golden", "ref_cpp_golden.npz")
F64 = dict(dtype=torch.float64)


def onehot_fixture():
    # testdense.py:20-34 / testsparse.py:34-48 (4 tokens there, the 4th all zero; W=4)
    q = torch.zeros(1, 4, 1, 4, **F64)
    k = torch.zeros(1, 4, 1, 4, **F64)
    v = torch.zeros(1, 4, 1, 4, **F64)
    q[0, 0, 0] = torch.tensor([0, 1, 0, 0.0])
    q[0, 1, 0] = torch.tensor([0, 0, 1, 0.0])
    q[0, 2, 0] = torch.tensor([1, 0, 0, 0.0])
    k[0, 0, 0] = torch.tensor([1, 0, 0, 0.0])
    k[0, 1, 0] = torch.tensor([0, 1, 0, 0.0])
    k[0, 2, 0] = torch.tensor([0, 0, 1, 0.0])
    v[0, 0, 0] = torch.tensor([1, 0, 0, 1.0])
    v[0, 1, 0] = torch.tensor([0, 1, 0, 2.0])
    v[0, 2, 0] = torch.tensor([0, 0, 1, 3.0])
    return q, k, v


def integer_fixture():
    # python/l1attn_sparse.py:450-482 (W=3)
    q = torch.tensor([[0, 1, 2], [2, 1, 0], [0, 0, 0]], **F64).reshape(1, 3, 1, 3)
    k = torch.tensor([[2, 1, 0], [0, 1, 2], [0, 1, 2]], **F64).reshape(1, 3, 1, 3)
    v = torch.tensor([[-2, 2, 3], [2, -2, 2], [3, 2, -2]], **F64).reshape(1, 3, 1, 3)
    return q, k, v


# ---------------------------------------------------------------- dense, known answers

def test_dense_fwd_onehot_hand_answer():
    q, k, _ = onehot_fixture()
    a = oracle.dense_fwd(q, k)[0, :, :, 0]  # [s, t]
    # L1 distances by hand, times -1/sqrt(4) = -0.5; rows = src s, cols = dst t
    expect = torch.tensor([
        [-1.0, -1.0, 0.0, -0.5],   # k0=[1,0,0,0] vs q0,q1,q2,q3
        [0.0, -1.0, -1.0, -0.5],   # k1=[0,1,0,0]
        [-1.0, 0.0, -1.0, -0.5],   # k2=[0,0,1,0]
        [-0.5, -0.5, -0.5, 0.0],   # k3=0
    ], **F64)
    assert torch.equal(a, expect)
    # a transposed implementation fails this fixture:
    assert not torch.equal(expect, expect.T)


def test_dense_fwd_integer_hand_answer():
    q, k, _ = integer_fixture()
    a = oracle.dense_fwd(q, k)[0, :, :, 0]
    l1 = torch.tensor([[4.0, 0, 3], [0, 4, 3], [0, 4, 3]], **F64)  # [s,t] by hand
    assert torch.allclose(a, -l1 / math.sqrt(3.0), rtol=0, atol=1e-15)


def test_dense_fwd_float32_variant_matches_float64():
    g = torch.Generator().manual_seed(5)
    q = torch.randn(2, 9, 3, 33, generator=g)
    k = torch.randn(2, 9, 3, 33, generator=g)
    a32 = oracle.dense_fwd(q, k)
    a64 = oracle.dense_fwd(q.double(), k.double())
    assert a32.dtype == torch.float32
    assert cf.rel_err(a32, a64) < 1e-6


# ------------------------------------------------- dense, closed forms and derivatives

@pytest.mark.parametrize("shape", [(2, 5, 3, 7), (1, 16, 2, 64), (3, 1, 1, 1), (1, 4, 5, 2)])
def test_dense_fwd_bwd_vs_autograd_closed_form(shape):
    B, T, H, W = shape
    g = torch.Generator().manual_seed(B * 1000 + T * 100 + H * 10 + W)
    q = torch.randn(B, T, H, W, generator=g, **F64).requires_grad_()
    k = torch.randn(B, T, H, W, generator=g, **F64).requires_grad_()
    da = torch.randn(B, T, T, H, generator=g, **F64)
    a = cf.dense_attn(q, k)
    a.backward(da)
    assert torch.allclose(oracle.dense_fwd(q.detach(), k.detach()), a.detach(), rtol=1e-13, atol=1e-13)
    dq, dk = oracle.dense_bwd(da, q.detach(), k.detach())
    assert torch.allclose(dq, q.grad, rtol=1e-12, atol=1e-12)
    assert torch.allclose(dk, k.grad, rtol=1e-12, atol=1e-12)
    # invariant: every pair contributes +x to dq and -x to dk
    assert torch.allclose(dq.sum(1), -dk.sum(1), rtol=1e-10, atol=1e-10)


def test_dense_bwd_ties_give_zero():
    q, k, _ = onehot_fixture()
    da = torch.ones(1, 4, 4, 1, **F64)
    dq, dk = oracle.dense_bwd(da, q, k)
    # q3 = 0 and k3 = 0 tie in all 4 channels; against k0..k2 (one-hot) only the hot
    # channel differs: dq[3, w] = scale * sum_s sign(0 - k[s,w]) = -0.5 * (-1) = +0.5 for w<3
    assert torch.equal(dq[0, 3, 0], torch.tensor([0.5, 0.5, 0.5, 0.0], **F64))
    # q0=[0,1,0,0]: channel 1: vs k0(0):+1, k1(1):0, k2(0):+1, k3(0):+1 -> -0.5*3
    assert dq[0, 0, 0, 1].item() == -1.5


def test_dense_bwd_finite_differences():
    g = torch.Generator().manual_seed(11)
    q = torch.randn(1, 3, 2, 4, generator=g, **F64)
    k = torch.randn(1, 3, 2, 4, generator=g, **F64)
    da = torch.randn(1, 3, 3, 2, generator=g, **F64)
    dq, dk = oracle.dense_bwd(da, q, k)
    eps = 1e-6
    for (x, gx, which) in ((q, dq, 0), (k, dk, 1)):
        num = torch.zeros_like(x)
        flat = x.view(-1)
        for i in range(flat.numel()):
            old = flat[i].item()
            flat[i] = old + eps
            fp = (oracle.dense_fwd(q, k) * da).sum().item()
            flat[i] = old - eps
            fm = (oracle.dense_fwd(q, k) * da).sum().item()
            flat[i] = old
            num.view(-1)[i] = (fp - fm) / (2 * eps)
        assert torch.allclose(gx, num, rtol=1e-6, atol=1e-7), which


# ------------------------------------------------------------- golden vectors (_ref)

def _gold():
    return np.load(GOLD)


@pytest.mark.parametrize("tag", ["dA", "dB"])
def test_dense_matches_reference_extension_golden(tag):
    z = _gold()
    t = lambda n: torch.from_numpy(z[f"{tag}_{n}"])
    a = oracle.dense_fwd(t("q"), t("k"))
    dq, dk = oracle.dense_bwd(t("da"), t("q"), t("k"))
    assert torch.allclose(a, t("attn"), rtol=1e-14, atol=1e-14)
    assert torch.allclose(dq, t("dq"), rtol=1e-13, atol=1e-13)
    assert torch.allclose(dk, t("dk"), rtol=1e-13, atol=1e-13)


@pytest.mark.parametrize("tag", ["sA", "sB"])
@pytest.mark.parametrize("sm", [True, False])
def test_sparse_and_bidi_match_reference_extension_golden(tag, sm):
    z = _gold()
    s = "sm" if sm else "nsm"
    t = lambda n: torch.from_numpy(z[f"{tag}_{n}"])
    coo, dmx = t("coo"), int(z[f"{tag}_mx"][0])
    vo, attn = oracle.sparse_fwd(t("v"), t("q"), t("k"), coo, dmx, sm)
    assert torch.allclose(vo, t(f"{s}_vo"), rtol=1e-13, atol=1e-13)
    assert torch.allclose(attn, t(f"{s}_attn"), rtol=1e-13, atol=1e-13)
    for jac in (0, 1):
        dv, dq, dk = oracle.sparse_bwd(t("dvo"), t("v"), t("q"), t("k"), coo, attn, dmx, sm, jac)
        assert torch.allclose(dv, t(f"{s}_dv"), rtol=1e-12, atol=1e-12)
        assert torch.allclose(dq, t(f"{s}_dq"), rtol=1e-12, atol=1e-12)
        assert torch.allclose(dk, t(f"{s}_dk"), rtol=1e-12, atol=1e-12)
    vo, attn = oracle.bidi_fwd(t("v"), t("vb"), t("q"), t("k"), coo, dmx, sm)
    assert torch.allclose(vo, t(f"{s}_bidi_vo"), rtol=1e-13, atol=1e-13)
    for jac in (0, 1):
        outs = oracle.bidi_bwd(t("dvo"), t("v"), t("vb"), t("q"), t("k"), coo, attn, dmx, sm, jac)
        for got, n in zip(outs, ("dvf", "dvb", "dq", "dk")):
            assert torch.allclose(got, t(f"{s}_bidi_{n}"), rtol=1e-12, atol=1e-12), n


def test_live_reference_extension_when_built():
    """When oracle/_ref exists (build container, or carried to the GPU box) compare live."""
    mods = oracle.ref_modules()
    if mods is None:
        pytest.skip("oracle/_ref not built")
    g = torch.Generator().manual_seed(77)
    q, k, v, vb, dvo = (torch.randn(2, 7, 3, 5, generator=g, **F64) for _ in range(5))
    da = torch.randn(2, 7, 7, 3, generator=g, **F64)
    (a,) = mods["l1attn_drv_cpp"].forward(q, k)
    assert torch.equal(oracle.dense_fwd(q, k), a)
    dq, dk = mods["l1attn_drv_cpp"].backward(da, q, k)
    odq, odk = oracle.dense_bwd(da, q, k)
    assert torch.allclose(odq, dq, rtol=1e-14, atol=1e-14) and torch.allclose(odk, dk, rtol=1e-14, atol=1e-14)
    co = torch.randint(0, 7, (30, 2), generator=g)
    coo, dmx, _ = oracle.expand_coo(co)
    for sm in (True, False):
        vo, attn = mods["l1attn_sparse_drv"].forward(v, q, k, coo, dmx, sm)
        ovo, oattn = oracle.sparse_fwd(v, q, k, coo, dmx, sm)
        assert torch.allclose(ovo, vo, rtol=1e-14, atol=1e-14)
        ref = mods["l1attn_sparse_drv"].backward(dvo, v, q, k, coo, attn, dmx, sm)
        for a_, b_ in zip(oracle.sparse_bwd(dvo, v, q, k, coo, oattn, dmx, sm), ref):
            assert torch.allclose(a_, b_, rtol=1e-13, atol=1e-13)
        vo, attn = mods["l1attn_sparse_bidi_drv"].forward(v, vb, q, k, coo, dmx, sm)
        ovo, oattn = oracle.bidi_fwd(v, vb, q, k, coo, dmx, sm)
        assert torch.allclose(ovo, vo, rtol=1e-14, atol=1e-14)
        ref = mods["l1attn_sparse_bidi_drv"].backward(dvo, v, vb, q, k, coo, attn, dmx, sm)
        for a_, b_ in zip(oracle.bidi_bwd(dvo, v, vb, q, k, coo, oattn, dmx, sm), ref):
            assert torch.allclose(a_, b_, rtol=1e-13, atol=1e-13)


# ------------------------------------------------------------------ sparse invariants

@pytest.mark.parametrize("sm", [True, False])
def test_sparse_full_list_equals_dense_with_noop(sm):
    # python/l1attn_sparse.py:488-512 on its integer fixture, and testsparse.py:50-62
    for q, k, v in (integer_fixture(), onehot_fixture()):
        T = q.shape[1]
        co = torch.cartesian_prod(torch.arange(T), torch.arange(T))
        coo, dmx, smx = oracle.expand_coo(co)
        vo, _ = oracle.sparse_fwd(v, q, k, coo, dmx, sm)
        expect = cf.dense_then_value(q, k, v, noop=sm) if sm else \
            torch.einsum("bsdh,bshw->bdhw", oracle.dense_fwd(q, k).exp(), v)
        assert torch.allclose(vo, expect, rtol=1e-13, atol=1e-13)
        perm = torch.randperm(co.shape[0], generator=torch.Generator().manual_seed(3))
        coo2, dmx2, _ = oracle.expand_coo(co[perm])
        vo2, _ = oracle.sparse_fwd(v, q, k, coo2, dmx2, sm)
        assert torch.allclose(vo2, expect, rtol=1e-13, atol=1e-13)


def test_fused_forward_oracle_pins():
    """oracle.fused_fwd (dense logits, no-op row, softmax over src, value sum) against three statements
    that share no code with it: the sparse oracle over the full cartesian list (itself pinned by the
    reference extension's golden vectors), the broadcast closed form, and a hand answer on the integer
    fixture (python/l1attn_sparse.py:450-470; W = 3)."""
    for q, k, v in (integer_fixture(), onehot_fixture()):
        T = q.shape[1]
        vo, lse = oracle.fused_fwd(q, k, v)
        coo, dmx, _ = oracle.expand_coo(torch.cartesian_prod(torch.arange(T), torch.arange(T)))
        ref, _ = oracle.sparse_fwd(v, q, k, coo, dmx, True)
        assert torch.allclose(vo, ref, rtol=1e-13, atol=1e-13)
        assert torch.allclose(vo, cf.dense_then_value(q, k, v, noop=True), rtol=1e-13, atol=1e-13)
        den = 1.0 + cf.dense_attn(q, k).exp().sum(1)
        assert torch.allclose(lse, den.log(), rtol=1e-13, atol=1e-13)
    # a transposed src/dst or a dropped "+1" must fail: asymmetric random case, denominators near 1
    g = torch.Generator().manual_seed(12)
    q, k, v = (torch.randn(2, 5, 3, 4, generator=g, dtype=torch.float64) for _ in range(3))
    vo, lse = oracle.fused_fwd(q, k, v)
    for b, t, h in ((0, 0, 0), (1, 4, 2), (0, 3, 1)):
        e = [math.exp(-float((q[b, t, h] - k[b, s, h]).abs().sum()) / 2.0) for s in range(5)]  # sqrt(4) = 2
        expect = sum(e[s] * v[b, s, h] for s in range(5)) / (1.0 + sum(e))
        assert torch.allclose(vo[b, t, h], expect, rtol=1e-13, atol=1e-15)
        assert abs(float(lse[b, t, h]) - math.log(1.0 + sum(e))) < 1e-13


def test_fused_backward_oracle_pins():
    """oracle.fused_bwd (hand-differentiated softmax and einsum, then the reference's dense backward loop) against
    torch autograd through the broadcast closed form, against the sparse oracle's backward over the full cartesian
    list (pinned by the reference extension's golden vectors), and by finite differences on one element each."""
    g = torch.Generator().manual_seed(21)
    B, T, H, W = 2, 6, 3, 4
    q, k, v, dvo = (torch.randn(B, T, H, W, generator=g, dtype=torch.float64) for _ in range(4))
    dq, dk, dv = oracle.fused_bwd(dvo, q, k, v)
    x = [t.clone().requires_grad_() for t in (q, k, v)]
    ref = torch.autograd.grad(cf.dense_then_value(*x, noop=True), x, dvo)
    for a, b in zip((dq, dk, dv), ref):
        assert torch.allclose(a, b, rtol=1e-12, atol=1e-13)
    coo, dmx, _ = oracle.expand_coo(torch.cartesian_prod(torch.arange(T), torch.arange(T)))
    _, attn = oracle.sparse_fwd(v, q, k, coo, dmx, True)
    sdv, sdq, sdk = oracle.sparse_bwd(dvo, v, q, k, coo, attn, dmx, True, 0)
    for a, b in zip((dq, dk, dv), (sdq, sdk, sdv)):
        assert torch.allclose(a, b, rtol=1e-11, atol=1e-12)
    loss = lambda q_, k_, v_: float((oracle.fused_fwd(q_, k_, v_)[0] * dvo).sum())
    eps = 1e-6
    for which, grad in ((0, dq), (1, dk), (2, dv)):
        args = [q.clone(), k.clone(), v.clone()]
        args[which][1, 2, 1, 3] += eps
        up = loss(*args)
        args[which][1, 2, 1, 3] -= 2 * eps
        assert abs((up - loss(*args)) / (2 * eps) - float(grad[1, 2, 1, 3])) < 1e-7


def test_sparse_integer_fixture_hand_answer():
    # python/l1attn_sparse.py:484 : co = [[0,0],[0,1],[1,0],[1,1],[2,2]], softmax on.
    # dst 0 sees k0 (L1=4) and k1 (L1=0): e = exp(-4/sqrt3), 1 ; denominator 1 + e + 1.
    q, k, v = integer_fixture()
    co = torch.tensor([[0, 0], [0, 1], [1, 0], [1, 1], [2, 2]])
    coo, dmx, _ = oracle.expand_coo(co)
    vo, _ = oracle.sparse_fwd(v, q, k, coo, dmx, True)
    e4, e3 = math.exp(-4 / math.sqrt(3)), math.exp(-3 / math.sqrt(3))
    v0, v1, v2 = v[0, 0, 0], v[0, 1, 0], v[0, 2, 0]
    assert torch.allclose(vo[0, 0, 0], (e4 * v0 + 1.0 * v1) / (2 + e4), rtol=1e-14, atol=0)
    assert torch.allclose(vo[0, 1, 0], (1.0 * v0 + e4 * v1) / (2 + e4), rtol=1e-14, atol=0)
    assert torch.allclose(vo[0, 2, 0], e3 * v2 / (1 + e3), rtol=1e-14, atol=0)


def _rand_graph(g, T, E):
    return torch.randint(0, T, (E, 2), generator=g)


@pytest.mark.parametrize("sm", [True, False])
def test_sparse_and_bidi_vs_autograd_closed_form(sm):
    g = torch.Generator().manual_seed(101)
    B, T, H, W, E = 2, 9, 3, 5, 40
    co = _rand_graph(g, T, E)  # duplicates and empty dst rows occur
    coo, dmx, smx = oracle.expand_coo(co)
    v, vb, q, k = (torch.randn(B, T, H, W, generator=g, **F64).requires_grad_() for _ in range(4))
    dvo = torch.randn(B, T, H, W, generator=g, **F64)
    out = cf.sparse_value(v, q, k, coo, sm)
    gv, gq, gk = torch.autograd.grad(out, (v, q, k), dvo)
    vo, attn = oracle.sparse_fwd(v.detach(), q.detach(), k.detach(), coo, dmx, sm)
    assert torch.allclose(vo, out.detach(), rtol=1e-12, atol=1e-13)
    for jac in (0, 1):
        dv, dq, dk = oracle.sparse_bwd(dvo, v.detach(), q.detach(), k.detach(), coo, attn, dmx, sm, jac)
        for a_, b_ in ((dv, gv), (dq, gq), (dk, gk)):
            assert torch.allclose(a_, b_, rtol=1e-11, atol=1e-12)
    out = cf.bidi_value(v, vb, q, k, coo, sm)
    gs = torch.autograd.grad(out, (v, vb, q, k), dvo)
    vo, attn = oracle.bidi_fwd(v.detach(), vb.detach(), q.detach(), k.detach(), coo, dmx, sm)
    assert torch.allclose(vo, out.detach(), rtol=1e-12, atol=1e-13)
    outs = oracle.bidi_bwd(dvo, v.detach(), vb.detach(), q.detach(), k.detach(), coo, attn, dmx, sm, 1)
    for a_, b_ in zip(outs, gs):
        assert torch.allclose(a_, b_, rtol=1e-11, atol=1e-12)
    # bidi with vb = 0 is the one-directional operator
    z = torch.zeros_like(vb.detach())
    vo_b, _ = oracle.bidi_fwd(v.detach(), z, q.detach(), k.detach(), coo, dmx, sm)
    vo_u, _ = oracle.sparse_fwd(v.detach(), q.detach(), k.detach(), coo, dmx, sm)
    assert torch.equal(vo_b, vo_u)


def test_bidi_fixture_hand_answer():
    # python/l1attn_sparse.py:522-578, use_softmax=False: p = exp(-L1/sqrt3)
    q, k, _ = integer_fixture()
    vf = torch.diag(torch.tensor([1.0, 2, 3], **F64)).reshape(1, 3, 1, 3)
    vb = -vf
    co = torch.tensor([[0, 0], [0, 1], [0, 2], [1, 0], [1, 1], [2, 0], [2, 1]])
    coo, dmx, smx = oracle.expand_coo(co)
    vo, _ = oracle.bidi_fwd(vf, vb, q, k, coo, dmx, False)
    l1 = {(0, 0): 4, (0, 1): 0, (0, 2): 0, (1, 0): 0, (1, 1): 4, (2, 0): 3, (2, 1): 3}  # (dst,src)
    expect = torch.zeros(3, 3, **F64)
    for (d, s), dist in l1.items():
        p = math.exp(-dist / math.sqrt(3))
        expect[d] += p * vf[0, s, 0]
        expect[s] += p * vb[0, d, 0]
    assert torch.allclose(vo[0, :, 0], expect, rtol=1e-14, atol=1e-15)


# ------------------------------------------------------------------------- expandCoo

def test_expand_coo_known_answers():
    # README.md:89 / check_sparse.py:43
    co = torch.cartesian_prod(torch.arange(3), torch.arange(3))
    coo, dmx, smx = oracle.expand_coo(co)
    assert coo[:, 2].tolist() == [0, 1, 2, 0, 1, 2, 0, 1, 2]
    assert coo[:, 3].tolist() == [0, 0, 0, 1, 1, 1, 2, 2, 2]
    assert (dmx, smx) == (3, 3) and coo.dtype == torch.int32
    # python/l1attn_sparse.py:576
    co = torch.tensor([[0, 0], [0, 1], [0, 2], [1, 0], [1, 1], [2, 0], [2, 1]])
    coo, dmx, smx = oracle.expand_coo(co)
    assert coo[:, 2].tolist() == [0, 1, 2, 0, 1, 0, 1]
    assert coo[:, 3].tolist() == [0, 0, 0, 1, 1, 2, 2]
    assert (dmx, smx) == (3, 3)
    coo, dmx, smx = oracle.expand_coo(torch.zeros(0, 2, dtype=torch.int64))
    assert coo.shape == (0, 4) and (dmx, smx) == (1, 1)


@pytest.mark.parametrize("seed", [0, 1, 2])
def test_expand_coo_bruteforce(seed):
    g = torch.Generator().manual_seed(seed)
    co = torch.randint(0, 13, (200, 2), generator=g)
    coo, dmx, smx = oracle.expand_coo(co)
    bcoo, bd, bs = cf.expand_coo_bruteforce(co)
    assert torch.equal(coo, bcoo) and (dmx, smx) == (bd, bs)
