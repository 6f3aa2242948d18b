"""GPU parity of expandCoo, sparse and bidirectional sparse L1 attention: HIP library through the
reference's Python API (and so through the C ABI) against the CPU oracle / fp64 closed forms.

Tolerances (max|x-ref|/max|ref| against fp64 on the same fp32-valued inputs): forward <= 1e-5,
gradients <= 1e-4; fp64 entry points <= 1e-11; expandCoo bit-exact.
"""
import os

import numpy as np
import pytest
import torch

import closed_forms as cf
import workloads
from oracle import oracle

pytestmark = pytest.mark.gpu

FWD_TOL, BWD_TOL, F64_TOL = 1e-5, 1e-4, 1e-11


def _m():
    import l1attn_sparse_cuda
    import l1attn_sparse_bidi_cuda
    return l1attn_sparse_cuda, l1attn_sparse_bidi_cuda


# --------------------------------------------------------------------------------- expandCoo

def test_expand_coo_known_answers():
    sp, bi = _m()
    co = torch.cartesian_prod(torch.arange(3), torch.arange(3))  # README.md:89
    for mod in (sp, bi):
        coo, dmx, smx = mod.expandCoo(co)
        assert coo.dtype == torch.int32 and coo.device == co.device and tuple(coo.shape) == (9, 4)
        assert coo[:, 2].tolist() == [0, 1, 2, 0, 1, 2, 0, 1, 2]
        assert coo[:, 3].tolist() == [0, 0, 0, 1, 1, 1, 2, 2, 2]
        assert (dmx, smx) == (3, 3)
    co = torch.tensor([[0, 0], [0, 1], [0, 2], [1, 0], [1, 1], [2, 0], [2, 1]]).cuda()  # python/l1attn_sparse.py:576
    coo, dmx, smx = sp.expandCoo(co)
    assert coo.is_cuda
    assert coo[:, 2].tolist() == [0, 1, 2, 0, 1, 0, 1] and coo[:, 3].tolist() == [0, 0, 0, 1, 1, 2, 2]
    coo, dmx, smx = sp.expandCoo(torch.zeros(0, 2, dtype=torch.int64))
    assert tuple(coo.shape) == (0, 4) and (dmx, smx) == (1, 1)


@pytest.mark.parametrize("E,K,dtype", [(1, 1, torch.int64), (777, 13, torch.int64), (5000, 50, torch.int32),
                                        (4097, 300, torch.int64), (200000, 65536, torch.int64),
                                        (300000, 70000, torch.int32), (50000, 3, torch.int64),
                                        (100000, 20000000, torch.int64)])
def test_expand_coo_bit_exact_vs_oracle(E, K, dtype):
    print("case expandCoo", E, K, dtype, flush=True)
    sp, _ = _m()
    g = torch.Generator().manual_seed(E + K)
    co = torch.randint(0, K, (E, 2), generator=g).to(dtype)
    ocoo, odmx, osmx = oracle.expand_coo(co)
    coo, dmx, smx = sp.expandCoo(co.cuda(), warn=False)
    assert torch.equal(coo.cpu(), ocoo) and (dmx, smx) == (odmx, osmx)


def test_expand_coo_benchmark_graphs_and_warnings(capsys):
    sp, bi = _m()
    co = workloads.uniform_degree_graph(512, 64, seed=1004)
    ocoo, odmx, osmx = oracle.expand_coo(co)
    coo, dmx, smx = sp.expandCoo(co.cuda(), warn=False)
    assert torch.equal(coo.cpu(), ocoo) and (dmx, smx) == (odmx, osmx)
    co = workloads.powerlaw_graph(4096, seed=1005)
    ocoo, odmx, osmx = oracle.expand_coo(co)
    coo, dmx, smx = bi.expandCoo(co.cuda(), warn=False)
    assert torch.equal(coo.cpu(), ocoo) and (dmx, smx) == (odmx, osmx)
    # warnings (stdout), python/l1attn_sparse.py:419-424 wording in the bidi copy
    capsys.readouterr()
    bi.expandCoo(torch.tensor([[0, 0], [2, 3]]))
    out = capsys.readouterr().out
    assert "Warning: degenerate sparse head - 1 not written" in out
    assert "Warning degenerate sparse head - 1 not read" in out and "2 not read" in out
    with pytest.raises(RuntimeError):
        sp.expandCoo(torch.tensor([[0, -1]]))


# ------------------------------------------------------------------------------ sparse / bidi

def _run_uni(v, q, k, coo, dmx, sm, dvo):
    sp, _ = _m()
    vd, qd, kd = (x.cuda().requires_grad_() for x in (v, q, k))
    vo = sp.L1AttnSparseFn.apply(vd, qd, kd, coo.cuda(), dmx, sm)
    vo.backward(dvo.cuda())
    torch.cuda.synchronize()
    return vo.detach().cpu(), vd.grad.cpu(), qd.grad.cpu(), kd.grad.cpu()


def _run_bidi(vf, vb, q, k, coo, dmx, sm, dvo):
    _, bi = _m()
    a, b, qd, kd = (x.cuda().requires_grad_() for x in (vf, vb, q, k))
    vo = bi.L1AttnSparseBidiFn.apply(a, b, qd, kd, coo.cuda(), dmx, sm)
    vo.backward(dvo.cuda())
    torch.cuda.synchronize()
    return vo.detach().cpu(), a.grad.cpu(), b.grad.cpu(), qd.grad.cpu(), kd.grad.cpu()


def _check(got, ref, tols):
    for i, (a, b, tol) in enumerate(zip(got, ref, tols)):
        err = cf.rel_err(a, b)
        assert err <= tol, (i, err)


def _oracle_uni(v, q, k, coo, dmx, sm, dvo, jac=0):
    v, q, k, dvo = (x.double() for x in (v, q, k, dvo))
    vo, attn = oracle.sparse_fwd(v, q, k, coo, dmx, sm)
    return (vo,) + tuple(oracle.sparse_bwd(dvo, v, q, k, coo, attn, dmx, sm, jac))


def _oracle_bidi(vf, vb, q, k, coo, dmx, sm, dvo, jac=0):
    vf, vb, q, k, dvo = (x.double() for x in (vf, vb, q, k, dvo))
    vo, attn = oracle.bidi_fwd(vf, vb, q, k, coo, dmx, sm)
    return (vo,) + tuple(oracle.bidi_bwd(dvo, vf, vb, q, k, coo, attn, dmx, sm, jac))


def _edge_lists_check_sparse(T, g):
    """The three edge lists of check_sparse.py:43-74: full, permuted, permuted minus four rows."""
    co = torch.cartesian_prod(torch.arange(T), torch.arange(T))
    perm = torch.randperm(co.shape[0], generator=g)
    return [co, co[perm], co[perm[:-4]]]


@pytest.mark.parametrize("dtype", [torch.float64, torch.float32])
@pytest.mark.parametrize("sm", [True, False])
def test_check_sparse_cases_vs_oracle(dtype, sm):
    # check_sparse.py:18-21: B=2, T=3, H=16, W=7
    print("case check_sparse", dtype, sm, flush=True)
    g = torch.Generator().manual_seed(31)
    B, T, H, W = 2, 3, 16, 7
    v, vb, q, k, dvo = (torch.randn(B, T, H, W, generator=g, dtype=dtype) for _ in range(5))
    tols_u = [F64_TOL] * 4 if dtype == torch.float64 else [FWD_TOL] + [BWD_TOL] * 3
    tols_b = [F64_TOL] * 5 if dtype == torch.float64 else [FWD_TOL] + [BWD_TOL] * 4
    for co in _edge_lists_check_sparse(T, g):
        coo, dmx, smx = oracle.expand_coo(co)
        _check(_run_uni(v, q, k, coo, dmx, sm, dvo), _oracle_uni(v, q, k, coo, dmx, sm, dvo), tols_u)
        _check(_run_bidi(v, vb, q, k, coo, dmx, sm, dvo), _oracle_bidi(v, vb, q, k, coo, dmx, sm, dvo), tols_b)


SHAPES = [
    # B, T, H, W, E
    (2, 9, 3, 5, 40),       # duplicates, dst rows without edges
    (1, 64, 8, 32, 900),    # config-4 head geometry: 8 heads x 8 lanes
    (2, 50, 4, 64, 700),    # config-5 head geometry: 4 heads x 16 lanes
    (1, 40, 20, 16, 500),   # more heads than one wave holds
    (1, 30, 2, 70, 300),    # scalar loads, several column chunks per lane
    (1, 20, 2, 320, 150),   # vector loads, several column chunks per lane
    (1, 33, 5, 1, 200),     # width 1
]


@pytest.mark.parametrize("shape", SHAPES)
@pytest.mark.parametrize("sm", [True, False])
def test_sparse_and_bidi_f32_vs_oracle(shape, sm):
    B, T, H, W, E = shape
    print("case sparse f32", shape, sm, flush=True)
    g = torch.Generator().manual_seed(sum(shape))
    co = torch.randint(0, T, (E, 2), generator=g)
    coo, dmx, smx = oracle.expand_coo(co)
    v, vb, q, k, dvo = (torch.randn(B, T, H, W, generator=g) for _ in range(5))
    _check(_run_uni(v, q, k, coo, dmx, sm, dvo), _oracle_uni(v, q, k, coo, dmx, sm, dvo, 1),
           [FWD_TOL] + [BWD_TOL] * 3)
    _check(_run_bidi(v, vb, q, k, coo, dmx, sm, dvo), _oracle_bidi(v, vb, q, k, coo, dmx, sm, dvo, 1),
           [FWD_TOL] + [BWD_TOL] * 4)


@pytest.mark.parametrize("tag", ["sA", "sB"])
@pytest.mark.parametrize("sm", [True, False])
def test_sparse_golden_reference_extension(tag, sm):
    """Inputs and outputs written by the reference's compiled CPU extension (fp64)."""
    print("case sparse golden", tag, sm, flush=True)
    z = np.load(os.path.join(os.path.dirname(__file__), "golden", "ref_cpp_golden.npz"))
    s = "sm" if sm else "nsm"
    t = lambda n: torch.from_numpy(z[f"{tag}_{n}"])
    coo, dmx = t("coo"), int(z[f"{tag}_mx"][0])
    got = _run_uni(t("v"), t("q"), t("k"), coo, dmx, sm, t("dvo"))
    _check(got, [t(f"{s}_vo"), t(f"{s}_dv"), t(f"{s}_dq"), t(f"{s}_dk")], [F64_TOL] * 4)
    got = _run_bidi(t("v"), t("vb"), t("q"), t("k"), coo, dmx, sm, t("dvo"))
    _check(got, [t(f"{s}_bidi_{n}") for n in ("vo", "dvf", "dvb", "dq", "dk")], [F64_TOL] * 5)
    # and expandCoo of the stored raw list reproduces the stored coo
    sp, _ = _m()
    coo2, dmx2, _ = sp.expandCoo(t("co"), warn=False)
    assert torch.equal(coo2, coo) and dmx2 == dmx


@pytest.mark.parametrize("sm", [True, False])
def test_sparse_full_list_equals_dense_attention(sm):
    """check_sparse invariant (i): full cartesian list == dense L1 attention with the no-op logit
    (python/l1attn_sparse.py:488-506), with the dense side computed by the dense HIP kernels."""
    print("case sparse == dense", sm, flush=True)
    import l1attn_cuda
    sp, _ = _m()
    g = torch.Generator().manual_seed(9)
    B, T, H, W = 2, 48, 4, 32
    v, q, k = (torch.randn(B, T, H, W, generator=g).cuda() for _ in range(3))
    co = torch.cartesian_prod(torch.arange(T), torch.arange(T))
    co = co[torch.randperm(co.shape[0], generator=g)]
    coo, dmx, _ = sp.expandCoo(co.cuda(), warn=False)
    vo = sp.L1AttnSparse()(v, q, k, coo, dmx, sm)
    a = l1attn_cuda.L1Attn()(q, k)
    if sm:
        a = torch.cat((a, torch.zeros(B, 1, T, H, device="cuda")), 1)  # testsparse.py:52-55
        p = torch.softmax(a, 1)[:, :-1]
    else:
        p = a.exp()
    ref = torch.einsum("bsdh,bshw->bdhw", p, v)
    assert cf.rel_err(vo.cpu(), ref.cpu().double()) <= 2e-5
    # README.md:93 calls the module with five arguments
    vo5 = sp.L1AttnSparse()(v, q, k, coo, dmx)
    if sm:
        assert torch.equal(vo5, vo)


def test_sparse_permutation_invariance_and_determinism():
    print("case sparse permutation", flush=True)
    sp, bi = _m()
    g = torch.Generator().manual_seed(17)
    B, T, H, W = 2, 128, 8, 32
    co = workloads.uniform_degree_graph(T, 16, seed=4)
    v, vb, q, k, dvo = (torch.randn(B, T, H, W, generator=g) for _ in range(5))
    coo, dmx, _ = oracle.expand_coo(co)
    r1 = _run_bidi(v, vb, q, k, coo, dmx, True, dvo)
    r2 = _run_bidi(v, vb, q, k, coo, dmx, True, dvo)
    for a, b in zip(r1, r2):
        assert torch.equal(a, b)  # bitwise run-to-run
    coo2, dmx2, _ = oracle.expand_coo(co[torch.randperm(co.shape[0], generator=g)])
    r3 = _run_bidi(v, vb, q, k, coo2, dmx2, True, dvo)
    _check(r3, [x.double() for x in r1], [1e-6] * 5)  # same sums in another order
    # bidi with vb = 0 is the one-directional operator
    ru = _run_uni(v, q, k, coo, dmx, True, dvo)
    rb = _run_bidi(v, torch.zeros_like(vb), q, k, coo, dmx, True, dvo)
    assert torch.equal(ru[0], rb[0]) and torch.equal(ru[1], rb[1])


@pytest.mark.parametrize("dtype", [torch.float32, torch.float64])
def test_sparse_long_segments_vs_oracle(dtype):
    """Segments longer than 128 edges are walked by a whole workgroup (eight waves, fixed-order
    combine): a hub dst with 700 incoming edges, a hub src with 500 outgoing ones, duplicates, and a
    segment of exactly 128 and 129 edges on either side of the threshold."""
    print("case sparse long segments", dtype, flush=True)
    g = torch.Generator().manual_seed(77)
    B, T, H, W = 2, 300, 4, 16
    rows = [torch.stack((torch.full((700,), 5), torch.randint(0, T, (700,), generator=g)), 1),
            torch.stack((torch.randint(0, T, (500,), generator=g), torch.full((500,), 9)), 1),
            torch.stack((torch.full((128,), 20), torch.arange(128)), 1),
            torch.stack((torch.full((129,), 21), torch.arange(129)), 1),
            torch.randint(0, T, (400, 2), generator=g)]
    co = torch.cat(rows, 0)
    co = co[torch.randperm(co.shape[0], generator=g)]
    coo, dmx, smx = oracle.expand_coo(co)
    assert dmx > 700 and smx > 500
    v, vb, q, k, dvo = (torch.randn(B, T, H, W, generator=g, dtype=dtype) for _ in range(5))
    f32 = dtype == torch.float32
    for sm in (True, False):
        _check(_run_uni(v, q, k, coo, dmx, sm, dvo), _oracle_uni(v, q, k, coo, dmx, sm, dvo, 1),
               [FWD_TOL] + [BWD_TOL] * 3 if f32 else [F64_TOL] * 4)
        _check(_run_bidi(v, vb, q, k, coo, dmx, sm, dvo), _oracle_bidi(v, vb, q, k, coo, dmx, sm, dvo, 1),
               [FWD_TOL] + [BWD_TOL] * 4 if f32 else [F64_TOL] * 5)
    r1 = _run_bidi(v, vb, q, k, coo, dmx, True, dvo)
    r2 = _run_bidi(v, vb, q, k, coo, dmx, True, dvo)
    for a, b in zip(r1, r2):
        assert torch.equal(a, b)


def test_sparse_value_width_differs_from_key_width():
    # allowed by the reference's CUDA path (v_width, cuda/l1attn_sparse_cuda_kernel.cu:385)
    print("case sparse Wv != W", flush=True)
    sp, _ = _m()
    g = torch.Generator().manual_seed(23)
    B, T, H, W, Wv = 2, 20, 3, 8, 12
    co = torch.randint(0, T, (90, 2), generator=g)
    coo, dmx, _ = oracle.expand_coo(co)
    q, k = (torch.randn(B, T, H, W, generator=g, dtype=torch.float64).cuda().requires_grad_() for _ in range(2))
    v = torch.randn(B, T, H, Wv, generator=g, dtype=torch.float64).cuda().requires_grad_()
    dvo = torch.randn(B, T, H, Wv, generator=g, dtype=torch.float64).cuda()
    vo = sp.L1AttnSparseFn.apply(v, q, k, coo.cuda(), dmx, True)
    got = torch.autograd.grad(vo, (v, q, k), dvo)
    v2, q2, k2 = (x.detach().clone().requires_grad_() for x in (v, q, k))
    ref_vo = cf.sparse_value(v2, q2, k2, coo.cuda(), True)
    ref = torch.autograd.grad(ref_vo, (v2, q2, k2), dvo)
    _check((vo.detach(),) + got, (ref_vo.detach(),) + ref, [F64_TOL] * 4)


def test_sparse_gradcheck_fp64():
    # check_sparse.py:177-281: gradcheck of the autograd Functions in float64
    print("case sparse gradcheck", flush=True)
    from torch.autograd import gradcheck
    sp, bi = _m()
    g = torch.Generator().manual_seed(41)
    B, T, H, W = 2, 3, 4, 7
    kw = dict(dtype=torch.float64, generator=g)
    v, vb, q, k = (torch.randn(B, T, H, W, **kw).cuda().requires_grad_() for _ in range(4))
    for co in _edge_lists_check_sparse(T, g):
        coo, dmx, _ = sp.expandCoo(co.cuda(), warn=False)
        for sm in (True, False):
            assert gradcheck(sp.L1AttnSparseFn.apply, (v, q, k, coo, dmx, sm), nondet_tol=0.0)
            assert gradcheck(bi.L1AttnSparseBidiFn.apply, (v, vb, q, k, coo, dmx, sm), nondet_tol=0.0)


def test_dense_gradcheck_fp64():
    # check.py:100-107
    from torch.autograd import gradcheck
    import l1attn_cuda
    g = torch.Generator().manual_seed(43)
    q, k = (torch.randn(1, 5, 2, 6, dtype=torch.float64, generator=g).cuda().requires_grad_() for _ in range(2))
    assert gradcheck(l1attn_cuda.L1AttnFn.apply, (q, k), nondet_tol=0.0)


@pytest.mark.parametrize("which", ["config4", "config5"])
def test_sparse_benchmark_geometry_vs_closed_form(which):
    """Benchmark graph families at reduced token count against the fp64 closed form on the GPU
    (index_add_ formulation); the loop oracle with its padded [B,T,mx,H] tensor is too slow here."""
    print("case sparse benchmark geometry", which, flush=True)
    sp, bi = _m()
    if which == "config4":
        B, T, H, W = 2, 1024, 8, 32
        co = workloads.uniform_degree_graph(T, 64, seed=1004)
    else:
        B, T, H, W = 1, 8192, 4, 64
        co = workloads.powerlaw_graph(T, seed=1005)
    coo, dmx, smx = sp.expandCoo(co.cuda(), warn=False)
    g = torch.Generator().manual_seed(5)
    vf, vb, q, k, dvo = (torch.randn(B, T, H, W, generator=g).cuda() for _ in range(5))
    a, b, qd, kd = (x.clone().requires_grad_() for x in (vf, vb, q, k))
    if which == "config4":
        vo = sp.L1AttnSparse()(a, qd, kd, coo, dmx)
        got = (vo.detach(),) + torch.autograd.grad(vo, (a, qd, kd), dvo)
        a2, q2, k2 = (x.double().requires_grad_() for x in (vf, q, k))
        rvo = cf.sparse_value(a2, q2, k2, coo, True)
        ref = (rvo.detach(),) + torch.autograd.grad(rvo, (a2, q2, k2), dvo.double())
    else:
        vo = bi.L1AttnSparseBidi()(a, b, qd, kd, coo, dmx)
        got = (vo.detach(),) + torch.autograd.grad(vo, (a, b, qd, kd), dvo)
        a2, b2, q2, k2 = (x.double().requires_grad_() for x in (vf, vb, q, k))
        rvo = cf.bidi_value(a2, b2, q2, k2, coo, True)
        ref = (rvo.detach(),) + torch.autograd.grad(rvo, (a2, b2, q2, k2), dvo.double())
    _check([x.cpu() for x in got], [x.cpu() for x in ref], [FWD_TOL] + [BWD_TOL] * (len(got) - 1))


def test_sparse_input_checks():
    sp, _ = _m()
    import _l1attn_hip as drv
    x = torch.randn(1, 4, 2, 8).cuda()
    coo = torch.tensor([[0, 1, 0, 0], [5, 0, 0, 0]], dtype=torch.int32).cuda()
    with pytest.raises(RuntimeError, match="outside"):
        sp.L1AttnSparse()(x, x, x, coo, 1)
    with pytest.raises(RuntimeError, match="must be a CUDA tensor"):
        drv.sparse_forward(x.cpu(), x, x, coo, 1, True)
    # empty edge list: all-zero output, zero gradients
    coo0 = torch.zeros(0, 4, dtype=torch.int32).cuda()
    xr = x.clone().requires_grad_()
    vo = sp.L1AttnSparse()(xr, xr, xr, coo0, 1)
    assert torch.count_nonzero(vo) == 0
    vo.sum().backward()
    assert torch.count_nonzero(xr.grad) == 0
