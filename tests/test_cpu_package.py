"""The host-CPU operator package (l1attn_cpp, l1attn_sparse_cpp, l1attn_sparse_bidi_cpp over libl1attn_cpu.so),
the twin of the reference's cpp/ package (cpp/setup.py:4-16), checked on the CPU.

The package is product code with its own kernels (row-owner sweeps over dst- and src-sorted segments, OpenMP);
it does not call the oracle.  It is checked here AGAINST the oracle (the loop-for-loop restatement of
cpp/*.cpp), against the golden vectors written by the reference's own compiled extension, against that
extension live when oracle/_ref is built, and by the reference's own test programme (check.py:75-107,
check_sparse.py:36-171, python/l1attn_sparse.py:444-514): forward equality, fp64 gradcheck, the three
invariants (full list == dense with the no-op logit, row-permutation invariance, dropped edges).

Tolerances: float64 against float64 oracle / golden <= 1e-12 of max|ref|; float32 against the float64 oracle on
the same float32-valued inputs <= 1e-5 forward, 1e-4 gradients; expandCoo exact.
"""
import ctypes
import os
import re

import numpy as np
import pytest
import torch
from torch.autograd import gradcheck

import closed_forms as cf
from oracle import oracle

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
GOLD = os.path.join(os.path.dirname(__file__), "golden", "ref_cpp_golden.npz")
HEADER = os.path.join(ROOT, "include", "l1attn_cpu.h")
F64_TOL, F32_FWD, F32_GRAD = 1e-12, 1e-5, 1e-4


def _mods():
    import l1attn_cpp
    import l1attn_sparse_cpp
    import l1attn_sparse_bidi_cpp
    return l1attn_cpp, l1attn_sparse_cpp, l1attn_sparse_bidi_cpp


def _gold():
    return {k: torch.from_numpy(v) for k, v in np.load(GOLD).items()}


def _graph(g, T, E):
    return torch.stack((torch.randint(0, T, (E,), generator=g), torch.randint(0, T, (E,), generator=g)), 1)


# ------------------------------------------------------------------------------------------ boundary

def test_cpu_library_exports_every_declared_symbol_and_header_is_c():
    import subprocess
    import tempfile
    import _l1attn_cpu
    src = re.sub(r"/\*.*?\*/", "", open(HEADER).read(), flags=re.S)
    names = sorted(set(re.findall(r"\b(l1attn_cpu_[a-z0-9_]+)\s*\(", src)))
    assert len(names) == 19
    L = ctypes.CDLL(_l1attn_cpu._LIB_PATH)
    for n in names:
        assert hasattr(L, n), n
    with tempfile.TemporaryDirectory() as d:
        c = os.path.join(d, "t.c")
        open(c, "w").write('#include "l1attn_cpu.h"\nint main(void){return L1ATTN_CPU_OK;}\n')
        subprocess.run(["gcc", "-std=c99", "-Wall", "-Werror", "-I", os.path.join(ROOT, "include"), "-c", c,
                        "-o", os.path.join(d, "t.o")], check=True)


def test_cpu_package_is_separate_from_the_gpu_path():
    """Neither direction of import exists: the GPU operators cannot fall back to the CPU library, and the CPU
    package refuses GPU-side use by construction (device check) and never touches the oracle."""
    pkg = os.path.join(ROOT, "l1-attention_amd")
    gpu_side = ["_l1attn_hip.py", "l1attn_cuda.py", "l1attn_sparse_cuda.py", "l1attn_sparse_bidi_cuda.py",
                "l1attn_cuda_drv.py", "l1attn_sparse_cuda_drv.py", "l1attn_sparse_bidi_cuda_drv.py"]
    cpu_side = ["_l1attn_cpu.py", "l1attn_cpp.py", "l1attn_sparse_cpp.py", "l1attn_sparse_bidi_cpp.py",
                "l1attn_drv_cpp.py", "l1attn_sparse_drv.py", "l1attn_sparse_bidi_drv.py"]
    for f in gpu_side:
        text = open(os.path.join(pkg, f)).read()
        assert "_l1attn_cpu" not in text and "_cpp" not in text.replace("l1attn_drv_cpp", ""), f
        assert "oracle" not in text, f
    for f in cpu_side:
        text = open(os.path.join(pkg, f)).read()
        assert "_l1attn_hip" not in text and "oracle" not in text, f
    for f in os.listdir(os.path.join(pkg, "csrc_cpu")):
        assert "oracle" not in open(os.path.join(pkg, "csrc_cpu", f)).read(), f


def test_cpu_binding_argument_errors():
    import _l1attn_cpu as drv
    l1, sp, bi = _mods()
    q = torch.randn(1, 4, 2, 8)
    with pytest.raises(RuntimeError, match="one shape"):
        drv.dense_forward(q, q[:, :3].contiguous())
    with pytest.raises(RuntimeError, match="q must be contiguous"):
        drv.dense_forward(q.transpose(1, 2), q.transpose(1, 2))
    with pytest.raises(RuntimeError, match="only float32 and float64"):
        drv.dense_forward(q.half(), q.half())
    with pytest.raises(RuntimeError, match="d_attn must be"):
        drv.dense_backward(torch.randn(1, 4, 4, 3), q, q)
    coo = torch.tensor([[0, 1, 0, 0], [3, 9, 0, 0]], dtype=torch.int32)
    with pytest.raises(RuntimeError, match="outside"):
        drv.sparse_forward(q, q, q, coo, 1, True)               # src 9 of 4 tokens
    coo = torch.tensor([[0, 1, 0, 0], [0, 2, 1, 0]], dtype=torch.int32)
    with pytest.raises(RuntimeError, match="outside"):
        drv.sparse_forward(q, q, q, coo, 1, True)               # slot 1 with dst_mxlen 1
    with pytest.raises(RuntimeError, match="int32"):
        drv.sparse_forward(q, q, q, coo.long(), 2, True)
    vo, attn = drv.sparse_forward(q, q, q, coo, 2, True)
    with pytest.raises(RuntimeError, match="attn must be"):
        drv.sparse_backward(vo, q, q, q, coo, attn[:, :, :1].contiguous(), 2, True)
    with pytest.raises(RuntimeError, match="co must hold integers"):
        drv.expand_coo(torch.zeros(3, 2))
    if torch.cuda.is_available():
        with pytest.raises(RuntimeError, match="must be a CPU tensor"):
            drv.dense_forward(q.cuda(), q.cuda())


# --------------------------------------------------------------------------------------------- dense

@pytest.mark.parametrize("tag", ["dA", "dB"])
def test_dense_matches_the_reference_extension_golden(tag):
    l1, _, _ = _mods()
    G = _gold()
    q, k, da = (G[f"{tag}_{n}"].clone().requires_grad_(n != "da") for n in ("q", "k", "da"))
    a = l1.L1AttnFn.apply(q, k)
    a.backward(da)
    assert cf.rel_err(a.detach(), G[f"{tag}_attn"]) <= F64_TOL
    assert cf.rel_err(q.grad, G[f"{tag}_dq"]) <= F64_TOL and cf.rel_err(k.grad, G[f"{tag}_dk"]) <= F64_TOL
    # the planted ties (k[0,1] = q[0,2]) contribute exactly nothing: sign(0) = 0
    import l1attn_drv_cpp
    dq, dk = l1attn_drv_cpp.backward(G[f"{tag}_da"], G[f"{tag}_q"], G[f"{tag}_k"])
    assert torch.equal(dq, q.grad) and torch.equal(dk, k.grad)


@pytest.mark.parametrize("shape", [(2, 64, 4, 32), (2, 5, 3, 7), (1, 16, 8, 64), (3, 1, 1, 1), (1, 37, 5, 33),
                                   (1, 9, 20, 65), (2, 0, 3, 4), (0, 4, 3, 4)])
@pytest.mark.parametrize("dtype", [torch.float64, torch.float32])
def test_dense_matches_the_oracle(shape, dtype):
    l1, _, _ = _mods()
    B, T, H, W = shape
    g = torch.Generator().manual_seed(B * 1000 + T * 10 + W)
    q, k = (torch.randn(B, T, H, W, generator=g, dtype=dtype) for _ in range(2))
    if T > 2 and B > 0:
        k[0, 1] = q[0, 2]                                    # exact ties
        q[0, 0, 0, 0] = 0.0
        k[0, 0, 0, 0] = -0.0                                 # +0 and -0 tie too
    da = torch.randn(B, T, T, H, generator=g, dtype=dtype)
    qg, kg = q.clone().requires_grad_(), k.clone().requires_grad_()
    a = l1.L1Attn()(qg, kg)
    assert a.shape == (B, T, T, H) and a.dtype == dtype
    a.backward(da)
    if B * T == 0:
        assert qg.grad.shape == q.shape
        return
    ra = oracle.dense_fwd(q.double(), k.double())
    rdq, rdk = oracle.dense_bwd(da.double(), q.double(), k.double())
    ftol, gtol = (F64_TOL, F64_TOL) if dtype == torch.float64 else (F32_FWD, F32_GRAD)
    assert cf.rel_err(a.detach(), ra) <= ftol
    assert cf.rel_err(qg.grad, rdq) <= gtol and cf.rel_err(kg.grad, rdk) <= gtol
    # the checksum that holds whatever the data: every pair enters dq and dk with opposite signs
    assert abs(float(qg.grad.double().sum() + kg.grad.double().sum())) <= 1e-4 * float(rdq.abs().sum() + 1)


def test_dense_hand_answer_onehot():
    """testdense.py:20-35: one-hot tokens, W = 4, so scale = -0.5 and every logit is -0.5 * L1 distance."""
    l1, _, _ = _mods()
    q = torch.zeros(1, 4, 1, 4, dtype=torch.float64)
    k = torch.zeros(1, 4, 1, 4, dtype=torch.float64)
    q[0, 0, 0, 1] = q[0, 1, 0, 2] = q[0, 2, 0, 0] = 1.0
    k[0, 0, 0, 0] = k[0, 1, 0, 1] = k[0, 2, 0, 2] = 1.0
    a = l1.L1Attn()(q, k)[0, :, :, 0]                        # [s, t]
    expect = torch.tensor([[-1.0, -1.0, 0.0, -0.5], [0.0, -1.0, -1.0, -0.5], [-1.0, 0.0, -1.0, -0.5],
                           [-0.5, -0.5, -0.5, 0.0]], dtype=torch.float64)
    assert torch.equal(a, expect)


def test_dense_gradcheck_fp64():
    """check.py:100-107 (gradcheck of the Function in float64; ties avoided as the reference's comment asks)."""
    l1, _, _ = _mods()
    g = torch.Generator().manual_seed(7)
    q = torch.randn(1, 6, 2, 5, generator=g, dtype=torch.float64, requires_grad=True)
    k = torch.randn(1, 6, 2, 5, generator=g, dtype=torch.float64, requires_grad=True)
    assert gradcheck(l1.L1AttnFn.apply, (q, k), eps=1e-6, atol=1e-6, nondet_tol=0.0)


def test_results_do_not_depend_on_threads_or_instruction_set():
    """One owner per output row: the same bits with 1, 3 and all threads.  The baseline and the AVX2 copies of the
    kernels may differ in rounding (fused multiply-add) but both are within tolerance of the oracle."""
    import subprocess
    import sys
    import _l1attn_cpu as drv
    l1, sp, _ = _mods()
    g = torch.Generator().manual_seed(11)
    q, k, v = (torch.randn(2, 50, 3, 20, generator=g) for _ in range(3))
    da = torch.randn(2, 50, 50, 3, generator=g)
    coo, dmx, _ = sp.expandCoo(_graph(g, 50, 400), warn=False)
    outs = []
    for n in (1, 3, 0):
        old = drv.set_threads(n)
        a = drv.dense_forward(q, k)[0]
        dq, dk = drv.dense_backward(da, q, k)
        vo, attn = drv.sparse_forward(v, q, k, coo, dmx, True)
        grads = drv.sparse_backward(vo, v, q, k, coo, attn, dmx, True)
        outs.append([a, dq, dk, vo, attn] + grads)
        drv.set_threads(old)
    for other in outs[1:]:
        for x, y in zip(outs[0], other):
            assert torch.equal(x, y)
    code = ("import sys, torch; sys.path.insert(0, %r); import _l1attn_cpu as d; g = torch.Generator().manual_seed(11);"
            "q, k, v = (torch.randn(2, 50, 3, 20, generator=g) for _ in range(3));"
            "torch.save(d.dense_forward(q, k)[0], sys.argv[1])" % os.path.join(ROOT, "l1-attention_amd"))
    import tempfile
    with tempfile.TemporaryDirectory() as d:
        path = os.path.join(d, "a.pt")
        subprocess.run([sys.executable, "-c", code, path], check=True, env=dict(os.environ, L1ATTN_CPU_ISA="generic"))
        a_generic = torch.load(path, weights_only=True)
    ref = oracle.dense_fwd(q.double(), k.double())
    assert cf.rel_err(a_generic, ref) <= F32_FWD and cf.rel_err(outs[0][0], ref) <= F32_FWD


# ----------------------------------------------------------------------------------------- expandCoo

def test_expand_coo_known_answers_and_brute_force(capsys):
    _, sp, bi = _mods()
    co = torch.cartesian_prod(torch.arange(3), torch.arange(3))          # README.md:89
    coo, dmx, smx = sp.expandCoo(co)
    assert coo.dtype == torch.int32 and coo[:, 2].tolist() == [0, 1, 2] * 3 and coo[:, 3].tolist() == [0, 0, 0, 1, 1, 1, 2, 2, 2]
    assert (dmx, smx) == (3, 3) and capsys.readouterr().out == ""
    co = torch.tensor([[0, 0], [0, 1], [0, 2], [1, 0], [1, 1], [2, 0], [2, 1]])  # python/l1attn_sparse.py:576
    coo, dmx, smx = bi.expandCoo(co)
    assert coo[:, 2].tolist() == [0, 1, 2, 0, 1, 0, 1] and coo[:, 3].tolist() == [0, 0, 0, 1, 1, 2, 2] and (dmx, smx) == (3, 3)
    e, dmx, smx = sp.expandCoo(torch.zeros(0, 2, dtype=torch.int64))
    assert e.shape == (0, 4) and (dmx, smx) == (1, 1)
    g = torch.Generator().manual_seed(3)
    for dt in (torch.int64, torch.int32, torch.int16, torch.uint8):
        co = torch.randint(0, 40, (300, 2), generator=g).to(dt)
        coo, dmx, smx = sp.expandCoo(co, warn=False)
        bcoo, bdmx, bsmx = cf.expand_coo_bruteforce(co)
        assert torch.equal(coo, bcoo) and (dmx, smx) == (bdmx, bsmx)
    # the reference's dict takes any integer: negative and huge keys go through the hash-map path
    co = torch.tensor([[-5, 2_000_000_000], [7, 2_000_000_000], [-5, 3], [-5, 2_000_000_000]])
    coo, dmx, smx = sp.expandCoo(co, warn=False)
    assert coo.tolist() == [[-5, 2_000_000_000, 0, 0], [7, 2_000_000_000, 0, 1], [-5, 3, 1, 0], [-5, 2_000_000_000, 2, 2]]
    assert (dmx, smx) == (3, 3)
    with pytest.raises(RuntimeError, match="code -4"):
        sp.expandCoo(torch.tensor([[0, 2 ** 40]]), warn=False)
    # a larger list against the oracle's loop (python/l1attn_sparse.py:382-427 restated)
    co = torch.randint(0, 5000, (200_000, 2), generator=g)
    coo, dmx, smx = sp.expandCoo(co, warn=False)
    ocoo, odmx, osmx = oracle.expand_coo(co)
    assert torch.equal(coo, ocoo) and (dmx, smx) == (odmx, osmx)
    # warnings of this copy of the reference: unwritten dst and unread src below the largest (cpp/l1attn_sparse_cpp.py:97-102)
    sp.expandCoo(torch.tensor([[0, 0], [2, 3]]))
    out = capsys.readouterr().out.splitlines()
    assert out == ["Warning: degenerate sparse head - 1 not written", "Warning degenerate sparse head - 1 not read",
                   "Warning degenerate sparse head - 2 not read"]


# ------------------------------------------------------------------------------------ sparse and bidi

@pytest.mark.parametrize("tag", ["sA", "sB"])
@pytest.mark.parametrize("sm", [True, False])
def test_sparse_and_bidi_match_the_reference_extension_golden(tag, sm):
    _, sp, bi = _mods()
    G = _gold()
    s = "sm" if sm else "nsm"
    coo, (dmx, smx) = G[f"{tag}_coo"], G[f"{tag}_mx"].tolist()
    mine, mdmx, msmx = sp.expandCoo(G[f"{tag}_co"], warn=False)
    assert torch.equal(mine, coo) and (mdmx, msmx) == (dmx, smx)
    v, q, k, vb = (G[f"{tag}_{n}"].clone().requires_grad_() for n in ("v", "q", "k", "vb"))
    dvo = G[f"{tag}_dvo"]
    vo = sp.L1AttnSparseFn.apply(v, q, k, coo, dmx, sm)
    grads = torch.autograd.grad(vo, (v, q, k), dvo)
    assert cf.rel_err(vo.detach(), G[f"{tag}_{s}_vo"]) <= F64_TOL
    for x, n in zip(grads, ("dv", "dq", "dk")):
        assert cf.rel_err(x, G[f"{tag}_{s}_{n}"]) <= F64_TOL, n
    # the saved tensor is the reference's padded [B,T,dst_mxlen,H] edge-weight tensor, slot for slot
    import l1attn_sparse_drv
    _, attn = l1attn_sparse_drv.forward(v.detach(), q.detach(), k.detach(), coo, dmx, sm)
    assert attn.shape == G[f"{tag}_{s}_attn"].shape and cf.rel_err(attn, G[f"{tag}_{s}_attn"]) <= F64_TOL
    vo = bi.L1AttnSparseBidiFn.apply(v, vb, q, k, coo, dmx, sm)
    grads = torch.autograd.grad(vo, (v, vb, q, k), dvo)
    assert cf.rel_err(vo.detach(), G[f"{tag}_{s}_bidi_vo"]) <= F64_TOL
    for x, n in zip(grads, ("dvf", "dvb", "dq", "dk")):
        assert cf.rel_err(x, G[f"{tag}_{s}_bidi_{n}"]) <= F64_TOL, n


@pytest.mark.parametrize("sm", [True, False])
@pytest.mark.parametrize("dtype", [torch.float64, torch.float32])
@pytest.mark.parametrize("shape", [(2, 3, 16, 7, 7, 9), (1, 40, 3, 32, 32, 500), (2, 17, 2, 5, 9, 60), (1, 300, 4, 64, 16, 2500)])
def test_sparse_and_bidi_match_the_oracle(shape, dtype, sm):
    """Random multigraphs (repeated edges, edgeless tokens), Wv != W, long segments; values, the padded edge-weight
    tensor and every gradient against the oracle's loops."""
    _, sp, bi = _mods()
    B, T, H, W, Wv, E = shape
    g = torch.Generator().manual_seed(T * 100 + E)
    coo, dmx, smx = sp.expandCoo(_graph(g, T, E), warn=False)
    q, k = (torch.randn(B, T, H, W, generator=g, dtype=dtype) for _ in range(2))
    vf, vb, dvo = (torch.randn(B, T, H, Wv, generator=g, dtype=dtype) for _ in range(3))
    k[0, 1] = q[0, 2]
    ftol, gtol = (F64_TOL, F64_TOL) if dtype == torch.float64 else (F32_FWD, F32_GRAD)
    leaves = [x.clone().requires_grad_() for x in (vf, vb, q, k)]
    vo = sp.L1AttnSparse()(leaves[0], leaves[2], leaves[3], coo, dmx, sm)
    grads = torch.autograd.grad(vo, (leaves[0], leaves[2], leaves[3]), dvo)
    d = [x.double() for x in (vf, vb, q, k, dvo)]
    if Wv == W:
        rvo, rattn = oracle.sparse_fwd(d[0], d[2], d[3], coo, dmx, sm)
        rgrads = oracle.sparse_bwd(d[4], d[0], d[2], d[3], coo, rattn, dmx, sm, 1)
        import _l1attn_cpu as drv
        attn = drv.sparse_forward(vf, q, k, coo, dmx, sm)[1]
        assert cf.rel_err(attn, rattn) <= ftol
    else:  # the oracle's loops need Wv == W (as cpp/l1attn_sparse_drv.cpp:42): closed form + autograd instead
        dl = [x.clone().requires_grad_() for x in d[:4]]
        rvo = cf.sparse_value(dl[0], dl[2], dl[3], coo, sm)
        rgrads = torch.autograd.grad(rvo, (dl[0], dl[2], dl[3]), d[4])
        rvo = rvo.detach()
    assert cf.rel_err(vo.detach(), rvo) <= ftol
    for x, y in zip(grads, rgrads):
        assert cf.rel_err(x, y) <= gtol
    vo = bi.L1AttnSparseBidi()(*leaves, coo, dmx, sm)
    grads = torch.autograd.grad(vo, leaves, dvo)
    if Wv == W:
        rvo, rattn = oracle.bidi_fwd(d[0], d[1], d[2], d[3], coo, dmx, sm)
        rgrads = oracle.bidi_bwd(d[4], d[0], d[1], d[2], d[3], coo, rattn, dmx, sm, 1)
    else:
        dl = [x.clone().requires_grad_() for x in d[:4]]
        rvo = cf.bidi_value(*dl, coo, sm)
        rgrads = torch.autograd.grad(rvo, dl, d[4])
        rvo = rvo.detach()
    assert cf.rel_err(vo.detach(), rvo) <= ftol
    for x, y in zip(grads, rgrads):
        assert cf.rel_err(x, y) <= gtol


def test_the_reference_test_programme_for_the_sparse_operators():
    """check_sparse.py:98-171 at its shape (B=2, T=3, H=16, W=7, float64): for the full cartesian list, a row
    permutation of it, and the permutation minus four edges, both use_softmax settings: forward equals the
    closed form, gradcheck passes; permutation leaves the result unchanged; and with the full list the operator
    equals dense attention with the no-op logit (python/l1attn_sparse.py:488-506)."""
    l1, sp, bi = _mods()
    B, T, H, W = 2, 3, 16, 7
    g = torch.Generator().manual_seed(5)
    kw = dict(generator=g, dtype=torch.float64)
    v, vb, q, k = (torch.randn(B, T, H, W, **kw).requires_grad_() for _ in range(4))
    full = torch.cartesian_prod(torch.arange(T), torch.arange(T))
    perm = full[torch.randperm(full.shape[0], generator=g)]
    results = {}
    for name, co in (("full", full), ("perm", perm), ("dropped", perm[:-4])):
        coo, dmx, smx = sp.expandCoo(co, warn=False)
        for sm in (True, False):
            vo = sp.L1AttnSparseFn.apply(v, q, k, coo, dmx, sm)
            assert cf.rel_err(vo.detach(), cf.sparse_value(v, q, k, coo, sm).detach()) <= F64_TOL
            assert gradcheck(sp.L1AttnSparseFn.apply, (v, q, k, coo, dmx, sm), eps=1e-6, atol=1e-6, nondet_tol=0.0)
            vob = bi.L1AttnSparseBidiFn.apply(v, vb, q, k, coo, dmx, sm)
            assert cf.rel_err(vob.detach(), cf.bidi_value(v, vb, q, k, coo, sm).detach()) <= F64_TOL
            assert gradcheck(bi.L1AttnSparseBidiFn.apply, (v, vb, q, k, coo, dmx, sm), eps=1e-6, atol=1e-6,
                             nondet_tol=0.0)
            results[name, sm] = vo.detach()
    for sm in (True, False):
        assert cf.rel_err(results["perm", sm], results["full", sm]) <= F64_TOL
    a = l1.L1Attn()(q, k)
    a = torch.cat((a, torch.zeros(B, 1, T, H, dtype=torch.float64)), 1)
    dense = torch.einsum("bsdh,bshw->bdhw", torch.softmax(a, 1)[:, :T], v)
    assert cf.rel_err(results["full", True], dense.detach()) <= F64_TOL


def test_sparse_integer_fixture_hand_answer():
    """python/l1attn_sparse.py:450-484: integer tokens, W = 3.  Token 0 attends to k0 and k1 with L1 distances 4 and
    0: weights e^{-4/sqrt3} and 1 over the denominator 1 + both."""
    _, sp, _ = _mods()
    F64 = dict(dtype=torch.float64)
    q = torch.tensor([[0, 1, 2], [2, 1, 0], [0, 0, 0]], **F64).reshape(1, 3, 1, 3)
    k = torch.tensor([[2, 1, 0], [0, 1, 2], [0, 1, 2]], **F64).reshape(1, 3, 1, 3)
    v = torch.tensor([[-2, 2, 3], [2, -2, 2], [3, 2, -2]], **F64).reshape(1, 3, 1, 3)
    coo, dmx, _ = sp.expandCoo(torch.tensor([[0, 0], [0, 1]]), warn=False)
    vo = sp.L1AttnSparse()(v, q, k, coo, dmx)
    e = np.exp(-4 / np.sqrt(3))
    expect = (e * v[0, 0, 0] + 1.0 * v[0, 1, 0]) / (1 + e + 1.0)
    assert torch.allclose(vo[0, 0, 0], expect, rtol=0, atol=1e-15)
    assert torch.equal(vo[0, 1:], torch.zeros(2, 1, 3, **F64))           # tokens without an incoming edge


def test_live_reference_extension_when_built():
    """When oracle/_ref holds the reference's own compiled CPU extension (the build container), the package and
    that extension are run on the same fresh float64 inputs, all three modules, both softmax settings."""
    mods = oracle.ref_modules()
    if mods is None:
        pytest.skip("oracle/_ref is not built here")
    import l1attn_drv_cpp, l1attn_sparse_drv, l1attn_sparse_bidi_drv
    g = torch.Generator().manual_seed(99)
    kw = dict(generator=g, dtype=torch.float64)
    B, T, H, W = 2, 12, 3, 9
    q, k, v, vb, dvo = (torch.randn(B, T, H, W, **kw) for _ in range(5))
    da = torch.randn(B, T, T, H, **kw)
    assert cf.rel_err(l1attn_drv_cpp.forward(q, k)[0], mods["l1attn_drv_cpp"].forward(q, k)[0]) <= F64_TOL
    for x, y in zip(l1attn_drv_cpp.backward(da, q, k), mods["l1attn_drv_cpp"].backward(da, q, k)):
        assert cf.rel_err(x, y) <= F64_TOL
    _, sp, _ = _mods()
    coo, dmx, _ = sp.expandCoo(_graph(g, T, 70), warn=False)
    for sm in (True, False):
        mine, ref = l1attn_sparse_drv.forward(v, q, k, coo, dmx, sm), mods["l1attn_sparse_drv"].forward(v, q, k, coo, dmx, sm)
        for x, y in zip(mine, ref):
            assert cf.rel_err(x, y) <= F64_TOL
        for x, y in zip(l1attn_sparse_drv.backward(dvo, v, q, k, coo, mine[1], dmx, sm),
                        mods["l1attn_sparse_drv"].backward(dvo, v, q, k, coo, ref[1], dmx, sm)):
            assert cf.rel_err(x, y) <= F64_TOL
        mine = l1attn_sparse_bidi_drv.forward(v, vb, q, k, coo, dmx, sm)
        ref = mods["l1attn_sparse_bidi_drv"].forward(v, vb, q, k, coo, dmx, sm)
        for x, y in zip(mine, ref):
            assert cf.rel_err(x, y) <= F64_TOL
        for x, y in zip(l1attn_sparse_bidi_drv.backward(dvo, v, vb, q, k, coo, mine[1], dmx, sm),
                        mods["l1attn_sparse_bidi_drv"].backward(dvo, v, vb, q, k, coo, ref[1], dmx, sm)):
            assert cf.rel_err(x, y) <= F64_TOL


# ------------------------------------------------------------------------------------------- fused

@pytest.mark.parametrize("shape", [(2, 64, 4, 32, 32), (1, 100, 3, 64, 64), (2, 9, 3, 5, 5), (1, 37, 3, 32, 20),
                                   (1, 1, 1, 1, 1), (2, 0, 3, 4, 4)])
@pytest.mark.parametrize("dtype", [torch.float64, torch.float32])
def test_fused_operator_matches_the_oracle(shape, dtype):
    """l1attn_cpp.L1AttnFused against the oracle's composition (the reference's dense CPU loop, then the no-op row,
    softmax and einsum of example-setfind/setfind.py:128-136, differentiated by hand), against torch autograd through
    the closed form where the value width differs, and against the same composition built on l1attn_cpp.L1Attn."""
    l1, _, _ = _mods()
    B, T, H, W, Wv = shape
    g = torch.Generator().manual_seed(sum(shape))
    q, k = (torch.randn(B, T, H, W, generator=g, dtype=dtype) for _ in range(2))
    v, dvo = (torch.randn(B, T, H, Wv, generator=g, dtype=dtype) for _ in range(2))
    x = [t.clone().requires_grad_() for t in (q, k, v)]
    vo = l1.L1AttnFused()(*x)
    assert vo.shape == v.shape and vo.dtype == dtype
    got = torch.autograd.grad(vo, x, dvo)
    if T == 0:
        return
    ftol, gtol = (F64_TOL, 1e-11) if dtype == torch.float64 else (F32_FWD, F32_GRAD)
    if W == Wv:
        ref, ref_lse = oracle.fused_fwd(q.double(), k.double(), v.double())
        rg = oracle.fused_bwd(dvo.double(), q.double(), k.double(), v.double())
        import _l1attn_cpu as drv
        assert cf.rel_err(drv.fused_forward(q, k, v)[1], ref_lse) <= ftol
    else:
        r = [t.double().requires_grad_() for t in (q, k, v)]
        ref = cf.dense_then_value(*r, noop=True)
        rg = torch.autograd.grad(ref, r, dvo.double())
        ref = ref.detach()
    assert cf.rel_err(vo.detach(), ref) <= ftol
    for a, b in zip(got, rg):
        assert cf.rel_err(a, b) <= gtol
    # the same numbers from the unfused composition on the dense operator of this package
    y = [t.clone().requires_grad_() for t in (q, k, v)]
    a = l1.L1Attn()(y[0], y[1])
    a = torch.cat((a, torch.zeros(B, 1, T, H, dtype=dtype)), 1)
    comp = torch.einsum("bsdh,bshw->bdhw", torch.softmax(a, 1)[:, :T], y[2])
    cg = torch.autograd.grad(comp, y, dvo)
    assert cf.rel_err(vo.detach(), comp.detach().double()) <= 2 * ftol
    for a_, b_ in zip(got, cg):
        assert cf.rel_err(a_, b_.double()) <= 2 * gtol


def test_fused_operator_gradcheck_and_sparse_equivalence():
    l1, sp, _ = _mods()
    g = torch.Generator().manual_seed(44)
    q, k, v = (torch.randn(1, 5, 2, 6, dtype=torch.float64, generator=g).requires_grad_() for _ in range(3))
    assert gradcheck(l1.L1AttnFusedFn.apply, (q, k, v), eps=1e-6, atol=1e-6, nondet_tol=0.0)
    # equals sparse attention over the full cartesian edge list (python/l1attn_sparse.py:488-506)
    T = 5
    coo, dmx, _ = sp.expandCoo(torch.cartesian_prod(torch.arange(T), torch.arange(T)), warn=False)
    assert cf.rel_err(l1.L1AttnFused()(q, k, v).detach(), sp.L1AttnSparse()(v, q, k, coo, dmx).detach()) <= F64_TOL
