"""GPU parity of the fused operator (L1 logits, softmax over src with the no-op logit, value sum in one
kernel; backward through one [B,T,T,H] tensor) through l1attn_cuda.L1AttnFused and so through
l1attn_fused_fwd_{f32,f64} and l1attn_fused_bwd_stage_{f32,f64}, of the experimental fixed-point dense
forward, and of the instruction-rate probe.

This file has not run on a GPU yet, which is why its name keeps it out of pytest's collection
(run it as `python -m pytest tests/wip_fused_gpu.py -m gpu`); rename it to test_*.py once it has
passed there.

Yardsticks: the CPU oracle (oracle.fused_fwd: the reference's dense CPU loop, then the no-op row,
softmax and einsum of example-setfind/setfind.py:128-136) at small sizes; at sizes the oracle's
[B,T,T,H] tensor would be slow for, the same composition in fp64 on the device from the dense HIP
operator (itself checked against the oracle elsewhere).  Tolerances: fp32 max|x-ref|/max|ref| <= 1e-5
against fp64 on the same fp32-valued inputs; fp64 entry point <= 1e-12.
"""
import pytest
import torch

import closed_forms as cf
import workloads
from oracle import oracle

pytestmark = pytest.mark.gpu


@pytest.fixture(autouse=True, scope="module")
def _opt_in():
    """These paths stay closed to the public operators until this file has passed on a GPU."""
    import _l1attn_hip as drv
    drv.enable_experimental("fused", "fixed")

F32_TOL, F64_TOL = 1e-5, 1e-12


def _fused():
    import l1attn_cuda
    return l1attn_cuda


SHAPES = [
    # B, T, H, W, Wv
    (2, 64, 4, 32, 32),     # first baseline configuration: tiled kernel, width 32
    (1, 100, 3, 64, 64),    # tiled kernel, ragged last dst tile, fewer heads than a workgroup holds
    (2, 70, 6, 16, 16),     # tiled kernel, width 16, ragged head group (6 = 4 + 2)
    (1, 33, 9, 64, 64),     # three head groups, the last with one head
    (2, 3, 16, 7, 7),       # generic kernel (check_sparse.py:18-21 shape)
    (1, 40, 2, 48, 48),     # tiled kernel, width 48
    (1, 36, 5, 96, 96),     # tiled kernel, width 96 (249-255 VGPRs)
    (1, 40, 2, 80, 80),     # generic kernel: width not among the tiled ones
    (1, 37, 3, 32, 20),     # generic kernel: value width differs
    (1, 31, 2, 64, 64),     # generic kernel: fewer than 32 tokens
]


@pytest.mark.parametrize("shape", SHAPES)
def test_fused_forward_vs_oracle(shape):
    B, T, H, W, Wv = shape
    print("case fused", shape, flush=True)
    import _l1attn_hip as drv
    g = torch.Generator().manual_seed(sum(shape))
    q, k = (torch.randn(B, T, H, W, generator=g) for _ in range(2))
    v = torch.randn(B, T, H, Wv, generator=g)
    if W == Wv:
        ref, ref_lse = oracle.fused_fwd(q.double(), k.double(), v.double())
    else:
        ref = cf.dense_then_value(q.double(), k.double(), v.double(), noop=True)
        ref_lse = (1.0 + cf.dense_attn(q.double(), k.double()).exp().sum(1)).log()
    vo, lse = drv.dense_fused_forward(q.cuda(), k.cuda(), v.cuda(), want_lse=True)
    torch.cuda.synchronize()
    assert cf.rel_err(vo.cpu(), ref) <= F32_TOL
    assert cf.rel_err(lse.cpu(), ref_lse) <= F32_TOL
    vo2 = _fused().L1AttnFused()(q.cuda(), k.cuda(), v.cuda())
    assert torch.equal(vo2, vo)  # module == driver, and bitwise run-to-run
    vo64, lse64 = drv.dense_fused_forward(q.double().cuda(), k.double().cuda(), v.double().cuda(), want_lse=True)
    assert cf.rel_err(vo64.cpu(), ref) <= F64_TOL
    assert cf.rel_err(lse64.cpu(), ref_lse) <= F64_TOL


@pytest.mark.parametrize("shape", [(2, 64, 4, 32), (1, 100, 3, 64), (2, 70, 6, 32), (1, 33, 9, 64), (2, 1024, 8, 64),
                                   (1, 40, 2, 48)])
def test_fused_pipelined_forward_equals_the_plain_one(shape):
    """l1attn_fused_fwd_pipe_f32 (k and v rows through the scalar-load pipeline; widths 32 and 64, any other width
    runs the plain kernels): the same arithmetic in the same order, so equal to l1attn_fused_fwd_f32 bit for bit,
    and within tolerance of the oracle.  Run after the plain forward's tests have passed."""
    B, T, H, W = shape
    print("case fused pipelined", shape, flush=True)
    import _l1attn_hip as drv
    g = torch.Generator().manual_seed(sum(shape))
    q, k, v = (torch.randn(B, T, H, W, generator=g).cuda() for _ in range(3))
    vo, lse = drv.dense_fused_forward(q, k, v, want_lse=True)
    vop, lsep = drv.dense_fused_forward(q, k, v, want_lse=True, pipelined=True)
    torch.cuda.synchronize()
    assert torch.equal(vop, vo) and torch.equal(lsep, lse)
    if T <= 128:
        ref, ref_lse = oracle.fused_fwd(q.cpu().double(), k.cpu().double(), v.cpu().double())
        assert cf.rel_err(vop.cpu(), ref) <= F32_TOL and cf.rel_err(lsep.cpu(), ref_lse) <= F32_TOL


@pytest.mark.parametrize("shape", [(2, 64, 4, 32), (1, 100, 3, 64), (2, 70, 9, 32), (1, 33, 9, 64), (2, 512, 8, 64)])
def test_fused_pipelined_backward_stage_equals_the_plain_one(shape):
    """l1attn_fused_bwd_stage_pipe_f32 (the dA and dv kernels with their wave-uniform rows through the scalar-load
    pipeline; widths 32 and 64): the same arithmetic in the same order, so dq, dk and dv of the whole backward
    equal the plain route's bit for bit.  Run after the plain backward's tests have passed."""
    B, T, H, W = shape
    print("case fused pipelined backward", shape, flush=True)
    import _l1attn_hip as drv
    g = torch.Generator().manual_seed(sum(shape) + 3)
    q, k, v, dvo = (torch.randn(B, T, H, W, generator=g).cuda() for _ in range(4))
    vo, lse = drv.dense_fused_forward(q, k, v, want_lse=True)
    plain = drv.dense_fused_backward(dvo, q, k, v, vo, lse)
    piped = drv.dense_fused_backward(dvo, q, k, v, vo, lse, pipelined=True)
    torch.cuda.synchronize()
    assert all(torch.equal(a, b) for a, b in zip(piped, plain))
    x = [t.clone().requires_grad_() for t in (q, k, v)]
    via_module = torch.autograd.grad(_fused().L1AttnFused(pipelined=True)(*x), x, dvo)
    assert all(torch.equal(a, b) for a, b in zip(via_module, plain))


def test_fused_forward_unaligned_views_take_the_generic_kernel():
    print("case fused unaligned", flush=True)
    import _l1attn_hip as drv
    g = torch.Generator().manual_seed(3)
    B, T, H, W = 1, 64, 2, 32
    flat = torch.randn(3, B * T * H * W + 1, generator=g).cuda()
    q, k, v = (flat[i, 1:].view(B, T, H, W) for i in range(3))  # 4-byte aligned only
    assert q.data_ptr() % 16 != 0 and q.is_contiguous()
    vo, _ = drv.dense_fused_forward(q, k, v)
    ref, _ = oracle.fused_fwd(q.cpu().double(), k.cpu().double(), v.cpu().double())
    assert cf.rel_err(vo.cpu(), ref) <= F32_TOL


@pytest.mark.parametrize("layernorm", [False, True])
def test_fused_forward_second_baseline_shape_vs_dense_operator(layernorm):
    """B16 T1024 H8 W64 (second baseline configuration, with its downstream softmax and einsum) at B=2:
    the fused kernel against the same composition in fp64 built on the dense HIP operator's fp64 entry."""
    print("case fused config 2", layernorm, flush=True)
    fz = _fused()
    B, T, H, W = 2, 1024, 8, 64
    q, k, v = workloads.dense_inputs(B, T, H, W, seed=1002, layernorm=layernorm, with_v=True)
    q, k, v = q.cuda(), k.cuda(), v.cuda()
    vo = fz.L1AttnFused()(q, k, v)
    a = fz.L1Attn()(q.double(), k.double())
    a = torch.cat((a, torch.zeros(B, 1, T, H, dtype=a.dtype, device=a.device)), 1)
    ref = torch.einsum("bsdh,bshw->bdhw", torch.softmax(a, 1)[:, :T], v.double())
    assert cf.rel_err(vo.cpu(), ref.cpu()) <= F32_TOL
    # equals sparse attention over the full cartesian list (python/l1attn_sparse.py:488-506)
    import l1attn_sparse_cuda as sp
    Ts = 96
    co = torch.cartesian_prod(torch.arange(Ts), torch.arange(Ts)).cuda()
    coo, dmx, _ = sp.expandCoo(co, warn=False)
    qs, ks, vs = (x[:, :Ts].contiguous() for x in (q, k, v))
    assert cf.rel_err(fz.L1AttnFused()(qs, ks, vs).cpu(), sp.L1AttnSparse()(vs, qs, ks, coo, dmx).cpu().double()) <= 2e-5


def test_fused_input_checks():
    print("case fused checks", flush=True)
    import _l1attn_hip as drv
    x = torch.randn(1, 32, 2, 16).cuda()
    with pytest.raises(RuntimeError, match="must be a CUDA tensor"):
        drv.dense_fused_forward(x.cpu(), x, x)
    with pytest.raises(RuntimeError, match="only float32 and float64"):
        drv.dense_fused_forward(x.half(), x.half(), x.half())


BWD_SHAPES = [
    # B, T, H, W, Wv
    (2, 64, 4, 32, 32),     # tiled kernels
    (1, 100, 3, 64, 64),    # tiled, ragged tile, 164 and 167 VGPR instantiations
    (2, 70, 6, 16, 16),     # tiled, ragged head group
    (1, 40, 2, 48, 48), (1, 36, 5, 96, 96),  # the other two tiled widths
    (2, 9, 3, 5, 5),        # generic kernels
    (1, 37, 3, 32, 20),     # generic kernels, value width differs
]


@pytest.mark.parametrize("shape", BWD_SHAPES)
def test_fused_backward_vs_oracle(shape):
    """dq, dk, dv of L1AttnFused against the oracle (oracle.fused_bwd; torch autograd through the fp64 closed form
    where the value width differs) on the same inputs:
    fp32 <= 1e-4 of the largest gradient, fp64 <= 1e-11; bitwise run-to-run."""
    B, T, H, W, Wv = shape
    print("case fused backward", shape, flush=True)
    fz = _fused()
    g = torch.Generator().manual_seed(sum(shape) + 1)
    q, k = (torch.randn(B, T, H, W, generator=g) for _ in range(2))
    v, dvo = (torch.randn(B, T, H, Wv, generator=g) for _ in range(2))
    if W == Wv:  # the oracle follows the reference's CPU loops, which have one width
        ref = oracle.fused_bwd(dvo.double(), q.double(), k.double(), v.double())
    else:
        r = [x.double().requires_grad_() for x in (q, k, v)]
        ref = torch.autograd.grad(cf.dense_then_value(*r, noop=True), r, dvo.double())
    for dt, tol in ((torch.float32, 1e-4), (torch.float64, 1e-11)):
        x = [t.to(dt).cuda().requires_grad_() for t in (q, k, v)]
        got = torch.autograd.grad(fz.L1AttnFused()(*x), x, dvo.to(dt).cuda())
        for a, b in zip(got, ref):
            assert cf.rel_err(a.cpu(), b) <= tol
        again = torch.autograd.grad(fz.L1AttnFused()(*x), x, dvo.to(dt).cuda())
        assert all(torch.equal(a, b) for a, b in zip(got, again))


def test_fused_gradcheck_fp64():
    print("case fused gradcheck", flush=True)
    from torch.autograd import gradcheck
    fz = _fused()
    g = torch.Generator().manual_seed(44)
    q, k, v = (torch.randn(1, 5, 2, 6, dtype=torch.float64, generator=g).cuda().requires_grad_() for _ in range(3))
    assert gradcheck(fz.L1AttnFusedFn.apply, (q, k, v), nondet_tol=0.0)


def test_fused_backward_second_baseline_shape_vs_composition():
    """B2 T1024 H8 W64: gradients of the fused operator against the unfused composition (L1Attn, zero logit row,
    softmax, einsum) differentiated by autograd through the dense HIP backward, both fp32: two routes to the
    same numbers, each within 1e-4 of fp64, so within 2e-4 of each other."""
    print("case fused backward config 2", flush=True)
    fz = _fused()
    B, T, H, W = 2, 1024, 8, 64
    q, k, v = (x.cuda() for x in workloads.dense_inputs(B, T, H, W, seed=1002, with_v=True))
    dvo = torch.randn(B, T, H, W, generator=torch.Generator().manual_seed(8)).cuda()
    x = [t.clone().requires_grad_() for t in (q, k, v)]
    got = torch.autograd.grad(fz.L1AttnFused()(*x), x, dvo)
    y = [t.clone().requires_grad_() for t in (q, k, v)]
    a = fz.L1Attn()(y[0], y[1])
    a = torch.cat((a, torch.zeros(B, 1, T, H, device=a.device)), 1)
    ref = torch.autograd.grad(torch.einsum("bsdh,bshw->bdhw", torch.softmax(a, 1)[:, :T], y[2]), y, dvo)
    for g_, r_ in zip(got, ref):
        assert cf.rel_err(g_.cpu(), r_.cpu().double()) <= 2e-4


def test_fused_backward_in_batch_slabs_equals_the_whole_batch():
    """The backward with a workspace bound that fits two of five batch entries (slabs of 2, 2, 1 through one
    shared buffer) against the same call with room for all five: a batch entry's gradients do not depend on which
    entries run beside it, so dv bitwise and dq, dk to 1e-6 of the largest gradient (their sums may be grouped
    by launch geometry)."""
    print("case fused backward slabs", flush=True)
    import _l1attn_hip as drv
    fz = _fused()
    B, T, H, W = 5, 96, 4, 32
    g = torch.Generator().manual_seed(77)
    q, k, v, dvo = (torch.randn(B, T, H, W, generator=g).cuda() for _ in range(4))
    vo, lse = drv.dense_fused_forward(q, k, v, want_lse=True)
    whole = drv.dense_fused_backward(dvo, q, k, v, vo, lse)
    old = drv.set_fused_workspace_bytes(2 * T * T * H * 4)
    try:
        assert drv.fused_backward_slab(B, T, H, 4) == 2
        slabs = drv.dense_fused_backward(dvo, q, k, v, vo, lse)
    finally:
        drv.set_fused_workspace_bytes(old)
    assert torch.equal(slabs[2], whole[2])
    for a, b in zip(slabs[:2], whole[:2]):
        assert cf.rel_err(a.cpu(), b.cpu().double()) <= 1e-6


def test_probe_other_instructions_runs():
    """The instruction-rate probe launches for every op code and rejects an unknown one."""
    print("case probe ops", flush=True)
    import _l1attn_hip as drv
    L = drv.lib()
    out = torch.zeros(4 * 512, device="cuda")
    for op in range(4):
        assert L.l1attn_probe_valu_op(drv.ptr(out), 4, 3, op, drv.stream_of(out)) == 0
    torch.cuda.synchronize()
    assert L.l1attn_probe_valu_op(drv.ptr(out), 4, 3, 4, drv.stream_of(out)) == -1


@pytest.mark.parametrize("shape,layernorm", [((2, 64, 4, 32), False), ((1, 100, 3, 64), False), ((2, 200, 16, 64), True),
                                              ((1, 1100, 5, 32), False)])
def test_fixed_point_forward_vs_oracle(shape, layernorm):
    """Experimental fixed-point forward (one v_sad_u32 per pair-element) against the fp64 oracle, same
    tolerance as the fp32 forward (1e-5 of the largest logit), beside the fp32 kernel's own error; exact
    zeros on the diagonal when k == q; a head of zeros; bitwise repeatability."""
    B, T, H, W = shape
    print("case fixed-point forward", shape, layernorm, flush=True)
    import _l1attn_hip as drv
    q, k, _ = workloads.dense_inputs(B, T, H, W, seed=sum(shape), layernorm=layernorm)
    q[:, :, 0, :] *= 37.0   # heads of different magnitude get different grids
    ref = oracle.dense_fwd(q.double(), k.double())
    a, = drv.dense_forward_fixed(q.cuda(), k.cuda())
    a32, = drv.dense_forward(q.cuda(), k.cuda())
    torch.cuda.synchronize()
    e_fix, e_f32 = cf.rel_err(a.cpu(), ref), cf.rel_err(a32.cpu(), ref)
    print("fixed", e_fix, "fp32", e_f32, flush=True)
    assert e_fix <= F32_TOL
    a2, = drv.dense_forward_fixed(q.cuda(), k.cuda())
    assert torch.equal(a, a2)
    d, = drv.dense_forward_fixed(q.cuda(), q.cuda())
    assert torch.count_nonzero(torch.diagonal(d, dim1=1, dim2=2)) == 0
    qz = q.clone()
    qz[:, :, H - 1, :] = 0
    z, = drv.dense_forward_fixed(qz.cuda(), qz.cuda())
    assert torch.count_nonzero(z[..., H - 1]) == 0 and torch.isfinite(z).all()
    with pytest.raises(RuntimeError, match="invalid argument"):
        drv.dense_forward_fixed(torch.zeros(1, 64, 2, 48).cuda(), torch.zeros(1, 64, 2, 48).cuda())


@pytest.mark.parametrize("ntok", [21, 45])
def test_fused_in_a_model_block(ntok):
    """The reference's transformer block (example-setfind/setfind.py:98-138: q from a linear layer, k a gated
    broadcast view of x, zero-token padding to a multiple of 16, one logit row overwritten with the no-op 0,
    softmax over src, contraction with v, sum over heads) with the fused operator in place of its five steps
    from the padding to the einsum: no padding is needed, the no-op is part of the operator.  Yardstick: the
    reference's graph in fp64 with the closed form for the logits; gradients back to x and the weights.
    21 tokens take the generic kernels, 45 the tiled ones."""
    print("case fused model block", ntok, flush=True)
    import math
    fz = _fused()
    batch, d_model, n_head = 3, 32, 4

    def qkv(x, wq, wv, wk):
        q = (x @ wq).reshape(batch, ntok, n_head, d_model)
        v = (x @ wv).reshape(batch, ntok, n_head, d_model)
        k = x.unsqueeze(2).expand(-1, -1, n_head, -1) * wk.unsqueeze(0).unsqueeze(0)
        return q, k, v

    def block_ref(x, wq, wv, wk):
        q, k, v = qkv(x, wq, wv, wk)
        padn = ((ntok + 15) // 16) * 16 - ntok
        zeros = torch.zeros(batch, padn, n_head, d_model, dtype=x.dtype, device=x.device)
        a = cf.dense_attn(torch.cat((q, zeros), 1), torch.cat((k, zeros), 1))
        a = a[:, :ntok + 1, :ntok, :].clone()
        a[:, ntok, :, :] = 0.0
        a = torch.softmax(a, 1)[:, :ntok]
        return torch.einsum("bsdh,bshw->bdhw", a, v).sum(2)

    def block_fused(x, wq, wv, wk):
        q, k, v = qkv(x, wq, wv, wk)
        return fz.L1AttnFused()(q, k, v).sum(2)

    def leaves(dtype):
        g = torch.Generator().manual_seed(99)
        x = torch.randn(batch, ntok, d_model, generator=g)
        wq = torch.randn(d_model, n_head * d_model, generator=g) / math.sqrt(d_model)
        wv = torch.randn(d_model, n_head * d_model, generator=g) / math.sqrt(d_model)
        wk = torch.randn(n_head, d_model, generator=g)
        return [t.to(dtype).cuda().requires_grad_() for t in (x, wq, wv, wk)]

    got, ref = leaves(torch.float32), leaves(torch.float64)
    out, out_ref = block_fused(*got), block_ref(*ref)
    gout = torch.randn(out.shape, generator=torch.Generator().manual_seed(5)).cuda()
    out.backward(gout)
    out_ref.backward(gout.double())
    assert cf.rel_err(out.detach().cpu(), out_ref.detach().cpu()) <= 1e-5
    for a, b in zip(got, ref):
        assert cf.rel_err(a.grad.cpu(), b.grad.cpu()) <= 1e-4
