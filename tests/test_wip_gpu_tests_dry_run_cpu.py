"""CPU-only: the not-yet-collected GPU test files (tests/wip_*.py) walked without a GPU, so that a slip in a test's
own yardstick, shapes or tolerances shows now and not on the first GPU run.

The kernels under test are replaced by stand-ins with the same driver signatures: the CPU operator package for
the operators that exist there, torch closed forms for the fused operator, the numpy model of
tests/test_fixed_point_model_cpu.py for the fixed-point forward, and "compute in float32, round once" for 16-bit
rows (which is what those kernels are specified to do).  `.cuda()` is the identity here.  What this proves is the
TEST: that its reference side is right and its tolerances are reachable by a correct implementation.  It says
nothing about the HIP kernels."""
import importlib.util
import os
import sys

import numpy as np
import pytest
import torch

import closed_forms as cf

HERE = os.path.dirname(os.path.abspath(__file__))


def _load(name):
    spec = importlib.util.spec_from_file_location(name, os.path.join(HERE, name + ".py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


def _fixed_model(q, k):
    from test_fixed_point_model_cpu import _model
    B, T, H, W = q.shape
    if W not in (32, 64) or T < 32:
        raise RuntimeError("l1attn_dense_fwd_fixed_f32: invalid argument (code -1)")
    out = torch.empty(B, T, T, H)
    for b in range(B):
        for h in range(H):
            out[b, :, :, h] = torch.from_numpy(_model(q[b, :, h].numpy(), k[b, :, h].numpy()))
    return [out]


@pytest.fixture()
def cpu_stand_ins(monkeypatch):
    import _l1attn_cpu as cpu
    import _l1attn_hip as drv
    import l1attn_sparse_cpp
    monkeypatch.setattr(torch.Tensor, "cuda", lambda self, *a, **k: self)
    monkeypatch.setattr(torch.cuda, "synchronize", lambda *a, **k: None)
    monkeypatch.setattr(drv, "_enabled", set())
    monkeypatch.setattr(drv, "check_input", lambda x, name: None)
    monkeypatch.setattr(drv, "dense_forward", lambda q, k: cpu.dense_forward(q.contiguous(), k.contiguous()))
    monkeypatch.setattr(drv, "dense_backward", lambda d, q, k: cpu.dense_backward(d.contiguous(), q, k))
    monkeypatch.setattr(drv, "dense_forward_fixed", _fixed_model)
    monkeypatch.setattr(drv, "expand_coo", cpu.expand_coo)
    monkeypatch.setattr(drv, "plan_for", lambda coo, n_tok: None)

    def fused_fwd(q, k, v, want_lse=False, pipelined=False):
        if q.dtype not in (torch.float32, torch.float64):
            raise RuntimeError("q: only float32 and float64 are implemented, got %s" % q.dtype)
        e = cf.dense_attn(q, k).exp()
        esum = e.sum(1)
        return [torch.einsum("bsdh,bshw->bdhw", e / (1.0 + esum)[:, None], v), torch.log1p(esum) if want_lse else None]

    def fused_bwd(dvo, q, k, v, vo, lse, pipelined=False):
        with torch.enable_grad():  # (called from inside a Function's backward, where recording is off)
            leaves = [x.detach().clone().requires_grad_() for x in (q, k, v)]
            return list(torch.autograd.grad(cf.dense_then_value(*leaves, noop=True), leaves, dvo))

    monkeypatch.setattr(drv, "dense_fused_forward", fused_fwd)
    monkeypatch.setattr(drv, "dense_fused_backward", fused_bwd)

    # 16-bit rows: float32 arithmetic on the 16-bit values, one rounding on store
    def f32(*xs):
        return [x.float().contiguous() for x in xs]

    def sparse_fwd(v, q, k, coo, dmx, sm, plan=None):
        vo, attn = cpu.sparse_forward(*f32(v, q, k), coo, dmx, sm) if v.dtype != torch.float64 else \
            cpu.sparse_forward(v, q, k, coo, dmx, sm)
        return [vo.to(v.dtype), attn]

    def sparse_bwd(dvo, v, q, k, coo, attn, dmx, sm, plan=None):
        if v.dtype == torch.float64:
            return cpu.sparse_backward(dvo, v, q, k, coo, attn, dmx, sm)
        return [g.to(v.dtype) for g in cpu.sparse_backward(*f32(dvo, v, q, k), coo, attn, dmx, sm)]

    def bidi_fwd(vf, vb, q, k, coo, dmx, sm, plan=None):
        # the kernels round vo once after the dst pass and once after the src pass has added its sum
        vo_d, attn = cpu.sparse_forward(*f32(vf, q, k), coo, dmx, sm)
        vo, _ = cpu.bidi_forward(*f32(vf, vb, q, k), coo, dmx, sm)
        if vf.dtype in (torch.float16, torch.bfloat16):
            vo = (vo_d.to(vf.dtype).float() + (vo - vo_d)).to(vf.dtype)
        return [vo.to(vf.dtype), attn]

    def bidi_bwd(dvo, vf, vb, q, k, coo, attn, dmx, sm, plan=None):
        return [g.to(vf.dtype) for g in cpu.bidi_backward(*f32(dvo, vf, vb, q, k), coo, attn, dmx, sm)]

    for name, fn in (("sparse_forward", sparse_fwd), ("sparse_backward", sparse_bwd), ("bidi_forward", bidi_fwd),
                     ("bidi_backward", bidi_bwd)):
        monkeypatch.setattr(drv, name, fn)
    monkeypatch.setitem(sys.modules, "l1attn_sparse_cuda_for_dry_run", l1attn_sparse_cpp)
    return drv


def test_wip_fused_gpu_tests_walk_on_stand_ins(cpu_stand_ins):
    t = _load("wip_fused_gpu")
    cpu_stand_ins.enable_experimental("fused", "fixed")
    for shape in t.SHAPES:
        t.test_fused_forward_vs_oracle(shape)
    for shape in [(2, 64, 4, 32), (1, 100, 3, 64), (1, 40, 2, 48)]:
        t.test_fused_pipelined_forward_equals_the_plain_one(shape)
    for shape in [(2, 64, 4, 32), (1, 33, 9, 64)]:
        t.test_fused_pipelined_backward_stage_equals_the_plain_one(shape)
    t.test_fused_forward_unaligned_views_take_the_generic_kernel()
    for shape in t.BWD_SHAPES:
        t.test_fused_backward_vs_oracle(shape)
    t.test_fused_gradcheck_fp64()
    for ntok in (21, 45):
        t.test_fused_in_a_model_block(ntok)
    for shape, ln in [((2, 64, 4, 32), False), ((1, 100, 3, 64), False), ((2, 200, 16, 64), True)]:
        t.test_fixed_point_forward_vs_oracle(shape, ln)
    # (the two tests at the second baseline configuration's size walk the same way in about twenty seconds each;
    # they are left out of the CPU suite for its running time)


def test_wip_sparse_half_gpu_tests_walk_on_stand_ins(cpu_stand_ins):
    t = _load("wip_sparse_half_gpu")
    cpu_stand_ins.enable_experimental("rows16")
    for dt in t.DTYPES:
        for shape in t.SHAPES:
            for sm in (True, False):
                t.test_half_forward_vs_f32_entry_and_oracle(dt, shape, sm)
        t.test_half_forward_long_segments(dt)
        for shape in [(2, 9, 3, 5, 5, 40), (1, 64, 8, 32, 32, 900), (2, 50, 4, 64, 64, 700), (2, 20, 3, 8, 12, 90)]:
            for sm in (True, False):
                t.test_half_backward_vs_autograd_closed_form(dt, shape, sm)
        t.test_half_empty_list(dt)
        for which in ("config4", "config5"):
            t.test_half_forward_benchmark_geometry(dt, which)


def test_wip_backward_form_gpu_tests_walk_on_stand_ins(cpu_stand_ins, monkeypatch):
    """tests/wip_bwd_prefetch_gpu.py (its smallest shape) and the backward test of tests/wip_rank_sort_gpu.py: the
    plans they assert on come from the real library's host logic, the opt-in and the selection of the form run as
    they will on the GPU, the backward itself is the CPU package's (whatever the form: all forms are specified to
    give the same bits)."""
    drv = cpu_stand_ins
    monkeypatch.setattr(drv, "_dense_bwd_form", (0, 0))
    t = _load("wip_bwd_prefetch_gpu")
    monkeypatch.setattr(t, "DEV", "cpu")
    assert [s for s, _ in t.SHAPES] == [(16, 1024, 8, 64), (4, 2048, 16, 64), (8, 4096, 16, 64)]
    for shape, kind in t.SHAPES[1:]:  # the larger shapes: their plan assertions only
        plans = [drv.dense_backward_plan(*shape, f) for f in (0, 1, 2)]
        assert plans[0][3] == 1 and [p[14] for p in plans] == [0, 1, 2] and (plans[1][2], int(plans[1][9] > 1)) == kind
    with pytest.warns(RuntimeWarning, match="loop_form"):
        t.test_two_step_prefetch_equals_the_default_backward(*t.SHAPES[0])
    assert drv._dense_bwd_form == (0, 0) and "bwd_pipe" in drv._enabled          # the form is put back afterwards
    r = _load("wip_rank_sort_gpu")
    with pytest.warns(RuntimeWarning, match="rank_sort=1"):
        r.test_backward_on_merge_sort_ranks_equals_the_default_backward()
    assert drv._dense_bwd_form == (0, 0) and "rank_merge" in drv._enabled
