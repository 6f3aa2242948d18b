"""GPU parity at the benchmark configurations' full sizes, the documented domain of the fast backward's sign, the
stand-ins for the reference's native modules, and the reference's model-level call patterns.

Collected after the other GPU test files on purpose (pytest runs files in name order): these are the long cases.
The checks themselves are tests/config_checks.py, which tests/test_config_checks_cpu.py runs on the CPU package
at reduced sizes.

Tolerances: float32 against float64 closed forms on the same float32-valued inputs, max|x-ref|/max|ref| <= 1e-5
forward, <= 1e-4 gradients.
"""
import math

import pytest
import torch

import closed_forms as cf
import config_checks as cc
import model_blocks as mb
from oracle import oracle

pytestmark = pytest.mark.gpu
DEV = torch.device("cuda:0")


def test_config2_full_batch_with_downstream_softmax_and_einsum():
    """B=16, T=1024, H=8, W=64: the operator on the whole batch (logits 0.5 GiB), yardstick batch by batch."""
    print("case config 2 at full size", flush=True)
    import l1attn_cuda
    errs = cc.dense_with_downstream(l1attn_cuda, DEV, 16, 1024, 8, 64)
    print("errors (logits, output, dq, dk):", errs, flush=True)
    assert errs[0] <= cc.FWD_TOL and errs[1] <= cc.FWD_TOL and errs[2] <= cc.BWD_TOL and errs[3] <= cc.BWD_TOL


def test_config3_full_size_layernorm_scaled_inputs():
    """B=8, T=4096, H=16, W=64 with the configuration's second input set (unit variance per token and head):
    sampled rows of the logits and both gradients in float64, the checksum and bitwise repeatability.  (The N(0,1)
    input set at this size is tests/test_dense_gpu.py::test_dense_headline_size_properties.)"""
    print("case config 3 at full size, LayerNorm-scaled inputs", flush=True)
    import _l1attn_hip as drv
    errs = cc.dense_sampled_rows(drv, DEV, 8, 4096, 16, 64, True, [(0, 0), (3, 5), (7, 4095), (5, 2049)])
    print("errors (logits, dq, dk, checksum):", errs, flush=True)
    assert errs[0] <= cc.FWD_TOL and errs[1] <= cc.BWD_TOL and errs[2] <= cc.BWD_TOL and errs[3] <= 1e-4
    torch.cuda.empty_cache()


def test_config4_full_size():
    """B=4, T=4096, H=8, W=32, degrees U{1..64}: about 133 k edges."""
    print("case config 4 at full size", flush=True)
    import l1attn_sparse_cuda
    E, errs = cc.sparse_uniform_graph(l1attn_sparse_cuda, DEV, 4, 4096, 8, 32)
    print("edges", E, "errors (vo, dv, dq, dk):", errs, flush=True)
    assert 120_000 <= E <= 146_000
    assert errs[0] <= cc.FWD_TOL and max(errs[1:]) <= cc.BWD_TOL


def test_config5_full_size():
    """B=1, T=65536, H=4, W=64, Zipf degrees clipped to [1, 2048] plus self loops: about 1.08 M edges."""
    print("case config 5 at full size", flush=True)
    import l1attn_sparse_bidi_cuda
    E, dmx, errs = cc.bidi_powerlaw_graph(l1attn_sparse_bidi_cuda, DEV, 1, 65536, 4, 64)
    print("edges", E, "dst_mxlen", dmx, "errors (vo, dvf, dvb, dq, dk):", errs, flush=True)
    assert 900_000 <= E <= 1_300_000 and dmx >= 1024
    assert errs[0] <= cc.FWD_TOL and max(errs[1:]) <= cc.BWD_TOL
    torch.cuda.empty_cache()


def _dense_bwd_gpu(q, k, da):
    import _l1attn_hip as drv
    dq, dk = drv.dense_backward(da.to(DEV), q.to(DEV), k.to(DEV))
    torch.cuda.synchronize()
    return dq.cpu(), dk.cpu()


def test_sign_domain_of_the_fast_float32_backward():
    """The float32 backward below 2048 tokens takes sign(q-k) as clamp((q - k) * 2^64, -1, 1) with q and k scaled
    first: exact while every magnitude is below 2^63 and every non-zero one at least 2^-41 (inputs scaled by 2^-20
    and 2^40 are inside).  A pre-pass of the same call checks that on the device, and outside it -- inputs scaled by
    2^-70, whose differences the scaling leaves fractional; by 2^64, which it overflows; one subnormal or infinite
    value -- dq and dk are recomputed with comparisons, so every case matches the oracle, whose sign() is the
    reference's comparison (cpp/l1attn_drv.cpp:7-11).  The float64 entry point and the generic float32 kernels
    (fewer than 16 tokens or fewer than 32 columns per token) compare exactly to begin with."""
    print("case sign domain", flush=True)
    import _l1attn_hip as drv
    B, T, H, W = 1, 192, 8, 64
    info = (drv.ctypes.c_int64 * 16)()
    assert drv.lib().l1attn_dense_bwd_plan_info(B, T, H, W, info) == 0
    assert info[0] == 1 and info[2] == 0 and info[15] == 256   # tiled path without column ranks: the form described above
    g = torch.Generator().manual_seed(77)
    q0, k0 = torch.randn(B, T, H, W, generator=g), torch.randn(B, T, H, W, generator=g)
    k0[0, 1] = q0[0, 2]                            # exact ties stay exact under scaling by powers of two
    da = torch.randn(B, T, T, H, generator=g)
    for e in (-20, 40, -70, 64):
        print("case sign domain: inputs scaled by 2^%d" % e, flush=True)
        q, k = q0 * 2.0 ** e, k0 * 2.0 ** e
        x = torch.cat([q.flatten(), k.flatten()]).abs()
        inside = float(x.max()) < 2.0 ** 63 and float(x[x != 0].min()) >= 2.0 ** -41
        assert inside == (e in (-20, 40))
        dq, dk = _dense_bwd_gpu(q, k, da)
        rdq, rdk = oracle.dense_bwd(da.double(), q.double(), k.double())
        assert cf.rel_err(dq, rdq) <= cc.BWD_TOL and cf.rel_err(dk, rdk) <= cc.BWD_TOL, e
    for where, value in (((0, 100, 3, 31), 1e-40), ((0, 5, 2, 7), float("inf"))):
        print("case sign domain: one value", value, flush=True)
        q, k = q0.clone(), k0.clone()
        k[where] = value
        dq, dk = _dense_bwd_gpu(q, k, da)
        rdq, rdk = oracle.dense_bwd(da.double(), q.double(), k.double())
        assert cf.rel_err(dq, rdq) <= cc.BWD_TOL and cf.rel_err(dk, rdk) <= cc.BWD_TOL, value
    # float64 and the generic float32 kernels have no such range
    for e in (-70, 62):
        q, k = (q0 * 2.0 ** e).double(), (k0 * 2.0 ** e).double()
        dq, dk = _dense_bwd_gpu(q, k, da.double())
        rdq, rdk = oracle.dense_bwd(da.double(), q, k)
        assert cf.rel_err(dq, rdq) <= 1e-12 and cf.rel_err(dk, rdk) <= 1e-12, e
        # fewer than 32 columns per token: the generic float32 kernels
        qn, kn, dan = q0[:, :, :2, :7].contiguous() * 2.0 ** e, k0[:, :, :2, :7].contiguous() * 2.0 ** e, da[..., :2].contiguous()
        assert drv.lib().l1attn_dense_bwd_plan_info(B, T, 2, 7, info) == 0 and info[0] == 0 and info[15] == 0
        dq, dk = _dense_bwd_gpu(qn, kn, dan)
        rdq, rdk = oracle.dense_bwd(dan.double(), qn.double(), kn.double())
        assert cf.rel_err(dq, rdq) <= cc.BWD_TOL and cf.rel_err(dk, rdk) <= cc.BWD_TOL, e


def test_native_module_stand_ins_on_the_gpu():
    """l1attn_cuda_drv / l1attn_sparse_cuda_drv / l1attn_sparse_bidi_cuda_drv called the way the reference's own
    autograd Functions call them (cuda/l1attn_cuda.py:9-24, cuda/l1attn_sparse_cuda.py:10-47,
    cuda/l1attn_sparse_bidi_cuda.py:10-48), against the oracle."""
    print("case native module stand-ins", flush=True)
    import l1attn_cuda_drv, l1attn_sparse_cuda_drv, l1attn_sparse_bidi_cuda_drv
    import l1attn_sparse_cuda
    g = torch.Generator().manual_seed(31)
    B, T, H, W = 2, 40, 4, 32
    q, k, v, vb, dvo = (torch.randn(B, T, H, W, generator=g) for _ in range(5))
    da = torch.randn(B, T, T, H, generator=g)
    qd, kd, vd, vbd, dvod = (x.to(DEV) for x in (q, k, v, vb, dvo))
    attn = l1attn_cuda_drv.forward(qd, kd)
    assert isinstance(attn, list) and len(attn) == 1
    d_q, d_k = l1attn_cuda_drv.backward(da.to(DEV), qd, kd)
    assert cf.rel_err(attn[0].cpu(), oracle.dense_fwd(q.double(), k.double())) <= cc.FWD_TOL
    rdq, rdk = oracle.dense_bwd(da.double(), q.double(), k.double())
    assert cf.rel_err(d_q.cpu(), rdq) <= cc.BWD_TOL and cf.rel_err(d_k.cpu(), rdk) <= cc.BWD_TOL
    with pytest.raises(RuntimeError, match="d_attn must be contiguous"):       # the reference driver's CHECK_INPUT
        l1attn_cuda_drv.backward(da.to(DEV).transpose(1, 2), qd, kd)
    co = torch.stack((torch.randint(0, T, (300,), generator=g), torch.randint(0, T, (300,), generator=g)), 1)
    coo, dmx, _ = l1attn_sparse_cuda.expandCoo(co.to(DEV), warn=False)
    ocoo = coo.cpu()
    for sm in (True, False):
        vo, saved = l1attn_sparse_cuda_drv.forward(vd, qd, kd, coo, dmx, sm)
        d_v, d_q, d_k = l1attn_sparse_cuda_drv.backward(dvod, vd, qd, kd, coo, saved, torch.tensor(dmx).item(),
                                                        torch.tensor(sm).item())
        rvo, rattn = oracle.sparse_fwd(v.double(), q.double(), k.double(), ocoo, dmx, sm)
        rg = oracle.sparse_bwd(dvo.double(), v.double(), q.double(), k.double(), ocoo, rattn, dmx, sm, 1)
        assert cf.rel_err(vo.cpu(), rvo) <= cc.FWD_TOL
        for x, y in zip((d_v, d_q, d_k), rg):
            assert cf.rel_err(x.cpu(), y) <= cc.BWD_TOL
        vo, saved = l1attn_sparse_bidi_cuda_drv.forward(vd, vbd, qd, kd, coo, dmx, sm)
        grads = l1attn_sparse_bidi_cuda_drv.backward(dvod, vd, vbd, qd, kd, coo, saved, dmx, sm)
        rvo, rattn = oracle.bidi_fwd(v.double(), vb.double(), q.double(), k.double(), ocoo, dmx, sm)
        rg = oracle.bidi_bwd(dvo.double(), v.double(), vb.double(), q.double(), k.double(), ocoo, rattn, dmx, sm, 1)
        assert cf.rel_err(vo.cpu(), rvo) <= cc.FWD_TOL
        for x, y in zip(grads, rg):
            assert cf.rel_err(x.cpu(), y) <= cc.BWD_TOL


def test_model_blocks_on_the_gpu():
    """The reference's two model-level call patterns (tests/model_blocks.py: the transformer block of
    example-setfind/setfind.py:98-138 and the torch.split block of example/model.py:46-59) through
    l1attn_cuda.L1Attn in float32, against the same graphs in float64 with the closed form for the logits."""
    print("case model blocks", flush=True)
    import l1attn_cuda
    batch, ntok, d_model, n_head = 3, 21, 32, 4
    got = mb.setfind_leaves(batch, ntok, d_model, n_head, torch.float32, DEV)
    ref = mb.setfind_leaves(batch, ntok, d_model, n_head, torch.float64, DEV)
    out = mb.setfind_block(*got, l1attn_cuda.L1Attn(), n_head)
    out_ref = mb.setfind_block(*ref, cf.dense_attn, n_head)
    gout = torch.randn(out.shape, generator=torch.Generator().manual_seed(5)).to(DEV)
    out.backward(gout)
    out_ref.backward(gout.double())
    assert cf.rel_err(out.detach(), out_ref.detach()) <= cc.FWD_TOL
    for a, b in zip(got, ref):
        assert cf.rel_err(a.grad, b.grad) <= cc.BWD_TOL
    bs, n_ctx, width, n_head = 2, 72, 192, 3      # heads of 64 columns: the tiled kernels behind strided views
    got = mb.split_leaves(bs, n_ctx, width, torch.float32, DEV)
    ref = mb.split_leaves(bs, n_ctx, width, torch.float64, DEV)
    out = mb.split_block(*got, l1attn_cuda.L1Attn(), n_head)
    out_ref = mb.split_block(*ref, cf.dense_attn, n_head)
    gout = torch.randn(out.shape, generator=torch.Generator().manual_seed(6)).to(DEV)
    out.backward(gout)
    out_ref.backward(gout.double())
    assert cf.rel_err(out.detach(), out_ref.detach()) <= cc.FWD_TOL
    for a, b in zip(got, ref):
        assert cf.rel_err(a.grad, b.grad) <= cc.BWD_TOL


def test_training_steps_on_the_gpu_operator_match_torch_autograd():
    """tests/test_training_loop_cpu.py's loop (a two-layer transformer on the reference example's task, six Adam
    steps) with l1attn_cuda.L1Attn in float64 on the GPU against the same graph on torch's autograd through the
    closed form: weights and losses agree to rounding."""
    print("case training loop", flush=True)
    import l1attn_cuda
    import test_training_loop_cpu as tl

    class OnGpu(torch.nn.Module):  # the loop's tensors live on the CPU; only the operator's run on the GPU
        def forward(self, q, k):
            return l1attn_cuda.L1Attn()(q.to(DEV), k.to(DEV)).cpu()

    net_a, loss_a = tl.train(OnGpu())
    net_b, loss_b = tl.train(cf.dense_attn)
    for la, lb in zip(loss_a, loss_b):
        assert abs(la - lb) <= 1e-9 * max(1.0, abs(lb))
    for pa, pb in zip(net_a.parameters(), net_b.parameters()):
        assert cf.rel_err(pa.detach(), pb.detach()) <= 1e-9
