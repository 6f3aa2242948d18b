"""GPU parity of the merge-sort column-rank kernel (csrc/rank_sort.hip) against the library-sort kernel that the
backward uses by default: the two must give identical rq and rk, and the whole backward through
l1attn_dense_bwd_ex_f32(rank_sort=1) must equal the default backward bit for bit.

This file has not run on a GPU yet, which is why its name keeps it out of pytest's collection
(run it as `python -m pytest tests/wip_rank_sort_gpu.py -m gpu`); rename it to test_*.py once it has passed there.
The kernel itself runs on the CPU in tests/test_cpu_emulation.py::test_column_rank_kernels_on_cpu.
"""
import os

import pytest
import torch

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.mark.parametrize("shape", [(2, 64, 2, 8), (1, 513, 2, 3), (1, 2048, 4, 16), (2, 4096, 2, 64), (1, 8192, 1, 8),
                                   (1, 3000, 3, 5)])
def test_merge_sort_ranks_equal_the_library_sort_ranks(shape):
    import _l1attn_hip as drv
    L = drv.lib()
    B, T, H, W = shape
    print("case merge-sort ranks", shape, flush=True)
    g = torch.Generator().manual_seed(sum(shape))
    q, k = (torch.randn(B, T, H, W, generator=g) for _ in range(2))
    idx = torch.randperm(T, generator=g)[: T // 8]
    q[:, idx] = k[:, idx.flip(0)]
    q[..., 0] = 0.0
    k[..., 0] = -0.0
    q[..., 1] = torch.round(q[..., 1])
    k[..., 1] = torch.round(k[..., 1])
    qd, kd = q.cuda(), k.cuda()
    out = [torch.empty_like(qd) for _ in range(4)]
    st = drv.stream_of(qd)
    assert L.l1attn_dense_column_ranks_f32(drv.ptr(qd), drv.ptr(kd), drv.ptr(out[0]), drv.ptr(out[1]), B, T, H, W, st) == 0
    assert L.l1attn_dense_column_ranks_merge_f32(drv.ptr(qd), drv.ptr(kd), drv.ptr(out[2]), drv.ptr(out[3]), B, T, H, W, st) == 0
    torch.cuda.synchronize()
    assert torch.equal(out[2], out[0]) and torch.equal(out[3], out[1])


def test_backward_on_merge_sort_ranks_equals_the_default_backward():
    """l1attn_dense_bwd_ex_f32 with rank_sort = 1 against the default entry point on one seeded problem of the
    rank path (T = 2048, 32 heads of 64 columns): bit-equal dq and dk."""
    import _l1attn_hip as drv
    B, T, H, W = 3, 2048, 32, 64
    assert drv.dense_backward_plan(B, T, H, W)[2] == 1
    g = torch.Generator().manual_seed(5)
    q, k = (torch.randn(B, T, H, W, generator=g).cuda() for _ in range(2))
    da = torch.empty(B, T, T, H)
    for b in range(B):
        da[b].normal_(generator=g)
    da = da.cuda()
    print("case backward with rank sort: default", flush=True)
    dq0, dk0 = drv.dense_backward(da, q, k)
    torch.cuda.synchronize()
    drv.enable_experimental("rank_merge")
    old = drv.set_dense_backward_form(rank_sort=1)
    try:
        print("case backward with rank sort: merge", flush=True)
        dq1, dk1 = drv.dense_backward(da, q, k)
        torch.cuda.synchronize()
    finally:
        drv.set_dense_backward_form(*old)
    assert torch.equal(dq0, dq1) and torch.equal(dk0, dk1)
