"""GPU parity of the dense backward's pipelined step loops (csrc/dense.hip, dense_bwd_f32_fast<..., DEEP>: two steps
of prefetch distance, and the same with two LDS planes and one barrier per step) against the one-step form the
backward uses by default: the same sums in the same order, so dq and dk must be equal bit for bit, in the sign and
the rank form, with one or several tiles per workgroup.

This file has not run on a GPU yet, which is why its name keeps it out of pytest's collection
(run it as `python -m pytest tests/wip_bwd_prefetch_gpu.py -m gpu`); rename it to test_*.py once it has passed there.
The kernels run on the CPU in tests/test_cpu_emulation_dense.py (AddressSanitizer and ThreadSanitizer).
"""
import os

import pytest
import torch

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
DEV = "cuda"

# B, T, H, W and what bwd_plan makes of it: (rank, tiles per workgroup > 1)
SHAPES = [((16, 1024, 8, 64), (0, 0)),     # second baseline configuration: sign form, one tile per workgroup
          ((4, 2048, 16, 64), (1, 0)),     # rank form
          ((8, 4096, 16, 64), (1, 1))]     # headline configuration: rank form, four tiles per workgroup


@pytest.mark.parametrize("shape,kind", SHAPES)
def test_two_step_prefetch_equals_the_default_backward(shape, kind):
    """l1attn_dense_bwd_ex_f32 with loop_form 1 and 2 against the default entry point on the same seeded problem."""
    import _l1attn_hip as drv
    B, T, H, W = shape
    plans = [drv.dense_backward_plan(B, T, H, W, f) for f in (0, 1, 2)]
    assert plans[0][3] == 1 and [p[14] for p in plans] == [0, 1, 2]          # branch-free; the three forms
    assert (plans[1][2], int(plans[1][9] > 1)) == kind
    g = torch.Generator(device=DEV).manual_seed(5)
    q, k = (torch.randn(B, T, H, W, generator=g, device=DEV) for _ in range(2))
    da = torch.empty(B, T, T, H, device=DEV)
    for b in range(B):
        da[b].normal_(generator=g)
    print("case backward with prefetch distance: one_step", shape, flush=True)
    dq1, dk1 = drv.dense_backward(da, q, k)
    torch.cuda.synchronize()
    drv.enable_experimental("bwd_pipe")
    for form, name in ((1, "two_steps"), (2, "two_steps_two_planes")):
        old = drv.set_dense_backward_form(loop_form=form)
        try:
            print("case backward with prefetch distance:", name, shape, flush=True)
            dq2, dk2 = drv.dense_backward(da, q, k)
            torch.cuda.synchronize()
        finally:
            drv.set_dense_backward_form(*old)
        assert torch.equal(dq1, dq2) and torch.equal(dk1, dk2), name
