"""GPU parity of the dense backward's pipelined step loops (csrc/dense.hip, dense_bwd_f32_fast<..., DEEP>: two steps
of prefetch distance, and the same with two LDS planes and one barrier per step) against the one-step form the
backward uses by default: the same sums in the same order, so dq and dk must be equal bit for bit, in the sign and
the rank form, with one or several tiles per workgroup.

This file has not run on a GPU yet, which is why its name keeps it out of pytest's collection
(run it as `python -m pytest tests/wip_bwd_prefetch_gpu.py -m gpu`); rename it to test_*.py once it has passed there.
The kernels run on the CPU in tests/test_cpu_emulation_dense.py (AddressSanitizer and ThreadSanitizer).
"""
import ctypes
import os
import subprocess
import sys

import pytest
import torch

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))

# B, T, H, W and what bwd_plan makes of it: (rank, tiles per workgroup > 1)
SHAPES = [((16, 1024, 8, 64), (0, 0)),     # second baseline configuration: sign form, one tile per workgroup
          ((4, 2048, 16, 64), (1, 0)),     # rank form
          ((8, 4096, 16, 64), (1, 1))]     # headline configuration: rank form, four tiles per workgroup


@pytest.mark.parametrize("shape,kind", SHAPES)
def test_two_step_prefetch_equals_the_default_backward(tmp_path, shape, kind):
    """The prefetch distance is read from the environment once per process, so each run is a child process; both
    write dq and dk of the same seeded problem, and the plan they ran on."""
    code = (
        "import sys, ctypes, torch; sys.path.insert(0, %r); import _l1attn_hip as drv;"
        "B, T, H, W = %r; g = torch.Generator(device='cuda').manual_seed(5);"
        "q = torch.randn(B, T, H, W, generator=g, device='cuda'); k = torch.randn(B, T, H, W, generator=g, device='cuda');"
        "da = torch.empty(B, T, T, H, device='cuda');"
        "[da[b].normal_(generator=g) for b in range(B)];"
        "info = (ctypes.c_int64 * 16)(); assert drv.lib().l1attn_dense_bwd_plan_info(B, T, H, W, info) == 0;"
        "dq, dk = drv.dense_backward(da, q, k); torch.cuda.synchronize();"
        "torch.save([dq.cpu(), dk.cpu(), torch.tensor(list(info))], sys.argv[1])"
        % (os.path.join(ROOT, "l1-attention_amd"), shape))
    outs = []
    for name, env in (("one_step", {}), ("two_steps", {"L1ATTN_BWD_PREFETCH": "2"}),
                      ("two_steps_two_planes", {"L1ATTN_BWD_PREFETCH": "3"})):
        path = str(tmp_path / (name + ".pt"))
        print("case backward with prefetch distance:", name, shape, flush=True)
        subprocess.run([sys.executable, "-c", code, path], check=True, env=dict(os.environ, **env), timeout=300)
        outs.append(torch.load(path, weights_only=True))
    (dq1, dk1, plan1), (dq2, dk2, plan2), (dq3, dk3, plan3) = outs
    assert int(plan1[3]) == 1 and [int(p[14]) for p in (plan1, plan2, plan3)] == [0, 1, 2]   # branch-free; the three forms
    assert (int(plan2[2]), int(int(plan2[9]) > 1)) == kind
    assert torch.equal(dq1, dq2) and torch.equal(dk1, dk2)
    assert torch.equal(dq1, dq3) and torch.equal(dk1, dk3)
