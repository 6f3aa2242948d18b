"""CPU-only: the yardstick side of the late GPU tests, walked without a GPU.

tests/test_y_configs_gpu.py compares the GPU operators with the oracle and the closed forms.  The CPU operator
package has the same Python surface, so here those test functions run with the CPU modules standing where the
GPU modules would be imported and the device set to the CPU: a slip in a test's own reference computation, shapes
or tolerances shows here rather than on the first GPU run.  The fast backward's sign range is walked with a torch
model of the kernel's arithmetic in place of the launch."""
import math
import sys

import pytest
import torch


@pytest.fixture()
def gpu_tests_on_cpu(monkeypatch):
    import l1attn_cpp, l1attn_drv_cpp, l1attn_sparse_bidi_drv, l1attn_sparse_cpp, l1attn_sparse_drv
    for name, mod in (("l1attn_cuda_drv", l1attn_drv_cpp), ("l1attn_sparse_cuda_drv", l1attn_sparse_drv),
                      ("l1attn_sparse_bidi_cuda_drv", l1attn_sparse_bidi_drv), ("l1attn_sparse_cuda", l1attn_sparse_cpp),
                      ("l1attn_cuda", l1attn_cpp)):
        monkeypatch.setitem(sys.modules, name, mod)
    import test_y_configs_gpu as t
    monkeypatch.setattr(t, "DEV", torch.device("cpu"))
    return t


def test_stand_in_and_model_block_tests_walk_on_the_cpu_package(gpu_tests_on_cpu):
    gpu_tests_on_cpu.test_native_module_stand_ins_on_the_gpu()
    gpu_tests_on_cpu.test_model_blocks_on_the_gpu()
    gpu_tests_on_cpu.test_training_steps_on_the_gpu_operator_match_torch_autograd()


def test_sign_range_test_walks_on_a_model_of_the_kernel(gpu_tests_on_cpu, monkeypatch):
    import _l1attn_hip as drv
    t = gpu_tests_on_cpu

    def model(q, k, da):
        W = q.shape[-1]
        scale = -1 / math.sqrt(W)
        x = torch.cat([q.flatten(), k.flatten()]).abs()
        outside = bool((~(x < 2.0 ** 63)).any() or ((x != 0) & (x < 2.0 ** -41)).any())   # what the pre-pass flags
        if q.dtype == torch.float64 or q.shape[2] * W < 32 or outside:                      # exact comparisons
            s = torch.sign(q[:, None].double() - k[:, :, None].double())
            s = torch.nan_to_num(s, nan=0.0)                                                  # inf - inf: neither > 0 nor < 0
        else:                                                     # float32: clamp((q*2^64 - k*2^64), -1, 1)
            s = ((q * 2.0 ** 64)[:, None] - (k * 2.0 ** 64)[:, :, None]).clamp(-1, 1).double()
        dq = scale * torch.einsum("bsthw,bsth->bthw", s, da.double())
        dk = -scale * torch.einsum("bsthw,bsth->bshw", s, da.double())
        return dq.to(q.dtype), dk.to(q.dtype)

    monkeypatch.setattr(t, "_dense_bwd_gpu", model)
    drv.lib()  # the real library: the test asks it how it would tile the shapes (host code, no launch)
    t.test_sign_domain_of_the_fast_float32_backward()
