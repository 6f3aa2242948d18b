"""The reference's two model-level call patterns (tests/model_blocks.py) through the CPU operator package,
float32 and float64, forward and gradients down to the inputs and weights, against the same graph in float64 with
the closed form for the logits.  The GPU operators run the same blocks in the GPU tests."""
import pytest
import torch

import closed_forms as cf
import model_blocks as mb


@pytest.mark.parametrize("dtype,ftol,gtol", [(torch.float64, 1e-12, 1e-12), (torch.float32, 1e-5, 1e-4)])
def test_setfind_block_on_the_cpu_package(dtype, ftol, gtol):
    import l1attn_cpp
    batch, ntok, d_model, n_head = 3, 21, 32, 4
    got = mb.setfind_leaves(batch, ntok, d_model, n_head, dtype, "cpu")
    ref = mb.setfind_leaves(batch, ntok, d_model, n_head, torch.float64, "cpu")
    out = mb.setfind_block(*got, l1attn_cpp.L1Attn(), n_head)
    out_ref = mb.setfind_block(*ref, cf.dense_attn, n_head)
    gout = torch.randn(out.shape, generator=torch.Generator().manual_seed(5))
    out.backward(gout.to(dtype))
    out_ref.backward(gout.double())
    assert cf.rel_err(out.detach(), out_ref.detach()) <= ftol
    for a, b in zip(got, ref):
        assert cf.rel_err(a.grad, b.grad) <= gtol


@pytest.mark.parametrize("dtype,ftol,gtol", [(torch.float64, 1e-12, 1e-12), (torch.float32, 1e-5, 1e-4)])
def test_split_block_on_the_cpu_package(dtype, ftol, gtol):
    import l1attn_cpp
    bs, n_ctx, width, n_head = 2, 24, 48, 3
    got = mb.split_leaves(bs, n_ctx, width, dtype, "cpu")
    ref = mb.split_leaves(bs, n_ctx, width, torch.float64, "cpu")
    out = mb.split_block(*got, l1attn_cpp.L1Attn(), n_head)
    out_ref = mb.split_block(*ref, cf.dense_attn, n_head)
    gout = torch.randn(out.shape, generator=torch.Generator().manual_seed(6))
    out.backward(gout.to(dtype))
    out_ref.backward(gout.double())
    assert cf.rel_err(out.detach(), out_ref.detach()) <= ftol
    for a, b in zip(got, ref):
        assert cf.rel_err(a.grad, b.grad) <= gtol


@pytest.mark.parametrize("dtype,ftol,gtol", [(torch.float64, 1e-12, 1e-11), (torch.float32, 1e-5, 1e-4)])
def test_setfind_block_with_the_fused_operator(dtype, ftol, gtol):
    """The reference's transformer block with the fused operator in place of its five steps from the zero-token
    padding to the einsum (no padding is needed, the no-op is part of the operator), against the reference's own
    graph in float64 with the closed form for the logits."""
    import l1attn_cpp
    batch, ntok, d_model, n_head = 3, 21, 32, 4

    def block_fused(x, wq, wv, wk):
        q = (x @ wq).reshape(batch, ntok, n_head, d_model)
        v = (x @ wv).reshape(batch, ntok, n_head, d_model)
        k = x.unsqueeze(2).expand(-1, -1, n_head, -1) * wk.unsqueeze(0).unsqueeze(0)
        return l1attn_cpp.L1AttnFused()(q, k, v).sum(2)

    got = mb.setfind_leaves(batch, ntok, d_model, n_head, dtype, "cpu")
    ref = mb.setfind_leaves(batch, ntok, d_model, n_head, torch.float64, "cpu")
    out = block_fused(*got)
    out_ref = mb.setfind_block(*ref, cf.dense_attn, n_head)
    gout = torch.randn(out.shape, generator=torch.Generator().manual_seed(5))
    out.backward(gout.to(dtype))
    out_ref.backward(gout.double())
    assert cf.rel_err(out.detach(), out_ref.detach()) <= ftol
    for a, b in zip(got, ref):
        assert cf.rel_err(a.grad, b.grad) <= gtol
