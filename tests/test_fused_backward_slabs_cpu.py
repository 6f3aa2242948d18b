"""CPU-only: the fused backward's walk through the batch in slabs (one shared buffer of logit gradients), with the
library's first stage replaced by a stand-in that computes the same thing from the host pointers it is handed and
the dense backward by the CPU package's.  What is checked is the driver's slicing: pointers, counts, the ragged last
slab, reuse of the buffer -- against torch autograd of the closed form, for every slab size."""
import contextlib
import ctypes

import numpy as np
import pytest
import torch

import closed_forms as cf


def _view(p, shape, dtype):
    n = int(np.prod(shape))
    buf = (ctypes.c_char * (n * np.dtype(dtype).itemsize)).from_address(p.value)
    return torch.from_numpy(np.frombuffer(buf, dtype=dtype).reshape(shape))


class _StageLib(object):
    """l1attn_fused_bwd_stage_{f32,f64} from their definitions: p = e^{a - lse}, dA[s,t] = p (v[s].dvo[t] -
    vo[t].dvo[t]), dv[s] = sum_t p dvo[t]."""
    calls = []

    def _stage(self, dtype):
        def stage(dvo, q, k, v, vo, lse, dA, dv, B, T, H, W, Wv, stream):
            _StageLib.calls.append(B)
            dvo, v, vo, dv = (_view(x, (B, T, H, Wv), dtype) for x in (dvo, v, vo, dv))
            q, k = (_view(x, (B, T, H, W), dtype) for x in (q, k))
            lse, dA = _view(lse, (B, T, H), dtype), _view(dA, (B, T, T, H), dtype)
            p = (cf.dense_attn(q, k) - lse[:, None]).exp()  # [b,s,t,h]
            dp = torch.einsum("bshw,bthw->bsth", v, dvo)
            dA.copy_(p * (dp - (vo * dvo).sum(-1)[:, None]))
            dv.copy_(torch.einsum("bsth,bthw->bshw", p, dvo))
            return 0
        return stage

    def __getattr__(self, name):
        if name == "l1attn_fused_bwd_stage_f32":
            return self._stage(np.float32)
        if name == "l1attn_fused_bwd_stage_f64":
            return self._stage(np.float64)
        raise AttributeError(name)


@pytest.mark.parametrize("dtype", [torch.float64, torch.float32])
def test_fused_backward_slabs(monkeypatch, dtype):
    import _l1attn_cpu as cpu
    import _l1attn_hip as drv
    monkeypatch.setattr(drv, "_enabled", set(drv.EXPERIMENTAL))
    monkeypatch.setattr(drv, "lib", lambda: _StageLib())
    monkeypatch.setattr(drv, "check_input", lambda x, name: None)
    monkeypatch.setattr(drv, "stream_of", lambda x: None)
    monkeypatch.setattr(drv, "dense_backward", lambda d, q, k: cpu.dense_backward(d, q, k))
    monkeypatch.setattr(torch.cuda, "device", lambda d: contextlib.nullcontext())
    B, T, H, W, Wv = 5, 9, 3, 6, 4
    g = torch.Generator().manual_seed(5)
    q, k = (torch.randn(B, T, H, W, generator=g, dtype=dtype) for _ in range(2))
    v, dvo = (torch.randn(B, T, H, Wv, generator=g, dtype=dtype) for _ in range(2))
    leaves = [x.clone().requires_grad_() for x in (q, k, v)]
    vo = cf.dense_then_value(*leaves, noop=True)
    want = torch.autograd.grad(vo, leaves, dvo)
    lse = torch.log1p(cf.dense_attn(q, k).exp().sum(1))
    entry = T * T * H * q.element_size()
    old = drv.set_fused_workspace_bytes(0)
    try:
        for budget, slabs in ((0, [1] * 5), (entry, [1] * 5), (2 * entry + 1, [2, 2, 1]), (3 * entry, [3, 2]),
                              (5 * entry, [5]), (1 << 30, [5])):
            drv.set_fused_workspace_bytes(budget)
            del _StageLib.calls[:]
            got = drv.dense_fused_backward(dvo, q, k, v, vo.detach().contiguous(), lse)
            assert _StageLib.calls == slabs, (budget, _StageLib.calls)
            for a, b in zip(got, want):
                assert cf.rel_err(a, b) <= (1e-12 if dtype == torch.float64 else 1e-5), budget
    finally:
        drv.set_fused_workspace_bytes(old)
    assert drv.fused_backward_slab(8, 4096, 16, 4) == 1 and old == 1 << 30  # 1 GiB per entry at the headline shape
    assert drv.fused_backward_slab(16, 1024, 8, 4) == 16
    with pytest.raises(ValueError):
        drv.set_fused_workspace_bytes(-1)
