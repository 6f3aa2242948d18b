"""Arithmetic model of the experimental fixed-point forward (l1attn_dense_fwd_fixed_f32), in numpy, against
the oracle.  The model restates what the three kernels do per (batch, head) -- grid g = max(|q|,|k|) * 2^-24
in fp32, u = rint(x / g) with an fp32 division, exact integer sum of |u_q - u_k| over W, logit =
float(sum) * (scale * g) in fp32 -- and checks the two claims the entry point's documentation makes: the sum
is at most 2^31 for W <= 64 (the accumulator is 32 bits unsigned), and the logits are within 1e-5 of the largest logit of the fp64 reference
(about 1e-7 on N(0,1) and LayerNorm-scaled inputs).  It is a model of the kernels, not the kernels: their
parity test is a GPU test."""
import math

import numpy as np
import pytest
import torch

from oracle import oracle


def _model(q, k):
    """q, k: float32 [T, W] of one (batch, head) -> logits [S, T] float32."""
    m = np.float32(max(np.abs(q).max(), np.abs(k).max()))
    g = max(m * np.float32(2.0 ** -24), np.float32(1.17549435e-38))
    uq = np.rint((q / g).astype(np.float32)).astype(np.int64)
    uk = np.rint((k / g).astype(np.float32)).astype(np.int64)
    assert np.abs(uq).max() <= 2 ** 24 and np.abs(uk).max() <= 2 ** 24
    s = np.abs(uq[None, :, :] - uk[:, None, :]).sum(-1)
    assert s.max() <= 2 ** 31  # 64 * 2^25 at most: inside the 32 unsigned bits of the accumulator
    scale = np.float32(-1.0 / math.sqrt(q.shape[1]))
    return s.astype(np.float32) * np.float32(scale * g)


def _inputs(kind, rng, T, W):
    x = rng.standard_normal((T, W))
    if kind == "layernorm":
        x = (x - x.mean(1, keepdims=True)) / x.std(1, keepdims=True)
    elif kind == "outliers":
        x = x * np.where(rng.random((T, W)) < 0.001, 1000.0, 1.0)
    elif kind == "offset":
        x = x + 100.0
    elif kind == "tiny":
        x = x * 1e-30
    elif kind == "zero":
        x = x * 0.0
    return x.astype(np.float32)


@pytest.mark.parametrize("kind,bound", [("randn", 5e-7), ("layernorm", 5e-7), ("outliers", 1e-5), ("offset", 1e-5),
                                        ("tiny", 5e-7), ("zero", 0.0)])
@pytest.mark.parametrize("W", [32, 64])
def test_fixed_point_model_within_forward_tolerance(kind, bound, W):
    rng = np.random.default_rng(7 + W)
    T = 256
    q, k = _inputs(kind, rng, T, W), _inputs(kind, rng, T, W)
    a = _model(q, k)
    tq, tk = (torch.from_numpy(x.astype(np.float64)).view(1, T, 1, W) for x in (q, k))
    ref = oracle.dense_fwd(tq, tk)[0, :, :, 0].numpy()
    err = np.abs(a - ref).max() / max(np.abs(ref).max(), 1e-300)
    assert err <= bound, err


def test_fixed_point_model_extremes():
    # every difference at its largest: q = +m, k = -m in all 64 columns -> |u_q - u_k| = 2^25 each and the sum is
    # 64 * 2^25 = 2^31, the largest value the accumulator ever holds; the logit is exact
    q = np.full((4, 64), 3.0, np.float32)
    k = np.full((4, 64), -3.0, np.float32)
    a = _model(q, k)
    assert np.all(a == np.float32(-6.0 * 64 / 8.0))
