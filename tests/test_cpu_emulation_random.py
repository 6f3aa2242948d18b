"""A seeded handful of random shapes through the CPU-emulated HIP kernels (fused forward and backward stage, plain
and pipelined; sparse and bidirectional in all four row types, hubs included; merge-sort ranks), under
AddressSanitizer, against the closed forms.  The fixed cases of the other emulation tests cover the corner
shapes by design; this one guards against the corner nobody thought of.  Kept to a few dozen seconds; the same
generator ran for two hours once (1078 cases) without a finding; L1ATTN_RANDOM_CASES=<n> and
L1ATTN_RANDOM_SEED=<s> in the environment run it longer or elsewhere."""
import os
import random
import struct
import subprocess

import numpy as np
import pytest
import torch

import closed_forms as cf
import test_cpu_emulation as tf
import test_cpu_emulation_sparse as ts

ENV = dict(os.environ, ASAN_OPTIONS="verify_asan_link_order=0:detect_leaks=0")


def _fused_case(rng, exe, d):
    W = rng.choice([16, 32, 48, 64, 96, 7, 33, 20])
    Wv = W if rng.random() < 0.8 else rng.choice([W, 12, 5])
    B, T, H = rng.randint(1, 2), rng.randint(1, 110), rng.randint(1, 12)
    if B * T * T * H * max(W, Wv) > 3e6:
        T = max(1, T // 3)
    g = torch.Generator().manual_seed(rng.randrange(1 << 30))
    q, k = (torch.randn(B, T, H, W, generator=g) for _ in range(2))
    v = torch.randn(B, T, H, Wv, generator=g)
    r = tf._run(exe, d, q, k, v, pipe=(W in (32, 64) and W == Wv and rng.random() < 0.5))
    ref, ref_lse = tf._ref(q, k, v)
    assert cf.rel_err(r["vo"], ref) <= 1e-5 and cf.rel_err(r["lse"], ref_lse) <= 1e-5, (B, T, H, W, Wv)
    tf._check_backward(r, q, k, v, 1e-4)


def _sparse_case(rng, exe, d):
    B, T, H = rng.randint(1, 2), rng.randint(1, 50), rng.randint(1, 20)
    W = rng.choice([1, 3, 4, 8, 12, 16, 32, 64, 70, 5])
    Wv = W if rng.random() < 0.7 else rng.choice([4, 8, 12, 7])
    E = rng.randint(1, 450)
    g = torch.Generator().manual_seed(rng.randrange(1 << 30))
    co = torch.randint(0, T, (E, 2), generator=g)
    if E > 300 and rng.random() < 0.6:  # a hub in each direction: segments beyond the long-segment threshold
        co[:160, 0] = rng.randrange(T)
        co[160:300, 1] = rng.randrange(T)
        co = co[torch.randperm(E, generator=g)]
    kind = rng.choice(["f32", "f64", "f16", "bf16"])
    sm, bidi = rng.random() < 0.6, rng.random() < 0.5
    dt = ts.TORCH_T.get(kind, torch.float32)
    q, k = (torch.randn(B, T, H, W, generator=g).to(dt).float() for _ in range(2))
    vf, vb = (torch.randn(B, T, H, Wv, generator=g).to(dt).float() for _ in range(2))
    vo, _, _ = ts._run(exe, d, vf, vb, q, k, co, sm, bidi, kind)
    x = [t.double() for t in (vf, vb, q, k)]
    ref = cf.bidi_value(*x, co, sm) if bidi else cf.sparse_value(x[0], x[2], x[3], co, sm)
    exact = kind in ("f32", "f64")
    if exact or float(ref.abs().max()) > 1e-4:  # (16-bit outputs below the type's range say nothing)
        assert cf.rel_err(vo, ref) <= ({"f32": 1e-5, "f64": 1e-12}.get(kind) or ts.TOL[kind]), (B, T, H, W, Wv, E, kind)
    _, dvf, _, dq, dk = ts._run.grads
    if exact or max(float(t.abs().max()) for t in (dvf, dq, dk)) > 1e-4:
        ts._check_grads(vf, vb, q, k, co, sm, bidi, {"f32": 1e-4, "f64": 1e-11}.get(kind) or ts.TOL[kind])


def _ranks_case(rng, exe, d):
    B, H, W = 1, rng.randint(1, 2), rng.randint(1, 2)
    T = rng.choice([rng.randint(1, 600), rng.randint(500, 2200), rng.randint(2000, 4200)])
    g = torch.Generator().manual_seed(rng.randrange(1 << 30))
    q, k = (torch.randn(B, T, H, W, generator=g) for _ in range(2))
    if rng.random() < 0.5:
        q, k = torch.round(q * 3), torch.round(k * 3)
    fin, fout = str(d / "in.bin"), str(d / "out.bin")
    with open(fin, "wb") as f:
        f.write(struct.pack("4q", B, T, H, W))
        f.write(q.numpy().tobytes())
        f.write(k.numpy().tobytes())
    r = subprocess.run([exe, fin, fout], env=ENV, capture_output=True, text=True)
    assert r.returncode == 0, r.stderr[-500:]
    raw, n = open(fout, "rb").read(), B * T * H * W
    rq = np.frombuffer(raw, np.float32, n).reshape(B, T, H, W)
    rk = np.frombuffer(raw, np.float32, n, n * 4).reshape(B, T, H, W)
    a, b = tf._reference_ranks(q, k)
    assert np.array_equal(rq, a) and np.array_equal(rk, b), (T, H, W)


@pytest.mark.skipif(not os.path.exists(ts.CLANG), reason="needs ROCm's clang++ as host compiler")
def test_random_shapes_through_the_emulated_kernels(tmp_path, emu_fused, emu_sparse, emu_ranks):
    d = tmp_path
    exes = {"fused": emu_fused, "sparse": emu_sparse, "ranks": emu_ranks}
    rng = random.Random(int(os.environ.get("L1ATTN_RANDOM_SEED", "20240607")))
    for i in range(int(os.environ.get("L1ATTN_RANDOM_CASES", "2"))):
        name, fn = (("fused", _fused_case), ("sparse", _sparse_case), ("sparse", _sparse_case), ("ranks", _ranks_case))[i % 4]
        fn(rng, exes[name], d)
