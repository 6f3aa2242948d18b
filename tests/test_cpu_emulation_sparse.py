"""CPU run of the sparse and bidirectional kernels, forward and backward (csrc/sparse.hip compiled for the host against
tests/cpu_emu/hip/hip_runtime.h: GPU threads are OS threads, cross-lane reads, fences and __syncthreads() are
barriers) under AddressSanitizer, for float32, float64, float16 and bfloat16 rows, against fp64 closed forms
and torch autograd through them.

It covers what the 16-bit entry points add to kernels that the GPU tests already cover in float32 and float64:
conversion on load, rounding on store, 8-byte row pieces, and the claim their GPU test rests on -- that the
one-directional 16-bit result is the float32 result rounded once (bit for bit) and the weights are the float32
weights.  The plan (dst- and src-sorted views of the edge list) is built here with numpy in the layout of
csrc/plan.h; the GPU plan builder is not part of this run.  Needs ROCm's clang++ as the host compiler (for
_Float16 and __bf16); skipped where it is absent.
"""
import os
import struct
import subprocess

import numpy as np
import pytest
import torch

import closed_forms as cf
from oracle import oracle

HERE = os.path.dirname(os.path.abspath(__file__))
EMU = os.path.join(HERE, "cpu_emu")
CLANG = "/opt/rocm/llvm/bin/clang++"
TYPES = {"f32": 0, "f64": 1, "f16": 2, "bf16": 3}
LONG = 128  # PLAN_LONG_SEGMENT of csrc/plan.h

pytestmark = pytest.mark.skipif(not os.path.exists(CLANG), reason="needs ROCm's clang++ as host compiler")


@pytest.fixture(scope="module")
def runner(emu_sparse):
    return emu_sparse


def _plan_arrays(co, T):
    """dst_ptr, src_ptr [T+2], csr_src, csr_row, csc_dst, csc_slot [E], long_dst, long_src (csrc/plan.h)."""
    dst, src = co[:, 0].numpy().astype(np.int64), co[:, 1].numpy().astype(np.int64)
    E = dst.shape[0]
    od = np.argsort(dst, kind="stable")
    slot_of_row = np.empty(E, np.int64)
    slot_of_row[od] = np.arange(E)
    os_ = np.argsort(src, kind="stable")

    def ptr(key):
        p = np.zeros(T + 2, np.int64)
        p[1:T + 1] = np.cumsum(np.bincount(key, minlength=T))
        p[T + 1] = E  # segment T: rows dropped for a bad index (none here)
        return p

    dp, sp = ptr(dst), ptr(src)
    long_d = np.nonzero(np.diff(dp[:T + 1]) > LONG)[0]
    long_s = np.nonzero(np.diff(sp[:T + 1]) > LONG)[0]
    i32 = lambda a: np.ascontiguousarray(a, dtype=np.int32)
    return [i32(dp), i32(sp), i32(src[od]), i32(od), i32(dst[os_]), i32(slot_of_row[os_]), i32(long_d), i32(long_s)]


def _run(exe, tmp_path, vf, vb, q, k, co, sm, bidi, kind, extra_env=None):
    B, T, H, W = q.shape
    Wv, E = vf.shape[3], co.shape[0]
    arrays = _plan_arrays(co, T)
    fin, fout = str(tmp_path / "in.bin"), str(tmp_path / "out.bin")
    with open(fin, "wb") as f:
        f.write(struct.pack("11q", B, T, H, W, Wv, E, int(sm), int(bidi), TYPES[kind], len(arrays[6]), len(arrays[7])))
        for a in arrays:
            f.write(a.tobytes())
        dvo = torch.randn(B, T, H, Wv, generator=torch.Generator().manual_seed(77))
        for x in (vf, vb, q, k, dvo):
            f.write(x.float().contiguous().numpy().tobytes())
    env = dict(os.environ, ASAN_OPTIONS="verify_asan_link_order=0:detect_leaks=0", **(extra_env or {}))
    r = subprocess.run([exe, fin, fout], env=env, capture_output=True, text=True)
    assert r.returncode == 0, (r.returncode, r.stderr[-2000:])
    raw = np.fromfile(fout, np.float64)
    nv = B * T * H * Wv
    vo = torch.from_numpy(raw[:nv].copy()).view(B, T, H, Wv)
    P = torch.from_numpy(raw[nv:nv + B * E * H].copy()).view(B, E, H)
    slot_row = torch.from_numpy(arrays[3].astype(np.int64))  # original row of each slot
    if True:  # the driver also ran the backward on dvo (rounded to the storage type)
        pos, nq = nv + B * E * H, B * T * H * W
        take = lambda n, shape: torch.from_numpy(raw[pos:pos + n].copy()).view(*shape)
        dvf = take(nv, (B, T, H, Wv)); pos += nv
        dvb = take(nv, (B, T, H, Wv)); pos += nv
        dq = take(nq, (B, T, H, W)); pos += nq
        dk = take(nq, (B, T, H, W)); pos += nq
        assert pos == raw.shape[0]
        dvo_s = dvo.to(TORCH_T[kind]) if kind in TORCH_T else dvo
        _run.grads = (dvo_s.double(), dvf, dvb, dq, dk)
    return vo, P, slot_row


def _check_grads(vf, vb, q, k, co, sm, bidi, tol):
    """The backward the last _run performed, against torch autograd through the fp64 closed form."""
    dvo, dvf, dvb, dq, dk = _run.grads
    x = [t.double().requires_grad_() for t in (vf, vb, q, k)]
    out = cf.bidi_value(x[0], x[1], x[2], x[3], co, sm) if bidi else cf.sparse_value(x[0], x[2], x[3], co, sm)
    ref = torch.autograd.grad(out, x, dvo, allow_unused=True)
    assert cf.rel_err(dvf, ref[0]) <= tol and cf.rel_err(dq, ref[2]) <= tol and cf.rel_err(dk, ref[3]) <= tol
    if bidi:
        assert cf.rel_err(dvb, ref[1]) <= tol


TOL = {"f16": 2.0 ** -10, "bf16": 2.0 ** -7}
TORCH_T = {"f16": torch.float16, "bf16": torch.bfloat16}


@pytest.mark.parametrize("shape,sm", [((2, 9, 3, 5, 5, 40), True),       # scalar path, dst rows without edges
                                      ((2, 9, 3, 5, 5, 40), False),
                                      ((1, 24, 8, 32, 32, 150), True),   # configuration-4 head geometry, 8-byte pieces
                                      ((1, 20, 3, 8, 12, 90), True),     # value width differs from key width
                                      ((1, 20, 3, 8, 12, 90), False)])
def test_sparse_forward_kernels_on_cpu(runner, tmp_path, shape, sm):
    B, T, H, W, Wv, E = shape
    g = torch.Generator().manual_seed(sum(shape))
    co = torch.randint(0, T, (E, 2), generator=g)
    for kind in ("f16", "bf16"):
        dt = TORCH_T[kind]
        q, k = (torch.randn(B, T, H, W, generator=g).to(dt).float() for _ in range(2))
        vf, vb = (torch.randn(B, T, H, Wv, generator=g).to(dt).float() for _ in range(2))
        # one-directional: float32 against the closed form, 16-bit == float32 rounded once, same weights
        vo32, P32, slot_row = _run(runner, tmp_path, vf, vb, q, k, co, sm, False, "f32")
        ref = cf.sparse_value(vf.double(), q.double(), k.double(), co, sm)
        assert cf.rel_err(vo32, ref) <= 1e-5
        p_ref = cf.edge_probs(q.double(), k.double(), co, sm)[:, slot_row]  # weights in slot order
        assert cf.rel_err(P32, p_ref) <= 1e-5
        _check_grads(vf, vb, q, k, co, sm, False, 1e-4)
        vo16, P16, _ = _run(runner, tmp_path, vf, vb, q, k, co, sm, False, kind)
        assert torch.equal(P16, P32)
        assert torch.equal(vo16.float(), vo32.float().to(dt).float())
        _check_grads(vf, vb, q, k, co, sm, False, TOL[kind])  # 16-bit gradients: one rounding on store
        # bidirectional: tolerance of the 16-bit type against the closed form
        vob, _, _ = _run(runner, tmp_path, vf, vb, q, k, co, sm, True, kind)
        ref = cf.bidi_value(vf.double(), vb.double(), q.double(), k.double(), co, sm)
        assert cf.rel_err(vob, ref) <= TOL[kind]
        _check_grads(vf, vb, q, k, co, sm, True, TOL[kind])
    # float64, both operators, forward and backward
    for bidi in (False, True):
        vo, _, _ = _run(runner, tmp_path, vf, vb, q, k, co, sm, bidi, "f64")
        ref = cf.bidi_value(vf.double(), vb.double(), q.double(), k.double(), co, sm) if bidi else \
            cf.sparse_value(vf.double(), q.double(), k.double(), co, sm)
        assert cf.rel_err(vo, ref) <= 1e-12
        _check_grads(vf, vb, q, k, co, sm, bidi, 1e-11)


def test_sparse_forward_long_segment_on_cpu(runner, tmp_path):
    """A dst with 150 incoming edges and a src with 140 outgoing ones: the workgroup-per-segment launch (eight
    waves, partial sums combined through LDS in wave order), float16 rows, both operators."""
    g = torch.Generator().manual_seed(4)
    B, T, H, W = 1, 40, 2, 16
    rows = [torch.stack((torch.full((150,), 5), torch.randint(0, T, (150,), generator=g)), 1),
            torch.stack((torch.randint(0, T, (140,), generator=g), torch.full((140,), 9)), 1),
            torch.randint(0, T, (30, 2), generator=g)]
    co = torch.cat(rows, 0)
    co = co[torch.randperm(co.shape[0], generator=g)]
    q, k, vf, vb = (torch.randn(B, T, H, W, generator=g).half().float() for _ in range(4))
    vo32, P32, _ = _run(runner, tmp_path, vf, vb, q, k, co, True, False, "f32")
    assert cf.rel_err(vo32, cf.sparse_value(vf.double(), q.double(), k.double(), co, True)) <= 1e-5
    vo16, P16, _ = _run(runner, tmp_path, vf, vb, q, k, co, True, False, "f16")
    assert torch.equal(P16, P32) and torch.equal(vo16.float(), vo32.float().half().float())
    vob, _, _ = _run(runner, tmp_path, vf, vb, q, k, co, True, True, "f16")
    assert cf.rel_err(vob, cf.bidi_value(vf.double(), vb.double(), q.double(), k.double(), co, True)) <= TOL["f16"]
    vob, _, _ = _run(runner, tmp_path, vf, vb, q, k, co, True, True, "f32")
    assert cf.rel_err(vob, cf.bidi_value(vf.double(), vb.double(), q.double(), k.double(), co, True)) <= 1e-5
    _check_grads(vf, vb, q, k, co, True, True, 1e-4)  # long segments in both backward passes



def test_sparse_kernels_under_thread_sanitizer(tmp_path, emu_sparse_tsan):
    """Forward and backward, one-directional and bidirectional, float32 and float16 rows, a hub in each direction
    (long segments): the wave-level exchanges through LDS and the workgroup barriers of sparse.hip leave no data
    race among the OS threads that stand for the lanes."""
    d, exe = tmp_path, emu_sparse_tsan
    env = {"TSAN_OPTIONS": "halt_on_error=1 report_signal_unsafe=0"}
    for (B, T, H, W, Wv, E, hub), kind, bidi in (((1, 24, 8, 32, 32, 150, False), "f32", True),
                                                 ((1, 30, 4, 64, 64, 400, True), "f32", False),
                                                 ((1, 30, 4, 64, 64, 400, True), "f16", True),
                                                 ((1, 20, 3, 8, 12, 90, False), "bf16", False)):
        g = torch.Generator().manual_seed(E)
        co = torch.randint(0, T, (E, 2), generator=g)
        if hub:
            co[:160, 0], co[160:300, 1] = 3, 5
        dt = TORCH_T.get(kind, torch.float32)
        q, k = (torch.randn(B, T, H, W, generator=g).to(dt).float() for _ in range(2))
        vf, vb = (torch.randn(B, T, H, Wv, generator=g).to(dt).float() for _ in range(2))
        vo, _, _ = _run(exe, d, vf, vb, q, k, co, True, bidi, kind, extra_env=env)
        x = [t.double() for t in (vf, vb, q, k)]
        ref = cf.bidi_value(*x, co, True) if bidi else cf.sparse_value(x[0], x[2], x[3], co, True)
        assert cf.rel_err(vo, ref) <= (1e-5 if kind == "f32" else TOL[kind])


def test_sparse_kernels_against_the_reference_extension_golden_vectors(runner, tmp_path):
    """Forward outputs of the reference's own compiled CPU extension (tests/golden/ref_cpp_golden.npz, written by
    tests/golden/make_golden.py: both edge lists, both `use_softmax`, one-directional and bidirectional) against
    the float64 kernels.  The runner takes its inputs as float32, so the comparison is at the rounding of the inputs
    (1e-6 of the largest output), not at the last bit."""
    z = np.load(os.path.join(HERE, "golden", "ref_cpp_golden.npz"))
    for tag in ("sA", "sB"):
        co = torch.from_numpy(z[tag + "_co"])
        v, vb, q, k = (torch.from_numpy(z["%s_%s" % (tag, n)]).float() for n in ("v", "vb", "q", "k"))
        for sm, name in ((True, "sm"), (False, "nsm")):
            vo, _, _ = _run(runner, tmp_path, v, vb, q, k, co, sm, False, "f64")
            assert cf.rel_err(vo, torch.from_numpy(z["%s_%s_vo" % (tag, name)])) <= 1e-6, (tag, name)
            vo, _, _ = _run(runner, tmp_path, v, vb, q, k, co, sm, True, "f64")
            assert cf.rel_err(vo, torch.from_numpy(z["%s_%s_bidi_vo" % (tag, name)])) <= 1e-6, (tag, name, "bidi")
