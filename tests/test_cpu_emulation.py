"""CPU run of the fused operator's kernels (forward and the backward's first stage) (csrc/fused.hip compiled with g++ against the host-only
stand-in header tests/cpu_emu/hip/hip_runtime.h, every GPU thread executed in turn) under
AddressSanitizer and UBSan, checked against the oracle.

What this covers: the kernels' index arithmetic, clamps of ragged tiles and head groups, store
predicates, launch geometry and the XCD block permutation (every output element written, no access
outside exactly-sized buffers), and the host dispatch between the tiled and the generic kernel.
What it cannot cover: anything the hardware decides (scalar loads, occupancy, timing).  Only kernels
without LDS, barriers and cross-lane operations can be run this way.
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


@pytest.fixture(scope="module")
def runner(emu_fused):
    return emu_fused


@pytest.fixture(scope="module")
def runner_tsan(emu_fused_tsan):
    return emu_fused_tsan


def _run(exe, tmp_path, q, k, v, misalign=0, pipe=False):
    """-> dict: vo, lse, threads (forward), dA, dv, bwd_threads (first stage of the backward on a seeded dvo),
    and dvo itself."""
    B, T, H, W = q.shape
    Wv = v.shape[3]
    kind = "f32" if q.dtype == torch.float32 else "f64"
    dvo = torch.randn(B, T, H, Wv, generator=torch.Generator().manual_seed(99), dtype=q.dtype)
    fin, fout = str(tmp_path / "in.bin"), str(tmp_path / "out.bin")
    with open(fin, "wb") as f:
        f.write(struct.pack("5q", B, T, H, W, Wv))
        for x in (q, k, v, dvo):
            f.write(x.contiguous().numpy().tobytes())
    env = dict(os.environ, ASAN_OPTIONS="verify_asan_link_order=0:detect_leaks=0")
    r = subprocess.run([exe, fin, fout, kind, str(misalign)] + (["pipe"] if pipe else []), env=env,
                       capture_output=True, text=True)
    assert r.returncode == 0, (r.returncode, r.stderr[-2000:])
    raw = open(fout, "rb").read()
    dt = np.float32 if kind == "f32" else np.float64
    isz = dt().itemsize
    out, pos = {"dvo": dvo}, 0
    for name, shape in (("vo", (B, T, H, Wv)), ("lse", (B, T, H)), ("threads", None), ("dA", (B, T, T, H)),
                        ("dv", (B, T, H, Wv)), ("bwd_threads", None)):
        if shape is None:
            out[name] = struct.unpack_from("q", raw, pos)[0]
            pos += 8
        else:
            n = int(np.prod(shape))
            out[name] = torch.from_numpy(np.frombuffer(raw, dt, n, pos).copy()).view(*shape)
            pos += n * isz
    assert pos == len(raw)
    return out


def _ref(q, k, v):
    q, k, v = q.double(), k.double(), v.double()
    if q.shape[3] == v.shape[3]:
        return oracle.fused_fwd(q, k, v)
    return cf.dense_then_value(q, k, v, noop=True), (1.0 + cf.dense_attn(q, k).exp().sum(1)).log()


def _check_backward(r, q, k, v, tol):
    """dA against torch autograd through the closed form (gradient of vo.dvo with respect to the logits), dv
    against autograd, and dq, dk = the oracle's dense backward of the emulated dA against autograd."""
    q, k, v, dvo = (x.double() for x in (q, k, v, r["dvo"]))
    a = cf.dense_attn(q, k).requires_grad_()
    vd = v.clone().requires_grad_()
    e = a.exp()
    vo = torch.einsum("bsdh,bshw->bdhw", e / (1.0 + e.sum(1, keepdim=True)), vd)
    dA_ref, dv_ref = torch.autograd.grad(vo, (a, vd), dvo)
    assert cf.rel_err(r["dA"], dA_ref) <= tol and cf.rel_err(r["dv"], dv_ref) <= tol
    qd, kd = q.clone().requires_grad_(), k.clone().requires_grad_()
    dq_ref, dk_ref = torch.autograd.grad(cf.dense_then_value(qd, kd, v, noop=True), (qd, kd), dvo)
    dq, dk = oracle.dense_bwd(r["dA"].double(), q, k)
    assert cf.rel_err(dq, dq_ref) <= tol and cf.rel_err(dk, dk_ref) <= tol
    if q.shape[3] == v.shape[3]:  # and the oracle's own backward agrees with autograd
        odq, odk, odv = oracle.fused_bwd(dvo, q, k, v)
        assert cf.rel_err(odq, dq_ref) <= 1e-11 and cf.rel_err(odk, dk_ref) <= 1e-11 and cf.rel_err(odv, dv_ref) <= 1e-11


TILED = [
    # B, T, H, W: shapes the f32 entry point gives to the tiled kernel
    (2, 64, 4, 32),    # first baseline configuration
    (1, 100, 3, 64),   # ragged last dst tile, fewer heads than a workgroup holds
    (2, 70, 6, 16),    # ragged head group (4 + 2)
    (3, 33, 9, 16),    # 27 workgroups: the XCD permutation leaves a remainder of three; dA kernel: 8 + 1 heads
    (1, 75, 16, 32),   # dA kernel: two full groups of eight heads; 75 = 9 flushes of 8 src rows + 3
    (1, 40, 2, 48), (1, 36, 5, 96),  # the other two tiled widths
]


@pytest.mark.parametrize("shape", TILED)
def test_fused_tiled_kernels_on_cpu(runner, tmp_path, shape):
    B, T, H, W = shape
    g = torch.Generator().manual_seed(sum(shape))
    q, k, v = (torch.randn(B, T, H, W, generator=g) for _ in range(3))
    r = _run(runner, tmp_path, q, k, v)
    NH, NHa = min(H, 4), min(H, 8)  # heads per workgroup: forward and dv kernels, dA kernel
    launch = -(-T // 64) * B * -(-H // NH) * 64 * NH  # a tiled kernel's launch, not a generic one's
    launch_a = -(-T // 64) * B * -(-H // NHa) * 64 * NHa
    assert r["threads"] == launch and r["bwd_threads"] == launch + launch_a
    ref, ref_lse = _ref(q, k, v)
    assert cf.rel_err(r["vo"], ref) <= 1e-5 and cf.rel_err(r["lse"], ref_lse) <= 1e-5
    _check_backward(r, q, k, v, 1e-4)


@pytest.mark.parametrize("shape", [(2, 64, 4, 32), (1, 100, 3, 64), (2, 70, 6, 32), (1, 33, 9, 64), (1, 1000, 1, 32)])
def test_fused_pipelined_forward_on_cpu(runner, tmp_path, shape):
    """The software-pipelined forward (l1attn_fused_fwd_pipe_f32) and, in the same run, the pipelined first stage of
    the backward (l1attn_fused_bwd_stage_pipe_f32: dA and dv).  The host stand-in for the scalar prefetch
    delivers a chunk's data at the wait and poisons the buffer at the load, so reading a buffer before its wait, a
    chunk taken from the wrong buffer, a wrong chunk address or a missing final drain all fail here.  Same arithmetic
    in the same order as the plain tiled kernel: equal bit for bit."""
    B, T, H, W = shape
    g = torch.Generator().manual_seed(sum(shape))
    q, k, v = (torch.randn(B, T, H, W, generator=g) for _ in range(3))
    plain = _run(runner, tmp_path, q, k, v)
    piped = _run(runner, tmp_path, q, k, v, pipe=True)
    NH = min(H, 4)
    assert piped["threads"] == -(-T // 64) * B * -(-H // NH) * 64 * NH
    assert torch.equal(piped["vo"], plain["vo"]) and torch.equal(piped["lse"], plain["lse"])
    assert torch.equal(piped["dA"], plain["dA"]) and torch.equal(piped["dv"], plain["dv"])
    NHa = min(H, 8)  # the dA kernel takes up to eight heads per workgroup
    assert piped["bwd_threads"] == plain["bwd_threads"] == -(-T // 64) * B * (-(-H // NHa) * 64 * NHa + -(-H // NH) * 64 * NH)
    ref, ref_lse = _ref(q, k, v)
    assert cf.rel_err(piped["vo"], ref) <= 1e-5 and cf.rel_err(piped["lse"], ref_lse) <= 1e-5
    _check_backward(piped, q, k, v, 1e-4)
    # widths without a pipelined kernel run what the plain entry runs
    if shape == (2, 64, 4, 32):
        q16, k16, v16 = q[..., :16].contiguous(), k[..., :16].contiguous(), v[..., :16].contiguous()
        assert torch.equal(_run(runner, tmp_path, q16, k16, v16, pipe=True)["vo"], _run(runner, tmp_path, q16, k16, v16)["vo"])


GENERIC = [
    # B, T, H, W, Wv
    (2, 3, 16, 7, 7), (1, 40, 2, 80, 80), (1, 37, 3, 32, 20), (1, 31, 2, 64, 64), (1, 1, 1, 1, 1),
]


@pytest.mark.parametrize("shape", GENERIC)
def test_fused_generic_kernels_on_cpu(runner, tmp_path, shape):
    B, T, H, W, Wv = shape
    g = torch.Generator().manual_seed(sum(shape))
    q, k = (torch.randn(B, T, H, W, generator=g) for _ in range(2))
    v = torch.randn(B, T, H, Wv, generator=g)
    ref, ref_lse = _ref(q, k, v)
    r = _run(runner, tmp_path, q, k, v)
    up = lambda n: -(-n // 256) * 256
    assert r["threads"] == up(B * T * H * Wv) and r["bwd_threads"] == up(B * T * T * H) + up(B * T * H * Wv)
    assert cf.rel_err(r["vo"], ref) <= 1e-5 and cf.rel_err(r["lse"], ref_lse) <= 1e-5
    _check_backward(r, q, k, v, 1e-4)
    r = _run(runner, tmp_path, q.double(), k.double(), v.double())
    assert cf.rel_err(r["vo"], ref) <= 1e-12 and cf.rel_err(r["lse"], ref_lse) <= 1e-12
    _check_backward(r, q, k, v, 1e-11)


def test_fused_unaligned_buffers_take_the_generic_kernels(runner, tmp_path):
    B, T, H, W = 1, 64, 2, 32
    g = torch.Generator().manual_seed(5)
    q, k, v = (torch.randn(B, T, H, W, generator=g) for _ in range(3))
    r = _run(runner, tmp_path, q, k, v, misalign=1)
    assert r["threads"] == B * T * H * W  # one thread per output element
    ref, ref_lse = _ref(q, k, v)
    assert cf.rel_err(r["vo"], ref) <= 1e-5 and cf.rel_err(r["lse"], ref_lse) <= 1e-5
    _check_backward(r, q, k, v, 1e-4)


def test_fused_kernels_have_no_data_race_between_barriers(runner_tsan, tmp_path):
    """The same run under ThreadSanitizer (GPU threads are OS threads, __syncthreads() a barrier): the LDS tile of
    the dA kernel is written and read by different threads, so a missing or misplaced barrier is a reported data
    race and a non-zero exit (checked once by removing the barrier after the flush).  Ragged tile, 8 + 1 heads."""
    B, T, H, W = 1, 75, 9, 16
    g = torch.Generator().manual_seed(1)
    q, k, v = (torch.randn(B, T, H, W, generator=g) for _ in range(3))
    r = _run(runner_tsan, tmp_path, q, k, v)
    _check_backward(r, q, k, v, 1e-4)
    # the pipelined dA kernel keeps a scalar prefetch in flight across the flush and its two barriers
    q, k, v = (torch.randn(1, 70, 9, 32, generator=g) for _ in range(3))
    _check_backward(_run(runner_tsan, tmp_path, q, k, v, pipe=True), q, k, v, 1e-4)


def test_fixed_point_prepass_kernels_on_cpu(tmp_path):
    """The grid and conversion kernels of the experimental fixed-point forward (csrc/fixed.hip; one with an LDS
    reduction) under AddressSanitizer: grids equal max(|q|,|k|) * 2^-24 per (batch, head) bit for bit, the
    converted values equal rint(x / grid) with the sign bit flipped, bit for bit, and decode to within three quarters of a
    grid step of the input; an all-zero head and a head 1000 times larger than the others."""
    exe = str(tmp_path / "run_fixed")
    subprocess.run(["g++", "-std=c++20", "-O1", "-g", "-pthread", "-fsanitize=address,undefined",
                    "-fno-sanitize-recover=all", "-I", EMU, "-x", "c++", os.path.join(EMU, "run_fixed.cpp"), "-o", exe],
                   check=True)
    B, T, H, W = 2, 37, 3, 32
    g = torch.Generator().manual_seed(11)
    q, k = (torch.randn(B, T, H, W, generator=g) for _ in range(2))
    q[:, :, 1] *= 1000.0
    q[1, :, 2] = 0
    k[1, :, 2] = 0
    fin, fout = str(tmp_path / "in.bin"), str(tmp_path / "out.bin")
    with open(fin, "wb") as f:
        f.write(struct.pack("4q", B, T, H, W))
        f.write(q.numpy().tobytes())
        f.write(k.numpy().tobytes())
    env = dict(os.environ, ASAN_OPTIONS="verify_asan_link_order=0:detect_leaks=0")
    r = subprocess.run([exe, fin, fout], env=env, capture_output=True, text=True)
    assert r.returncode == 0, (r.returncode, r.stderr[-2000:])
    raw = open(fout, "rb").read()
    n = B * T * H * W
    gq = np.frombuffer(raw, np.float32, B * H).reshape(B, H)
    uq = np.frombuffer(raw, np.uint32, n, B * H * 4).reshape(B, T, H, W)
    uk = np.frombuffer(raw, np.uint32, n, B * H * 4 + n * 4).reshape(B, T, H, W)
    qn, kn = q.numpy(), k.numpy()
    m = np.maximum(np.abs(qn).max(axis=(1, 3)), np.abs(kn).max(axis=(1, 3)))            # [B,H]
    g_ref = np.maximum(m * np.float32(2.0 ** -24), np.float32(1.17549435e-38)).astype(np.float32)
    assert np.array_equal(gq, g_ref)
    for x, u in ((qn, uq), (kn, uk)):
        i_ref = np.rint((x / g_ref[:, None, :, None]).astype(np.float32)).astype(np.int64)
        assert np.abs(i_ref).max() <= 2 ** 24
        assert np.array_equal(u, ((i_ref + 2 ** 31) % 2 ** 32).astype(np.uint32))
        decoded = (u.astype(np.int64) - 2 ** 31) * g_ref[:, None, :, None].astype(np.float64)
        # half a step from rint, up to a quarter more from the fp32 rounding of the quotient below 2^23
        assert np.all(np.abs(decoded - x) <= 0.7500001 * g_ref[:, None, :, None])
    assert np.all(uq[1, :, 2] == 2 ** 31) and np.all(uk[1, :, 2] == 2 ** 31)


@pytest.fixture(scope="module", params=["merge", "library"])
def ranks_runner(request):
    """The rank kernel written for this library (csrc/rank_sort.hip), and the one the backward uses by default
    (csrc/dense_rank.hip) with a host stand-in for the library block sort it calls: same ranks by definition."""
    return request.getfixturevalue("emu_ranks" if request.param == "merge" else "emu_ranks_lib")


def _reference_ranks(q, k):
    """rq, rk of one [B,T,H,W] pair by their definition, with numpy: per column, rk = 2 * #{k' < k} - 1/2 and
    rq = 2 * #{k' < q}, minus one where q ties with no k.  -0 and +0 are equal."""
    qn, kn = q.numpy().astype(np.float64) + 0.0, k.numpy().astype(np.float64) + 0.0
    B, T, H, W = qn.shape
    rq, rk = np.empty_like(qn), np.empty_like(kn)
    for b in range(B):
        for h in range(H):
            for w in range(W):
                ks = np.sort(kn[b, :, h, w])
                less_k = np.searchsorted(ks, kn[b, :, h, w], side="left")
                rk[b, :, h, w] = 2 * less_k - 0.5
                less_q = np.searchsorted(ks, qn[b, :, h, w], side="left")
                tie = np.searchsorted(ks, qn[b, :, h, w], side="right") > less_q
                rq[b, :, h, w] = 2 * less_q - np.where(tie, 0, 1)
    return rq, rk


@pytest.mark.parametrize("shape", [(1, 4096, 1, 2), (1, 1000, 2, 2), (2, 300, 1, 3), (1, 2049, 1, 2), (1, 5000, 1, 1),
                                   (1, 1, 1, 5), (1, 513, 3, 1)])
def test_column_rank_kernels_on_cpu(tmp_path, shape, ranks_runner):
    """Both column-rank kernels (csrc/rank_sort.hip: registers, LDS and barriers only; csrc/dense_rank.hip around
    a stand-in for the library sort) under AddressSanitizer:
    every items-per-thread instantiation (T up to 512, 1024, 2048, 4096, 8192), ragged lengths (padding keys),
    planted ties between q and k, repeated k values, both zeros; ranks equal their definition exactly, and
    clamp(rq - rk, 0, 1) is 1, 1/2, 0 for q >, ==, < k on every pair of a column."""
    exe = ranks_runner
    B, T, H, W = shape
    g = torch.Generator().manual_seed(sum(shape))
    q, k = (torch.randn(B, T, H, W, generator=g) for _ in range(2))
    if T > 8:
        idx = torch.randperm(T, generator=g)[: T // 8]
        q[:, idx] = k[:, idx.flip(0)]                    # ties between q and k
        k[:, : T // 16] = k[:, T // 16: 2 * (T // 16)]   # repeated k values
        q[0, 0, 0, 0], k[0, 1, 0, 0] = 0.0, -0.0
    if W > 1:
        q[..., 1] = torch.round(q[..., 1])               # a column on a coarse grid: long runs of equal keys
        k[..., 1] = torch.round(k[..., 1])
    fin, fout = str(tmp_path / "in.bin"), str(tmp_path / "out.bin")
    with open(fin, "wb") as f:
        f.write(struct.pack("4q", B, T, H, W))
        f.write(q.numpy().tobytes())
        f.write(k.numpy().tobytes())
    env = dict(os.environ, ASAN_OPTIONS="verify_asan_link_order=0:detect_leaks=0")
    r = subprocess.run([exe, fin, fout], env=env, capture_output=True, text=True)
    assert r.returncode == 0, (r.returncode, r.stderr[-2000:])
    raw = open(fout, "rb").read()
    n = B * T * H * W
    rq = np.frombuffer(raw, np.float32, n).reshape(B, T, H, W)
    rk = np.frombuffer(raw, np.float32, n, n * 4).reshape(B, T, H, W)
    ref_rq, ref_rk = _reference_ranks(q, k)
    assert np.array_equal(rq, ref_rq) and np.array_equal(rk, ref_rk)
    if T <= 1000:  # all pairs of every column
        hv = np.clip(rq[:, :, None] - rk[:, None], 0.0, 1.0)             # [B,T(dst),S(src),H,W]
        sign = np.sign((q.numpy()[:, :, None] + 0.0) - (k.numpy()[:, None] + 0.0))
        assert np.array_equal(2 * hv - 1, sign)


@pytest.mark.parametrize("shape,kernel", [((1, 1000, 1, 2), "merge"), ((1, 2049, 1, 1), "merge"),
                                          ((2, 700, 1, 3), "library")])
def test_column_rank_kernels_have_no_data_race(tmp_path, shape, kernel, request):
    """The merge rounds work in place in LDS: every thread reads its inputs, a barrier, every thread writes its
    outputs, a barrier.  Under ThreadSanitizer a thread that wrote before another had read would be a data race.
    The default kernel hands its sorted keys to every thread's searches through LDS behind one barrier."""
    emu_ranks_tsan = request.getfixturevalue("emu_ranks_tsan" if kernel == "merge" else "emu_ranks_lib_tsan")
    B, T, H, W = shape
    g = torch.Generator().manual_seed(sum(shape))
    q, k = (torch.randn(B, T, H, W, generator=g) for _ in range(2))
    fin, fout = str(tmp_path / "in.bin"), str(tmp_path / "out.bin")
    with open(fin, "wb") as f:
        f.write(struct.pack("4q", B, T, H, W))
        f.write(q.numpy().tobytes())
        f.write(k.numpy().tobytes())
    env = dict(os.environ, TSAN_OPTIONS="halt_on_error=1 report_signal_unsafe=0")
    r = subprocess.run([emu_ranks_tsan, fin, fout], env=env, capture_output=True, text=True)
    assert r.returncode == 0, (r.returncode, r.stderr[:3000])
    n = B * T * H * W
    raw = open(fout, "rb").read()
    ref_rq, ref_rk = _reference_ranks(q, k)
    assert np.array_equal(np.frombuffer(raw, np.float32, n).reshape(B, T, H, W), ref_rq)
    assert np.array_equal(np.frombuffer(raw, np.float32, n, n * 4).reshape(B, T, H, W), ref_rk)
