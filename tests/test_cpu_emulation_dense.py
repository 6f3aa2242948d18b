"""CPU-only: the dense operator's kernel source (csrc/dense.hip: forward, backward, fixed-point forward) compiled
for the host and run through the library's own entry points, against the oracle.

tests/cpu_emu/run_dense.cpp includes the kernel file as it is.  GPU threads are OS threads, the LDS barrier is a
barrier among them, DPP row shifts and raw buffer accesses are host functions, and the two headers that hold the
library's hand-written instructions (csrc/sload.h, csrc/gfx950.h) are replaced by stand-ins that compute what those
instructions compute (the scalar prefetch delivers at its wait and poisons at its load).  Everything else -- the
host logic that picks kernels, grids, tile plans and workspace, every index, clamp, predicate and LDS offset of the
kernels -- is the product's.  Buffers and the launch's LDS have their exact sizes under AddressSanitizer, outputs
start as NaN (an element never written fails the comparison), and one build runs under ThreadSanitizer (a missing
barrier is a data race).  This says nothing about timing, register allocation or the instruction encodings.

The 512-thread tile kernels are chosen by the library from 1024 tokens and a few thousand workgroups on; the runner
can build their plan for any length ("wide"), which is how they are walked here at 100 to 260 tokens."""
import os
import re
import struct
import subprocess

import numpy as np
import pytest
import torch

import closed_forms as cf
from oracle import oracle

HERE = os.path.dirname(os.path.abspath(__file__))
EMU = os.path.join(HERE, "cpu_emu")
ENV = dict(os.environ, ASAN_OPTIONS="verify_asan_link_order=0:detect_leaks=0",
           TSAN_OPTIONS="halt_on_error=1 report_signal_unsafe=0")


def _run(exe, d, shape, mode="f32", extra=(), seed=0, ties=False, scale=1.0, inputs=None):
    """-> dict with attn, dq, dk (as far as the mode has them), plan, and the inputs (seeded, or `inputs` = q, k, dA)."""
    B, T, H, W = shape
    dt = torch.float64 if mode == "f64" else torch.float32
    g = torch.Generator().manual_seed(seed)
    q, k = (torch.randn(B, T, H, W, generator=g, dtype=dt) * scale for _ in range(2))
    if ties:  # half-integers: exact ties between q and k, and among the k of a column
        q, k = torch.round(q * 2) / 2, torch.round(k * 2) / 2
    dA = torch.randn(B, T, T, H, generator=g, dtype=dt)
    if inputs is not None:
        q, k, dA = (x.to(dt).contiguous() for x in inputs)
    fin, fout = str(d / "in.bin"), str(d / "out.bin")
    with open(fin, "wb") as f:
        f.write(struct.pack("4q", B, T, H, W))
        for x in (q, k, dA):
            f.write(x.numpy().tobytes())
    r = subprocess.run([exe, fin, fout, mode] + [str(x) for x in extra], env=ENV, capture_output=True, text=True)
    assert r.returncode == 0, (shape, mode, extra, r.returncode, r.stderr[-3000:])
    raw = open(fout, "rb").read()
    npdt = np.float64 if mode == "f64" else np.float32
    it, na, n = np.dtype(npdt).itemsize, B * T * T * H, B * T * H * W
    out = {"q": q, "k": k, "dA": dA, "attn": torch.from_numpy(np.frombuffer(raw, npdt, na).reshape(B, T, T, H).copy())}
    off = na * it
    if mode != "fixed":
        out["dq"] = torch.from_numpy(np.frombuffer(raw, npdt, n, off).reshape(B, T, H, W).copy())
        out["dk"] = torch.from_numpy(np.frombuffer(raw, npdt, n, off + n * it).reshape(B, T, H, W).copy())
        off += 2 * n * it
    assert len(raw) == off + 17 * 8
    out["domain_flag"] = int(np.frombuffer(raw, np.int64, 1, off + 16 * 8)[0])
    keys = ("tiled", "wide", "rank", "branch_free", "threads", "n_cc", "n_tt", "tt_rows", "per", "group", "n_groups")
    out["plan"] = dict(zip(keys, np.frombuffer(raw, np.int64, 16, off).tolist()))
    return out


def _check(r, fwd_tol, bwd_tol):
    q, k, dA = (r[n].double() for n in ("q", "k", "dA"))
    assert cf.rel_err(r["attn"], oracle.dense_fwd(q, k)) <= fwd_tol      # (NaN, i.e. an unwritten element, fails too)
    if "dq" in r:
        rdq, rdk = oracle.dense_bwd(dA, q, k)
        assert cf.rel_err(r["dq"], rdq) <= bwd_tol and cf.rel_err(r["dk"], rdk) <= bwd_tol


@pytest.fixture(scope="module")
def runner(emu_dense):
    return emu_dense


# shape, and what it is there for
LIBRARY_CASES = [
    ((2, 64, 4, 32), "first baseline configuration: pipelined forward 32, 32-token tiles"),
    ((1, 3, 2, 7), "the reference's test shape: one-workgroup forward, untiled backward"),
    ((2, 17, 3, 5), "short odd sequence, H*W < 32"),
    ((1, 70, 2, 9), "no multiple of anything: grid-stride forward, untiled backward"),
    ((1, 40, 2, 7), "width 7 on zero-padded rows of 16"),
    ((2, 100, 3, 33), "width 33 on padded rows of 48, ragged last tile, heads straddling column chunks"),
    ((1, 50, 2, 65), "width 65 on padded rows of 80"),
    ((1, 40, 1, 100), "width 100 on padded rows of 128 (half-head kernel)"),
    ((1, 70, 20, 16), "twenty heads: two head groups in the forward, eight staged values per thread"),
    ((1, 40, 16, 8), "sixteen staged values per thread"),
    ((1, 64, 4, 48), "forward 48"),
    ((1, 96, 2, 80), "forward 80"),
    ((1, 64, 3, 96), "pipelined forward 96"),
    ((1, 64, 2, 112), "forward 112"),
    ((1, 64, 2, 128), "width 128 as two half-heads of the pipelined forward 64"),
    ((2, 33, 1, 320), "width beyond the tiled forward"),
    ((1, 72, 16, 64), "headline head geometry: sixteen waves per forward workgroup, two column chunks"),
    ((1, 264, 2, 64), "several src chunks per dst tile in the forward"),
]


@pytest.mark.parametrize("shape,why", LIBRARY_CASES, ids=[str(c[0]) for c in LIBRARY_CASES])
def test_dense_kernels_as_the_library_picks_them(runner, tmp_path, shape, why):
    _check(_run(runner, tmp_path, shape, seed=sum(shape)), 1e-5, 1e-4)


def test_the_cases_reach_the_kernel_families(runner, tmp_path):
    """The plans of the shapes above, so that a change of the host logic that moves a case to another kernel
    (and silently thins this file's coverage) is noticed."""
    tiled = {s: _run(runner, tmp_path, s)["plan"] for s in [(2, 64, 4, 32), (1, 70, 20, 16), (1, 40, 16, 8), (1, 3, 2, 7)]}
    assert [tiled[s]["tiled"] for s in tiled] == [1, 1, 1, 0]
    assert [tiled[s]["per"] for s in list(tiled)[:3]] == [4, 8, 16] and tiled[(2, 64, 4, 32)]["tt_rows"] == 32


def test_dense_float64_and_ties(runner, tmp_path):
    for shape in ((2, 20, 3, 5), (1, 70, 2, 9)):
        _check(_run(runner, tmp_path, shape, mode="f64", seed=4), 1e-13, 1e-13)
    r = _run(runner, tmp_path, (2, 64, 4, 32), ties=True, seed=9)
    assert float((r["q"][:, :, None] == r["k"][:, None]).float().mean()) > 0.1  # sign(0) = 0 matters here
    _check(r, 1e-6, 1e-5)
    _check(_run(runner, tmp_path, (1, 33, 2, 7), ties=True, seed=9), 1e-6, 1e-5)  # untiled kernels, exact compares


def test_sign_domain_guard_of_the_tiled_backward(runner, tmp_path):
    """The tiled float32 backward without column ranks takes sign(q - k) from the difference of q * 2^64 and
    k * 2^64, which is exact while every magnitude is below 2^63 and every non-zero one at least 2^-41.  A pre-pass
    raises a flag in the workspace otherwise and a fix-up kernel redoes dq and dk with comparisons, so the result is
    the reference's sign() (cpp/l1attn_drv.cpp:7-11) for every input: tiny values whose differences the scaling
    would leave fractional, magnitudes it would overflow, infinities.  Inside the range the flag stays clear and
    the fix-up kernel leaves the tiled result alone."""
    shape = (2, 64, 4, 32)                                                    # 32-token tiles, two per sequence
    g = torch.Generator().manual_seed(31)
    q0, k0 = (torch.randn(*shape, generator=g) for _ in range(2))
    k0[0, 1] = q0[0, 2]                                                       # exact ties stay exact under powers of two
    dA = torch.randn(2, 64, 64, 4, generator=g)
    for e, flagged in ((0, 0), (-20, 0), (40, 0), (-36, 1), (-70, 1), (64, 1)):   # (2^-36: some values below 2^-41)
        r = _run(runner, tmp_path, shape, inputs=(q0 * 2.0 ** e, k0 * 2.0 ** e, dA))
        assert r["plan"]["tiled"] == 1 and r["plan"]["rank"] == 0 and r["domain_flag"] == flagged, e
        rdq, rdk = oracle.dense_bwd(dA.double(), r["q"].double(), r["k"].double())
        assert cf.rel_err(r["dq"], rdq) <= 1e-4 and cf.rel_err(r["dk"], rdk) <= 1e-4, e
    # one value outside the range is enough: a subnormal, a value of 2^63, an infinity in k
    for where, value in (((1, 63, 3, 31), 1e-40), ((0, 0, 0, 0), 2.0 ** 63), ((1, 5, 2, 7), float("inf"))):
        q, k = q0.clone(), k0.clone()
        (q if value != float("inf") else k)[where] = value
        r = _run(runner, tmp_path, shape, inputs=(q, k, dA))
        assert r["domain_flag"] == 1
        rdq, rdk = oracle.dense_bwd(dA.double(), q.double(), k.double())
        assert cf.rel_err(r["dq"], rdq) <= 1e-4 and cf.rel_err(r["dk"], rdk) <= 1e-4, value
    # exact zeros are inside the range (|0 - x| is a whole multiple of 2^-64 whenever x is)
    q = q0.clone()
    q[:, ::3] = 0.0
    assert _run(runner, tmp_path, shape, inputs=(q, k0, dA))["domain_flag"] == 0
    # a caller that vouches for the range skips check and fix-up: same result inside the range (the flag word is
    # never written), the stated formula -- not the sign -- outside it
    inside = _run(runner, tmp_path, shape, inputs=(q0, k0, dA))
    vouched = _run(runner, tmp_path, shape, inputs=(q0, k0, dA), extra=("assume",))
    assert vouched["domain_flag"] == int.from_bytes(b"\xa5" * 4, "little", signed=True)
    assert torch.equal(vouched["dq"], inside["dq"]) and torch.equal(vouched["dk"], inside["dk"])
    tiny = _run(runner, tmp_path, shape, inputs=(q0 * 2.0 ** -70, k0 * 2.0 ** -70, dA), extra=("assume",))
    s = ((tiny["q"].double() * 2.0 ** 64)[:, None] - (tiny["k"].double() * 2.0 ** 64)[:, :, None]).float().double().clamp(-1, 1)
    sc = -1.0 / 32 ** 0.5
    assert cf.rel_err(tiny["dq"], sc * torch.einsum("bsthw,bsth->bthw", s, dA.double())) <= 1e-4
    assert cf.rel_err(tiny["dk"], -sc * torch.einsum("bsthw,bsth->bshw", s, dA.double())) <= 1e-4
    rdq, _ = oracle.dense_bwd(dA.double(), tiny["q"].double(), tiny["k"].double())
    assert cf.rel_err(tiny["dq"], rdq) > 0.5
    # plans that keep no flag: the untiled kernels compare exactly whatever the range
    r = _run(runner, tmp_path, (1, 12, 2, 7), scale=2.0 ** -70, seed=3)
    assert r["plan"]["tiled"] == 0 and r["domain_flag"] == -1
    _check(r, 1e-5, 1e-4)


def test_dense_kernels_against_the_reference_extension_golden_vectors(runner, tmp_path):
    """tests/golden/ref_cpp_golden.npz holds inputs and outputs of the reference's own compiled CPU extension
    (cpp/l1attn_drv.cpp; written by tests/golden/make_golden.py), with exact ties planted.  The float64 kernels sum
    in the reference's order: equal to the last bit.  The float32 kernels on the same inputs: the usual tolerances."""
    z = np.load(os.path.join(HERE, "golden", "ref_cpp_golden.npz"))
    for tag in ("dA", "dB"):
        q, k, da = (torch.from_numpy(z["%s_%s" % (tag, n)]) for n in ("q", "k", "da"))
        want = [torch.from_numpy(z["%s_%s" % (tag, n)]) for n in ("attn", "dq", "dk")]
        r = _run(runner, tmp_path, tuple(q.shape), mode="f64", inputs=(q, k, da))
        for name, w in zip(("attn", "dq", "dk"), want):
            assert torch.equal(r[name], w), (tag, name)
        r = _run(runner, tmp_path, tuple(q.shape), mode="f32", inputs=(q, k, da))
        f32_in = [x.float().double() for x in (q, k)]  # what the float32 kernels were given
        assert cf.rel_err(r["attn"], oracle.dense_fwd(*f32_in)) <= 1e-5
        assert cf.rel_err(r["attn"], want[0]) <= 1e-5 and cf.rel_err(r["dk"], want[2]) <= 1e-4
        # (dq, dk of float32-rounded inputs may differ from the float64 golden where a tie is broken by the rounding)
        rdq, rdk = oracle.dense_bwd(da.float().double(), *f32_in)
        assert cf.rel_err(r["dq"], rdq) <= 1e-4 and cf.rel_err(r["dk"], rdk) <= 1e-4


WIDE_CASES = [
    # shape, tile height, rank form, tiles per workgroup, half-integer inputs
    ((2, 128, 2, 64), 64, 0, 1, False),     # branch-free step loop, one tile per workgroup
    ((2, 128, 2, 64), 64, 1, 1, True),      # ... on column ranks
    ((3, 128, 8, 64), 64, 0, 2, True),      # grouped tiles: the later tile adds to the stored partial; batch loop
    ((3, 128, 2, 64), 64, 1, 2, False),
    ((1, 256, 4, 64), 64, 1, 4, False),     # the headline instantiation <64,512,4,rank,grouped,branch-free>
    ((1, 100, 3, 33), 64, 0, 1, False),     # general form: ragged tile, idle lanes shadowing a column
    ((1, 136, 4, 64), 64, 1, 1, True),      # general form on ranks: T not a multiple of 64
    ((1, 140, 16, 32), 64, 0, 1, False),    # eight staged values per thread
    ((1, 100, 8, 64), 72, 1, 1, True),
    ((1, 150, 8, 64), 80, 1, 1, False),
    ((1, 150, 8, 64), 88, 0, 1, False),
    ((1, 90, 16, 64), 72, 0, 1, False),     # two column chunks
    ((1, 100, 5, 96), 64, 1, 1, False),     # heads of 96 columns: a chunk of 480 columns touches five heads
]


@pytest.mark.parametrize("shape,tt,rank,group,ties", WIDE_CASES, ids=["%s-tt%d-r%d-g%d" % (c[0], c[1], c[2], c[3]) for c in WIDE_CASES])
def test_dense_backward_wide_tile_kernels(runner, tmp_path, shape, tt, rank, group, ties):
    # (the rank form sums 2*hv*g and subtracts the row and column sums of g: a few more roundings than the oracle's sum)
    _check(_run(runner, tmp_path, shape, extra=("wide", tt, rank, group), seed=sum(shape) + tt, ties=ties), 1e-5, 1e-4)


_ONE_STEP = {}  # results of the one-step loop, shared by the two forms compared with it


@pytest.mark.parametrize("form", ["deep", "deep2"])
@pytest.mark.parametrize("shape,rank,group", [((3, 128, 2, 64), 0, 2), ((1, 256, 2, 64), 1, 4), ((1, 64, 1, 64), 1, 1)])
def test_pipelined_step_loops_equal_the_one_step_loop(runner, tmp_path, shape, rank, group, form):
    """dense_bwd_f32_fast<..., DEEP>.  "deep": two register sets of prefetched values alternate and the step loop
    runs two steps per iteration.  "deep2": the two steps also stage their tiles in two LDS planes and keep one
    barrier each.  Same sums in the same order: dq and dk equal the one-step loop's bit for bit (and the oracle's
    within the usual tolerance), also at the shortest sequence (64 tokens = sixteen steps), over several tiles per
    workgroup (where the rank form's row sums of one tile are read from the plane the next tile writes first) and
    with half-integer inputs (ties)."""
    deep = _run(runner, tmp_path, shape, extra=("wide", 64, rank, group, form), seed=5, ties=bool(rank))
    _check(deep, 1e-5, 1e-4)
    key = (shape, rank, group)
    if key not in _ONE_STEP:
        _ONE_STEP[key] = _run(runner, tmp_path, shape, extra=("wide", 64, rank, group), seed=5, ties=bool(rank))
    one = _ONE_STEP[key]
    assert torch.equal(deep["dq"], one["dq"]) and torch.equal(deep["dk"], one["dk"])


def test_all_tie_column_in_the_rank_form(runner, tmp_path):
    """A column in which every q equals every k has sign(q - k) = 0 throughout: the reference's gradients there are
    exactly zero (cpp/l1attn_drv.cpp:7-11).  The sign form reproduces the zeros; the rank form computes
    2 * sum(hv * g) - sum(g) with hv = 1/2, which leaves the rounding residue of the two sums.  This pins the size
    of that residue: below 1e-5 of the largest gradient, the forward tolerance."""
    B, T, H, W = 1, 128, 2, 64
    g = torch.Generator().manual_seed(31)
    q, k = torch.randn(B, T, H, W, generator=g), torch.randn(B, T, H, W, generator=g)
    q[..., 5] = k[..., 5] = 0.75
    dA = torch.randn(B, T, T, H, generator=g)
    fin, fout = str(tmp_path / "in.bin"), str(tmp_path / "out.bin")
    res = {}
    for rank in (0, 1):
        with open(fin, "wb") as f:
            f.write(struct.pack("4q", B, T, H, W))
            for x in (q, k, dA):
                f.write(x.numpy().tobytes())
        r = subprocess.run([runner, fin, fout, "f32", "wide", "64", str(rank), "1"], env=ENV, capture_output=True, text=True)
        assert r.returncode == 0, r.stderr[-2000:]
        raw = np.fromfile(fout, np.float32, count=B * T * T * H + 2 * B * T * H * W)[B * T * T * H:]
        res[rank] = torch.from_numpy(raw.copy()).view(2, B, T, H, W)
    rdq, rdk = oracle.dense_bwd(dA.double(), q.double(), k.double())
    assert float(rdq[..., 5].abs().max()) == 0.0 and float(rdk[..., 5].abs().max()) == 0.0
    assert float(res[0][..., 5].abs().max()) == 0.0                                  # sign form: exact zeros
    big = float(max(rdq.abs().max(), rdk.abs().max()))
    assert 0.0 < float(res[1][..., 5].abs().max()) <= 1e-5 * big                      # rank form: a residue, this small
    assert cf.rel_err(res[1][0], rdq) <= 1e-4 and cf.rel_err(res[1][1], rdk) <= 1e-4


def test_plans_outside_the_kernels_limits_are_refused(runner, tmp_path):
    """The runner's plan builder mirrors the library's limits: sixteen lanes per staged (src row, head) in the rank
    form, at most eight staged values per thread."""
    for shape, extra in (((1, 100, 3, 33), ("wide", 72, 1, 1)), ((1, 150, 4, 32), ("wide", 88, 0, 1))):
        with pytest.raises(AssertionError, match=r"wide.*, 4, "):
            _run(runner, tmp_path, shape, extra=extra)
    with pytest.raises(AssertionError, match=r"deep.*, 4, "):  # two-step prefetch exists in the branch-free form only
        _run(runner, tmp_path, (1, 100, 2, 64), extra=("wide", 64, 0, 1, "deep"))


@pytest.mark.parametrize("shape", [(1, 64, 4, 32), (1, 100, 3, 64), (2, 40, 2, 64)])
def test_fixed_point_forward_kernel(runner, tmp_path, shape):
    """dense_fwd_f32_pipe<W, true> behind both pre-passes: the 24-bit grid per (batch, head) keeps the logits
    within 1e-5 of the float64 oracle on N(0,1) inputs."""
    _check(_run(runner, tmp_path, shape, mode="fixed", seed=sum(shape)), 1e-5, None)


def test_dense_kernels_under_thread_sanitizer(tmp_path, emu_dense_tsan):
    """A barrier missing between a step's LDS writes and reads, or between two steps, is a data race here.
    Shapes with whole column chunks only: lanes beyond the last column deliberately redo the chunk's first
    column and store the same bits to the same address, which ThreadSanitizer rightly calls a race."""
    d, exe = tmp_path, emu_dense_tsan
    _check(_run(exe, d, (1, 64, 4, 32), seed=1), 1e-5, 1e-4)
    _check(_run(exe, d, (1, 70, 3, 64), seed=2), 1e-5, 1e-4)
    _check(_run(exe, d, (1, 128, 4, 64), extra=("wide", 64, 1, 2), seed=3), 1e-5, 1e-4)
    _check(_run(exe, d, (1, 136, 2, 64), extra=("wide", 72, 0, 1), seed=4), 1e-5, 1e-4)
    _check(_run(exe, d, (1, 128, 4, 64), extra=("wide", 64, 1, 2, "deep"), seed=6), 1e-5, 1e-4)
    _check(_run(exe, d, (2, 64, 2, 64), extra=("wide", 64, 0, 1, "deep"), seed=7), 1e-5, 1e-4)
    # one barrier per step, two LDS planes: the rank form over several tiles per workgroup is the case that needs
    # the extra barrier per tile (found here: without it the next tile's first write races the row-sum reads)
    _check(_run(exe, d, (1, 256, 2, 64), extra=("wide", 64, 1, 4, "deep2"), seed=8), 1e-5, 1e-4)
    _check(_run(exe, d, (3, 128, 2, 64), extra=("wide", 64, 0, 2, "deep2"), seed=9), 1e-5, 1e-4)
    _check(_run(exe, d, (1, 64, 2, 64), mode="fixed", seed=5), 1e-5, None)
    r = _run(exe, d, (1, 64, 4, 32), seed=1, scale=2.0 ** -70)   # sign-domain flag raised: the fix-up kernels run
    assert r["domain_flag"] == 1
    _check(r, 1e-5, 1e-4)


def _dims(exe, shape):
    r = subprocess.run([exe, "dims"] + [str(x) for x in shape], env=ENV, capture_output=True, text=True)
    assert r.returncode == 0, (shape, r.stderr[-800:])   # an invalid launch aborts the runner
    rcs = dict(re.findall(r"^(forward|backward|fixed) rc (-?\d+)$", r.stdout, flags=re.M))
    launches = [(m[0].strip("()"), tuple(int(x) for x in m[1].split()), int(m[2]), int(m[3]))
                for m in re.findall(r"^(.+?) \| (\d+ \d+ \d+) \| (\d+) \| (\d+)$", r.stdout, flags=re.M)]
    return rcs, launches


def test_launch_geometry_at_full_size(runner):
    """Every launch of the dense forward, backward and fixed-point forward at sizes no emulation can run: the
    three dense baseline configurations and the 40 cells of the reference's timing grid at its batch of 512
    (benchmark.py:57-66).  The host logic runs as in the library with nothing behind the pointers; the runner
    checks each launch against what a HIP launch accepts (grid 2^31-1 x 65535 x 65535, 1024 threads, 64 KiB of
    dynamic LDS) and reports it."""
    rcs, launches = _dims(runner, (8, 4096, 16, 64))
    assert rcs == {"forward": "0", "backward": "0", "fixed": "0"}
    assert launches[:4] == [("dense_fwd_f32_pipe<64, false>", (64, 4, 8), 1024, 0),
                            ("dense_bwd_f32_fast<64, 512, 4, true, true, true>", (16, 2, 8), 512, 4 * 8 * 68 * 4),
                            ("dense_bwd_reduce_colsum", (2048, 1, 1), 256, 0),
                            ("dense_bwd_reduce_dk<true, true, false>", (32768, 1, 1), 256, 0)]
    # without column ranks the backward brackets its kernels with the sign-domain check and the exact fix-up
    rcs, launches = _dims(runner, (16, 1024, 8, 64))
    assert rcs["backward"] == "0" and [l[0] for l in launches[1:]][:6] == [
        "dense_bwd_clear_flag", "dense_bwd_sign_domain", "dense_bwd_f32_fast<64, 512, 4, false, false, true>",
        "dense_bwd_reduce_dk<true, false, false>", "dense_bwd_exact_if_flagged", "fixed_absmax"]
    assert launches[3] == ("dense_bwd_f32_fast<64, 512, 4, false, false, true>", (16, 1, 16), 512, 8704)
    assert launches[2][1] == (4096, 1, 1) and launches[5][1] == (16 * 1024 * 8 * 64 // 256, 2, 1)
    assert _dims(runner, (2, 64, 4, 32))[0]["backward"] == "0"
    kernels = set()
    for T in (16, 32, 64, 128, 256):
        for W in (16, 32, 33, 64, 65, 96, 97, 128):
            rcs, launches = _dims(runner, (512, T, 8, W))
            assert rcs["forward"] == "0" and rcs["backward"] == "0", (T, W, rcs)
            kernels.update(name for name, _, _, _ in launches)
    # the grid walks the one-workgroup forward, five widths of the tiled forward and the 32-token backward tiles
    assert {"dense_fwd_small<T>", "dense_fwd_f32_fast<16>", "dense_fwd_f32_pipe<32, false>", "dense_fwd_f32_fast<48>",
            "dense_fwd_f32_pipe<64, false>", "dense_fwd_f32_fast<80>", "dense_fwd_f32_pipe<96, false>", "dense_pad_rows",
            "dense_bwd_f32_fast<32, 1024, 1, false, false, false>"} <= kernels
    # sizes at the edges of what the host logic accepts end in a return code, not in a launch that HIP would refuse
    for shape in ((65535, 32, 1, 32), (70000, 32, 1, 32), (1, 8192, 64, 128), (1, 100000, 1, 32), (3, 16, 4096, 16)):
        _dims(runner, shape)
