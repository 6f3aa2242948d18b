"""CPU run of the edge-list kernels (csrc/coo.hip compiled for the host against tests/cpu_emu/hip/hip_runtime.h) under
AddressSanitizer + UndefinedBehaviorSanitizer and under ThreadSanitizer: l1attn_expand_coo bit for bit against the
oracle's restatement of the reference loop (python/l1attn_sparse.py:382-427), the reference's known answers
(README.md:89; python/l1attn_sparse.py:576) and an O(E^2) count; l1attn_sparse_plan_build against stable sorts in
numpy in the layout of csrc/plan.h.

Every kernel of coo.hip runs from its source here: coo_extract, radix_hist, scan_exclusive, radix_scatter,
ranks_from_sorted, segment_ptrs, plan_fill_csr, plan_fill_csc, max_segment, fill_words, plan_header.  Ballots,
shuffles and __syncthreads() are barriers among OS threads and atomics are host atomics; the one place where lanes
pass values through LDS between two cross-lane operations is a barrier among the lanes involved.  What this cannot
show is what only a GPU can: the instruction encodings, timing, and the hardware's own lockstep.
"""
import os
import struct
import subprocess

import numpy as np
import pytest
import torch

import closed_forms as cf
from oracle import oracle

LONG = 128  # PLAN_LONG_SEGMENT of csrc/plan.h
MAGIC = 0x4C314132
ENV = dict(os.environ, ASAN_OPTIONS="verify_asan_link_order=0:detect_leaks=0",
           TSAN_OPTIONS="halt_on_error=1 report_signal_unsafe=0")


def _call(exe, tmp_path, mode, co, T=0):
    co = co.contiguous()
    bits = 64 if co.dtype == torch.int64 else 32
    E, stride = (co.shape[0], co.shape[1]) if co.dim() == 2 else (0, 2)
    fin, fout = str(tmp_path / "in.bin"), str(tmp_path / "out.bin")
    with open(fin, "wb") as f:
        f.write(struct.pack("5q", mode, bits, stride, E, T))
        f.write(co.numpy().tobytes())
    r = subprocess.run([exe, fin, fout], env=ENV, capture_output=True, text=True, timeout=600)
    assert r.returncode == 0, (r.returncode, r.stderr[-3000:])
    return np.fromfile(fout, np.int32)


def expand(exe, tmp_path, co):
    raw = _call(exe, tmp_path, 0, co)
    E = co.shape[0]
    assert raw.shape[0] == 3 + 4 * E
    return int(raw[0]), torch.from_numpy(raw[3:].copy()).view(E, 4), int(raw[1]), int(raw[2])


def _align64(n):
    return (n + 63) // 64 * 64


def plan(exe, tmp_path, coo, T):
    """rc of build and check, header, and the plan's arrays by name (csrc/plan.h)."""
    raw = _call(exe, tmp_path, 1, coo, T)
    E = coo.shape[0]
    rc, rc2, hdr, w = int(raw[0]), int(raw[1]), raw[2:18], raw[18:]
    pa, ea = _align64(T + 2), _align64(max(E, 1))
    cap = E // LONG + 1
    off, out = 64, {}
    for name, n, used in (("dst_ptr", pa, T + 2), ("src_ptr", pa, T + 2), ("csr_src", ea, E), ("csr_row", ea, E),
                          ("csc_dst", ea, E), ("csc_slot", ea, E), ("long_dst", _align64(cap), cap),
                          ("long_src", _align64(cap), cap)):
        out[name] = w[off:off + used].astype(np.int64)
        off += n
    assert off == w.shape[0]
    return rc, rc2, hdr, w[:16], out


def check_plan(exe, tmp_path, coo, T):
    """The built plan against stable sorts of the valid rows; rows with an index outside [0, T) are dropped."""
    E = coo.shape[0]
    rc, rc2, hdr, head, a = plan(exe, tmp_path, coo, T)
    assert rc == 0
    d, s = coo[:, 0].numpy().astype(np.int64), coo[:, 1].numpy().astype(np.int64)
    ok = (d >= 0) & (d < T) & (s >= 0) & (s < T)
    bad = int((~ok).any())
    assert rc2 == (-4 if bad else 0)
    dk, sk = np.where(ok, d, T), np.where(ok, s, T)  # dropped rows sort behind the last token
    od, os_ = np.argsort(dk, kind="stable"), np.argsort(sk, kind="stable")
    slot_of_row = np.empty(E, np.int64)
    slot_of_row[od] = np.arange(E)

    def ptr(key):
        p = np.zeros(T + 2, np.int64)
        p[1:] = np.cumsum(np.bincount(key, minlength=T + 1))
        return p
    dp, sp = ptr(dk), ptr(sk)
    assert np.array_equal(a["dst_ptr"], dp) and np.array_equal(a["src_ptr"], sp)
    assert np.array_equal(a["csr_row"], od) and np.array_equal(a["csr_src"], sk[od])
    assert np.array_equal(a["csc_dst"], dk[os_]) and np.array_equal(a["csc_slot"], slot_of_row[os_])
    degd, degs = np.diff(dp[:T + 1]), np.diff(sp[:T + 1])
    ld, ls = np.nonzero(degd > LONG)[0], np.nonzero(degs > LONG)[0]
    want = [MAGIC, E, T, bad, int(degd.max()) if T else 0, int(degs.max()) if T else 0, int(dp[T]), len(ld), len(ls)]
    assert list(hdr[:9]) == want and list(head[:9]) == want
    # the lists of long segments come in any order
    assert sorted(a["long_dst"][:len(ld)]) == list(ld) and sorted(a["long_src"][:len(ls)]) == list(ls)
    return hdr


def test_expand_coo_known_answers_on_cpu(emu_coo, tmp_path):
    co = torch.cartesian_prod(torch.arange(3), torch.arange(3))                                   # README.md:89
    rc, coo, dmx, smx = expand(emu_coo, tmp_path, co)
    assert rc == 0 and (dmx, smx) == (3, 3)
    assert coo[:, 2].tolist() == [0, 1, 2, 0, 1, 2, 0, 1, 2] and coo[:, 3].tolist() == [0, 0, 0, 1, 1, 1, 2, 2, 2]
    co = torch.tensor([[0, 0], [0, 1], [0, 2], [1, 0], [1, 1], [2, 0], [2, 1]], dtype=torch.int32)  # python/l1attn_sparse.py:576
    rc, coo, dmx, smx = expand(emu_coo, tmp_path, co)
    assert rc == 0 and (dmx, smx) == (3, 3) and torch.equal(coo[:, :2], co)
    assert coo[:, 2].tolist() == [0, 1, 2, 0, 1, 0, 1] and coo[:, 3].tolist() == [0, 0, 0, 1, 1, 2, 2]
    rc, coo, dmx, smx = expand(emu_coo, tmp_path, torch.zeros(0, 2, dtype=torch.int64))          # E = 0 -> (empty, 1, 1)
    assert rc == 0 and (dmx, smx) == (1, 1) and coo.numel() == 0
    # a negative index, or one beyond int32, is refused before anything is sorted
    assert expand(emu_coo, tmp_path, torch.tensor([[0, 1], [2, -1]]))[0] == -4
    assert expand(emu_coo, tmp_path, torch.tensor([[0, 1], [2 ** 31, 1]]))[0] == -4


@pytest.mark.parametrize("E,n_tok,dtype,stride", [
    (1, 1, torch.int64, 2),
    (300, 7, torch.int32, 2),          # one tile, heavy ties
    (2048, 300, torch.int64, 2),       # exactly one tile of the radix sort, two digit passes
    (2049, 3, torch.int32, 3),         # one row into the second tile; a third column is ignored
    (5000, 70000, torch.int64, 2),     # three digit passes, mostly unique keys
    (6500, 40, torch.int32, 2),        # four tiles, long runs of one key across tile and wave boundaries
])
def test_expand_coo_bit_exact_on_cpu(emu_coo, tmp_path, E, n_tok, dtype, stride):
    g = torch.Generator().manual_seed(E + n_tok)
    co = torch.randint(0, n_tok, (E, stride), generator=g).to(dtype)
    rc, coo, dmx, smx = expand(emu_coo, tmp_path, co)
    ocoo, odmx, osmx = oracle.expand_coo(co[:, :2])
    assert rc == 0 and torch.equal(coo, ocoo) and (dmx, smx) == (odmx, osmx)
    if E <= 2100:
        bcoo, bd, bs = cf.expand_coo_bruteforce(co[:, :2])
        assert torch.equal(coo, bcoo) and (dmx, smx) == (bd, bs)


def test_expand_coo_sorted_and_constant_columns_on_cpu(emu_coo, tmp_path):
    """Inputs a radix sort can get wrong without random data showing it: already sorted keys, reverse-sorted keys,
    one key for every row (a single digit bucket across all tiles), and the largest int32 index."""
    E = 2100
    ar = torch.arange(E)
    for co in (torch.stack([ar // 3, ar % 5], 1), torch.stack([(E - 1 - ar) // 2, ar.flip(0)], 1),
               torch.stack([torch.full((E,), 9), ar % 2], 1),
               torch.stack([torch.where(ar % 2 == 0, 2 ** 31 - 1, 0), ar % 7], 1)):
        rc, coo, dmx, smx = expand(emu_coo, tmp_path, co)
        # (the O(E^2) count: the oracle keeps one counter per possible key, 2^31 of them for the last case)
        ocoo, odmx, osmx = cf.expand_coo_bruteforce(co)
        assert rc == 0 and torch.equal(coo, ocoo) and (dmx, smx) == (odmx, osmx)


@pytest.mark.parametrize("E,T,seed", [(0, 5, 0), (1, 1, 1), (40, 9, 2), (2048, 64, 3), (4100, 33, 4), (3000, 3000, 5)])
def test_plan_build_on_cpu(emu_coo, tmp_path, E, T, seed):
    g = torch.Generator().manual_seed(seed)
    coo = torch.randint(0, T, (E, 4), generator=g).to(torch.int32)
    hdr = check_plan(emu_coo, tmp_path, coo, T)
    if (E, T) == (4100, 33):
        assert hdr[7] > 0 and hdr[8] > 0  # segments beyond 128 edges, in both views


def test_plan_build_drops_rows_with_bad_indices_on_cpu(emu_coo, tmp_path):
    g = torch.Generator().manual_seed(11)
    T = 50
    coo = torch.randint(0, T, (2500, 2), generator=g).to(torch.int32)
    coo[7, 0], coo[100, 1], coo[2499, 0], coo[2100, 1] = -1, T, T + 5, -3
    hdr = check_plan(emu_coo, tmp_path, coo, T)
    assert hdr[3] == 1 and hdr[6] == 2496


def test_edge_list_kernels_on_cpu_under_thread_sanitizer(emu_coo_tsan, tmp_path):
    """ThreadSanitizer sees every LDS and global access of the sort: the per-wave digit counters of radix_scatter are
    read by a digit's lanes and then written by its first lane, which is ordered by the wave's lockstep on the GPU
    and by the barrier standing for it here; anything else unordered would be reported."""
    g = torch.Generator().manual_seed(21)
    co = torch.randint(0, 300, (2100, 2), generator=g)   # two tiles of the sort
    rc, coo, dmx, smx = expand(emu_coo_tsan, tmp_path, co)
    ocoo, odmx, osmx = oracle.expand_coo(co)
    assert rc == 0 and torch.equal(coo, ocoo) and (dmx, smx) == (odmx, osmx)
    check_plan(emu_coo_tsan, tmp_path, ocoo, 300)
