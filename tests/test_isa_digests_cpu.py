"""CPU-only: the machine code of the kernels that passed the GPU test suite has not changed since.

tests/golden/isa_digests_gpu_tested.json holds, per kernel, the digest of the gfx950 instruction stream compiled
from the sources of the last commit whose kernels ran the GPU tests (written by tests/golden/make_isa_digests.py).
The build writes the same digests for the current sources into l1-attention_amd/isa_digests.txt.  Every kernel of
the tested set must still be there with the same digest; the exceptions are listed below with their reason.
"""
import json
import os
import re
import shutil
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
GOLD = os.path.join(ROOT, "tests", "golden", "isa_digests_gpu_tested.json")
NOW = os.path.join(ROOT, "l1-attention_amd", "isa_digests.txt")

# Kernels of the tested set that exist in another form today.
REPLACED = {
    # The pipelined forward gained a template flag and one kernel argument (the fixed-point variant's grid pointer):
    # <W> is now <W, false>; its instruction stream differs from the tested one in the offsets of the
    # kernel-argument loads (and the order of two adjacent ones) and in nothing else: the digests that leave
    # those offsets out are equal.
    "dense.hip dense_fwd_f32_pipe<32>": "dense.hip dense_fwd_f32_pipe<32, false>",
    "dense.hip dense_fwd_f32_pipe<64>": "dense.hip dense_fwd_f32_pipe<64, false>",
    "dense.hip dense_fwd_f32_pipe<96>": "dense.hip dense_fwd_f32_pipe<96, false>",
}
# Instantiations the host no longer selects (grouped dst tiles now always run the branch-free step loop).
DROPPED = {"dense.hip dense_bwd_f32_fast<64, 512, 4, false, true, false>",
           "dense.hip dense_bwd_f32_fast<64, 512, 4, true, true, false>",
           "dense.hip dense_bwd_f32_fast<64, 512, 8, false, true, false>"}


def _short(mangled):
    d = subprocess.run(["c++filt", mangled], stdout=subprocess.PIPE, text=True, check=True).stdout.strip()
    m = re.search(r"\(anonymous namespace\)::(\w+(?:<[^>]*>)?)\(", d)
    return m.group(1) if m else d


def _today(name):
    # the sparse kernels gained a storage type as last template argument; in the float32 and float64
    # instantiations it equals the compute type, which is how the tested kernels are named today
    m = re.match(r"(sparse\.hip sparse_\w+)<(float|double), (.*)>$", name)
    if m:
        return "%s<%s, %s, %s>" % (m.group(1), m.group(2), m.group(3), m.group(2))
    # the tiled dense backward gained a last template argument (the form of the branch-free step loop); the tested
    # kernels are the instantiations of form 0
    m = re.match(r"(dense\.hip dense_bwd_f32_fast)<(.*)>$", name)
    if m:
        return "%s<%s, 0>" % (m.group(1), m.group(2))
    # and its reduction kernel a flag for reading several partial arrays ahead, off in the tested kernels
    m = re.match(r"(dense\.hip dense_bwd_reduce_dk)<(.*)>$", name)
    return "%s<%s, false>" % (m.group(1), m.group(2)) if m else name


def test_gpu_tested_kernels_are_unchanged():
    if not os.path.exists(NOW) or shutil.which("c++filt") is None:
        pytest.skip("needs the digest table of a build and c++filt")
    gold = json.load(open(GOLD))
    now, now_masked = {}, {}
    for line in open(NOW):
        src, mangled, digest, count, masked = line.split()
        now["%s %s" % (src, _short(mangled))] = (digest, int(count))
        now_masked["%s %s" % (src, _short(mangled))] = (masked, int(count))
    assert len(gold["kernels"]) == 121 and len(now) >= 200
    same, moved = 0, []
    for name, (digest, count) in gold["kernels"].items():
        if name in DROPPED:
            assert _today(name) not in now
            continue
        if name in REPLACED:
            d, c = now[REPLACED[name]]
            assert c == count and d != digest  # same length; the argument offsets differ, and nothing else:
            assert now_masked[REPLACED[name]] == tuple(gold["kernels_kernarg_offsets_masked"][name]), name
            moved.append(name)
            continue
        assert _today(name) in now, "kernel of the tested set is gone: " + name
        assert now[_today(name)] == (digest, count), "machine code changed since it ran on a GPU: " + name
        assert now_masked[_today(name)] == tuple(gold["kernels_kernarg_offsets_masked"][name]), name
        same += 1
    assert same == 115 and len(moved) == 3
