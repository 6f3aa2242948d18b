"""Writes tests/golden/isa_digests_gpu_tested.json: for every kernel of the HIP sources as they were at a given
commit, the digest of its gfx950 instruction stream (build.isa_digests: instructions and operands in order,
without comments, labels and directives), keyed by "<source file> <demangled kernel name with template
arguments>".  Run in the build container (needs git, hipcc and c++filt; no GPU):

    python tests/golden/make_isa_digests.py 19a3f4b

The commit to give is the last one whose kernels ran the GPU test suite (the runs of 19a3f4b are recorded in
gpu_pytest_log_of_the_digested_kernels.txt beside this file); tests/test_isa_digests_cpu.py then
shows, kernel by kernel, that the library built from the current sources runs the same machine code.  A second
table holds the digests with the immediate offsets of the loads from the kernel-argument pointer left out: a kernel
that only gained an argument agrees with its tested form there.
"""
import glob
import json
import os
import re
import subprocess
import sys
import tempfile

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
sys.path.insert(0, os.path.join(ROOT, "l1-attention_amd"))
import build  # noqa: E402


def short_name(mangled):
    d = subprocess.run(["c++filt", mangled], stdout=subprocess.PIPE, text=True, check=True).stdout.strip()
    m = re.search(r"\(anonymous namespace\)::(\w+(?:<[^>]*>)?)\(", d)
    return m.group(1) if m else d


def digests_of_tree(pkg):
    """({kernel: [digest, instructions]}, the same with the offsets of kernel-argument loads left out)."""
    out, masked = {}, {}
    for src in sorted(glob.glob(os.path.join(pkg, "csrc", "*.hip"))):
        cmd = [os.environ.get("HIPCC", "/opt/rocm/bin/hipcc"), "--offload-arch=" + build.ARCH, "-O3", "-std=c++17",
               "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops", "-I", os.path.join(pkg, "csrc"),
               "-S", "--cuda-device-only", src, "-o", "-"]
        text = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.DEVNULL, text=True, check=True).stdout
        names = {}
        for k, (h, n) in sorted(build.isa_digests(text).items()):
            names[k] = "%s %s" % (os.path.basename(src), short_name(k))
            out[names[k]] = [h, n]
        for k, (h, n) in sorted(build.isa_digests(text, mask_kernarg_offsets=True).items()):
            masked[names[k]] = [h, n]
    return out, masked


def main():
    commit = sys.argv[1]
    with tempfile.TemporaryDirectory() as d:
        wt = os.path.join(d, "wt")
        subprocess.run(["git", "-C", ROOT, "worktree", "add", "-q", wt, commit], check=True)
        try:
            kernels, masked = digests_of_tree(os.path.join(wt, "l1-attention_amd"))
        finally:
            subprocess.run(["git", "-C", ROOT, "worktree", "remove", "--force", wt], check=True)
    full = subprocess.run(["git", "-C", ROOT, "rev-parse", commit], stdout=subprocess.PIPE, text=True).stdout.strip()
    path = os.path.join(HERE, "isa_digests_gpu_tested.json")
    json.dump({"commit": full, "arch": build.ARCH, "kernels": kernels, "kernels_kernarg_offsets_masked": masked},
              open(path, "w"), indent=0, sort_keys=True)
    print("wrote", path, len(kernels), "kernels of", full)


if __name__ == "__main__":
    main()
