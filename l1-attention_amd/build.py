"""Compile the HIP sources under csrc/ into libl1attn_hip.so next to this file.

    python build.py            # hipcc --offload-arch=gfx950, in-tree output

hipcc cross-compiles without a GPU.  Packed fp32 instructions are disabled for all device
code (-packed-fp32-ops): the kernels issue scalar-per-lane fp32 VALU operations only.
"""
import glob
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
LIB = os.path.join(HERE, "libl1attn_hip.so")
ARCH = "gfx950"


def sources():
    return sorted(glob.glob(os.path.join(HERE, "csrc", "*.hip")))


def build(verbose=False):
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    objs = []
    procs = []
    os.makedirs(os.path.join(HERE, "build"), exist_ok=True)
    for src in sources():
        obj = os.path.join(HERE, "build", os.path.basename(src) + ".o")
        cmd = [hipcc, "--offload-arch=" + ARCH, "-O3", "-std=c++17", "-fPIC",
               "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
               "-I", os.path.join(HERE, "csrc"), "-c", src, "-o", obj]
        if verbose:
            print(" ".join(cmd))
        procs.append((src, subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)))
        objs.append(obj)
    for src, p in procs:
        out, _ = p.communicate()
        # the host pass warns that it does not know the packed-fp32 feature; that is expected
        out = "\n".join(l for l in out.splitlines() if "packed-fp32-ops" not in l)
        if p.returncode != 0:
            raise RuntimeError("hipcc failed on %s:\n%s" % (src, out))
        if verbose and out.strip():
            print(out)
    cmd = [hipcc, "--offload-arch=" + ARCH, "-shared", "-fPIC", "-o", LIB] + objs
    if verbose:
        print(" ".join(cmd))
    subprocess.run(cmd, check=True)
    return LIB


if __name__ == "__main__":
    print(build(verbose="-v" in sys.argv))
