import os
import subprocess
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
for p in (ROOT, os.path.join(ROOT, "l1-attention_amd"), os.path.join(ROOT, "tests")):
    if p not in sys.path:
        sys.path.insert(0, p)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


def pytest_collection_modifyitems(config, items):
    import torch
    if torch.cuda.is_available():
        return
    skip = pytest.mark.skip(reason="no GPU visible")
    for item in items:
        if "gpu" in item.keywords:
            item.add_marker(skip)


EMU = os.path.join(ROOT, "tests", "cpu_emu")
CLANG = "/opt/rocm/llvm/bin/clang++"


# runner -> (source name, host compiler, sanitizers)
RUNNERS = {"fused": ("fused", "g++", "address,undefined"), "sparse": ("sparse", CLANG, "address,undefined"),
           "ranks": ("ranks", "g++", "address,undefined"), "dense": ("dense", "g++", "address,undefined"),
           "fused_tsan": ("fused", "g++", "thread"), "sparse_tsan": ("sparse", CLANG, "thread"),
           "dense_tsan": ("dense", "g++", "thread"), "ranks_tsan": ("ranks", "g++", "thread"),
           "coo": ("coo", "g++", "address,undefined"), "coo_tsan": ("coo", "g++", "thread"),
           "ranks_lib": ("ranks_lib", "g++", "address,undefined"), "ranks_lib_tsan": ("ranks_lib", "g++", "thread")}


@pytest.fixture(scope="session")
def _emu_builds(tmp_path_factory):
    """The CPU builds of the kernel files' runners (tests/cpu_emu/run_<name>.cpp), under AddressSanitizer +
    UndefinedBehaviorSanitizer and under ThreadSanitizer, started side by side at the first request and shared by
    every emulation test module of the session.  Line tables only: enough for a sanitizer report to name the line."""
    d = tmp_path_factory.mktemp("emu")
    jobs = {}
    for name, (src, cxx, san) in RUNNERS.items():
        if cxx == CLANG and not os.path.exists(CLANG):
            continue
        exe = str(d / ("run_" + name))
        lines = "-gline-tables-only" if cxx == CLANG else "-g1"
        cmd = [cxx, "-std=c++20", "-O1", lines, "-pthread", "-fsanitize=" + san] + \
              (["-fno-sanitize-recover=all"] if san != "thread" else []) + \
              ["-I", EMU, "-x", "c++", os.path.join(EMU, "run_%s.cpp" % src), "-o", exe]
        jobs[name] = (exe, cmd, subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True))
    return jobs


def _emu_runner(builds, name):
    if name not in builds:
        pytest.skip("needs ROCm's clang++ as host compiler")
    exe, cmd, proc = builds[name]
    text, _ = proc.communicate() if proc.returncode is None else ("", None)
    assert proc.returncode == 0, "%s\n%s" % (" ".join(cmd), text)
    return exe


@pytest.fixture(scope="session")
def emu_fused(_emu_builds):
    return _emu_runner(_emu_builds, "fused")


@pytest.fixture(scope="session")
def emu_sparse(_emu_builds):
    return _emu_runner(_emu_builds, "sparse")


@pytest.fixture(scope="session")
def emu_ranks(_emu_builds):
    return _emu_runner(_emu_builds, "ranks")


@pytest.fixture(scope="session")
def emu_dense(_emu_builds):
    return _emu_runner(_emu_builds, "dense")


@pytest.fixture(scope="session")
def emu_fused_tsan(_emu_builds):
    return _emu_runner(_emu_builds, "fused_tsan")


@pytest.fixture(scope="session")
def emu_sparse_tsan(_emu_builds):
    return _emu_runner(_emu_builds, "sparse_tsan")


@pytest.fixture(scope="session")
def emu_dense_tsan(_emu_builds):
    return _emu_runner(_emu_builds, "dense_tsan")


@pytest.fixture(scope="session")
def emu_ranks_tsan(_emu_builds):
    return _emu_runner(_emu_builds, "ranks_tsan")


@pytest.fixture(scope="session")
def emu_coo(_emu_builds):
    return _emu_runner(_emu_builds, "coo")


@pytest.fixture(scope="session")
def emu_coo_tsan(_emu_builds):
    return _emu_runner(_emu_builds, "coo_tsan")


@pytest.fixture(scope="session")
def emu_ranks_lib(_emu_builds):
    return _emu_runner(_emu_builds, "ranks_lib")


@pytest.fixture(scope="session")
def emu_ranks_lib_tsan(_emu_builds):
    return _emu_runner(_emu_builds, "ranks_lib_tsan")
