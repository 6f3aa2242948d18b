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


def _emu_runner(tmp_path_factory, name, cxx):
    """The CPU build of one kernel file's runner (tests/cpu_emu/run_<name>.cpp) under AddressSanitizer and
    UndefinedBehaviorSanitizer; built once per session, every emulation test module shares it."""
    exe = str(tmp_path_factory.mktemp("emu_" + name) / ("run_" + name))
    subprocess.run([cxx, "-std=c++20", "-O1", "-g", "-pthread", "-fsanitize=address,undefined",
                    "-fno-sanitize-recover=all", "-I", EMU, "-x", "c++", os.path.join(EMU, "run_%s.cpp" % name), "-o", exe],
                   check=True)
    return exe


@pytest.fixture(scope="session")
def emu_fused(tmp_path_factory):
    return _emu_runner(tmp_path_factory, "fused", "g++")


@pytest.fixture(scope="session")
def emu_sparse(tmp_path_factory):
    if not os.path.exists(CLANG):
        pytest.skip("needs ROCm's clang++ as host compiler")
    return _emu_runner(tmp_path_factory, "sparse", CLANG)


@pytest.fixture(scope="session")
def emu_ranks(tmp_path_factory):
    return _emu_runner(tmp_path_factory, "ranks", "g++")
