"""CPU-only: the GPU test files run end to end on the CPU -- the real Python operators and drivers, the real ctypes
binding with its argtypes, and a library built from the product's kernel sources for the host
(tests/cpu_emu/lib_*.cpp: dense.hip, dense_rank.hip, fixed.hip, fused.hip, rank_sort.hip and sparse.hip as they are,
GPU threads as OS threads; host stand-ins only for the library block sort inside dense_rank.hip and, to keep the runs
short, for coo.hip, whose kernels run from source in tests/test_cpu_emulation_coo.py).

Everything else on the CPU either runs the kernels through C++ runners (which call the entry points themselves) or
walks the drivers against stand-ins that accept anything.  Neither notices a driver that passes the right kinds of
arguments in the wrong order.  Here the drivers' own calls reach the kernels, and the GPU tests' own comparisons
against the oracle judge the result: the test functions are taken from tests/test_*_gpu.py and tests/wip_*_gpu.py
unchanged, at the shapes an emulation can walk.  Tensors stay on the CPU: `.cuda()` is a copy in host memory and
`Tensor.is_cuda` says yes."""
import contextlib
import ctypes
import importlib.util
import os
import subprocess

import pytest
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
EMU = os.path.join(HERE, "cpu_emu")
CLANG = "/opt/rocm/llvm/bin/clang++"
PARTS = (("lib_dense", "g++"), ("lib_fixed", "g++"), ("lib_fused", "g++"), ("lib_ranks", "g++"),
         ("lib_ranks_default", "g++"), ("lib_sparse", CLANG), ("lib_host", "g++"))

pytestmark = pytest.mark.skipif(not os.path.exists(CLANG), reason="needs ROCm's clang++ (bfloat16 and float16 on the host)")


@pytest.fixture(scope="module")
def emulated_library_path(tmp_path_factory):
    d = tmp_path_factory.mktemp("emulib")
    jobs = []
    for name, cxx in PARTS:
        lines = "-gline-tables-only" if cxx == CLANG else "-g1"
        cmd = [cxx, "-std=c++20", "-O1", lines, "-fPIC", "-pthread", "-I", EMU, "-x", "c++", "-c",
               os.path.join(EMU, name + ".cpp"), "-o", str(d / (name + ".o"))]
        jobs.append((cmd, subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)))
    for cmd, p in jobs:
        text, _ = p.communicate()
        assert p.returncode == 0, "%s\n%s" % (" ".join(cmd), text[-3000:])
    lib = str(d / "libl1attn_emu.so")
    # linked by clang++: its runtime holds the float <-> bfloat16 conversions the sparse kernels call on the host
    subprocess.run([CLANG, "-shared", "-pthread", "-o", lib] + [str(d / (n + ".o")) for n, _ in PARTS], check=True)
    return lib


@pytest.fixture()
def on_the_emulated_library(emulated_library_path, monkeypatch):
    import _l1attn_hip as drv
    monkeypatch.setattr(drv, "_LIB_PATH", emulated_library_path)
    monkeypatch.setattr(drv, "_lib", None)                 # lib() loads the path above and sets its argtypes on it
    monkeypatch.setattr(drv, "_enabled", set(drv.EXPERIMENTAL))
    monkeypatch.setattr(drv, "stream_of", lambda x: ctypes.c_void_p(None))
    # a copy, as on a GPU: x.cuda().requires_grad_() must not turn x itself into a leaf that collects gradients
    monkeypatch.setattr(torch.Tensor, "cuda", lambda self, *a, **k: self.clone())
    real_to = torch.Tensor.to

    def to(self, *a, **k):  # .to("cuda") stays where it is
        is_gpu = lambda x: (isinstance(x, str) and x.startswith("cuda")) or (isinstance(x, torch.device) and x.type == "cuda")
        a = tuple("cpu" if is_gpu(x) else x for x in a)
        if is_gpu(k.get("device")):
            k["device"] = "cpu"
        return real_to(self, *a, **k)

    monkeypatch.setattr(torch.Tensor, "to", to)
    monkeypatch.setattr(torch.Tensor, "is_cuda", property(lambda self: True))
    monkeypatch.setattr(torch.cuda, "synchronize", lambda *a, **k: None)
    monkeypatch.setattr(torch.cuda, "device", lambda d: contextlib.nullcontext())
    assert drv.lib().l1attn_version() == -1                # the emulated library, not the product's
    return drv


def _load(name):
    spec = importlib.util.spec_from_file_location(name, os.path.join(HERE, name + ".py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


# One or two small cases per driver function: what this file adds to the other CPU tests is that every pointer and
# size a driver passes lands in the right parameter; the kernels' shapes are walked in tests/test_cpu_emulation*.py.
# L1ATTN_EMULATED_LIBRARY_FULL=1 runs the longer selection (about four minutes).
FULL = bool(os.environ.get("L1ATTN_EMULATED_LIBRARY_FULL"))


def test_dense_gpu_tests_on_the_emulated_library(on_the_emulated_library):
    t = _load("test_dense_gpu")
    shapes = [(2, 64, 4, 32), (2, 3, 16, 7), (1, 100, 3, 33)]
    if FULL:
        shapes += [(1, 16, 8, 64), (1, 70, 20, 48), (1, 40, 2, 128), (3, 33, 1, 65)]
    for shape in shapes:
        t.test_dense_f32_vs_oracle(shape)
    for shape in [(2, 5, 3, 7)] + ([(2, 64, 4, 32), (1, 16, 8, 64), (1, 100, 3, 33)] if FULL else []):
        t.test_dense_f64_vs_oracle(shape)
    t.test_dense_golden_reference_extension()
    t.test_dense_forward_odd_width_with_and_without_workspace()
    t.test_dense_in_a_model_block()
    if FULL:
        t.test_dense_ties_onehot_fixture()
        t.test_dense_deterministic_and_inputs_untouched()


def test_sparse_gpu_tests_on_the_emulated_library(on_the_emulated_library):
    t = _load("test_sparse_gpu")
    t.test_check_sparse_cases_vs_oracle(torch.float64, True)       # full, permuted, permuted minus four; uni and bidi
    t.test_sparse_golden_reference_extension("sA", True)
    t.test_sparse_value_width_differs_from_key_width()
    if FULL:
        t.test_check_sparse_cases_vs_oracle(torch.float32, False)
        for shape in t.SHAPES[:4]:
            for sm in (True, False):
                t.test_sparse_and_bidi_f32_vs_oracle(shape, sm)
        t.test_sparse_golden_reference_extension("sB", False)
        t.test_sparse_full_list_equals_dense_attention(False)     # sparse operator against the dense operator


def test_fused_gpu_tests_on_the_emulated_library(on_the_emulated_library):
    t = _load("wip_fused_gpu")
    for shape in (t.SHAPES if FULL else t.SHAPES[:1] + t.SHAPES[4:5] + t.SHAPES[8:9]):
        t.test_fused_forward_vs_oracle(shape)
    for shape in [(2, 64, 4, 32)] + ([(1, 100, 3, 64), (1, 33, 9, 64), (1, 40, 2, 48)] if FULL else []):
        t.test_fused_pipelined_forward_equals_the_plain_one(shape)
    t.test_fused_pipelined_backward_stage_equals_the_plain_one((1, 33, 9, 64))
    for shape in (t.BWD_SHAPES[:5] if FULL else t.BWD_SHAPES[:1]):
        t.test_fused_backward_vs_oracle(shape)
    t.test_fused_backward_in_batch_slabs_equals_the_whole_batch()
    t.test_fixed_point_forward_vs_oracle((2, 64, 4, 32), False)
    if FULL:
        t.test_fused_gradcheck_fp64()
        t.test_fused_in_a_model_block(21)


def test_sparse_half_gpu_tests_on_the_emulated_library(on_the_emulated_library):
    t = _load("wip_sparse_half_gpu")
    t.test_half_forward_vs_f32_entry_and_oracle(torch.float16, t.SHAPES[0], True)
    t.test_half_backward_vs_autograd_closed_form(torch.bfloat16, (2, 9, 3, 5, 5, 40), True)
    for dt in t.DTYPES:
        t.test_half_empty_list(dt)
    if FULL:
        t.test_half_forward_vs_f32_entry_and_oracle(torch.bfloat16, t.SHAPES[1], False)
        t.test_half_backward_vs_autograd_closed_form(torch.float16, (2, 20, 3, 8, 12, 90), False)


@pytest.mark.skipif(not FULL, reason="part of the longer selection (L1ATTN_EMULATED_LIBRARY_FULL=1)")
def test_bench_on_the_emulated_library(on_the_emulated_library, monkeypatch, capsys):
    """bench.py's default run and its --extra legs at shrunken sizes, with the real drivers and kernels behind
    them: the script's own direct library calls (instruction probes, both column-rank entry points) and every leg's
    value check run for real.  Timings mean nothing here."""
    import json
    import sys
    import time

    import bench as b

    class Event(object):
        def __init__(self, enable_timing=False):
            self.t = None

        def record(self, stream=None):
            self.t = time.perf_counter()

        def elapsed_time(self, other):
            return max((other.t - self.t) * 1e3, 1e-6)

    def once(fn, iters, warm=2):  # time_gpu with a single call: an emulated launch takes long enough
        t0 = time.perf_counter()
        fn()
        return (time.perf_counter() - t0) * 1e3

    monkeypatch.setattr(b, "time_gpu", once)
    monkeypatch.setattr(torch.cuda, "is_available", lambda: True)
    monkeypatch.setattr(torch.cuda, "Event", Event)
    for name in ("empty_cache", "reset_peak_memory_stats"):
        monkeypatch.setattr(torch.cuda, name, lambda *a, **k: None)
    for name in ("memory_allocated", "max_memory_allocated"):
        monkeypatch.setattr(torch.cuda, name, lambda *a, **k: 0)
    monkeypatch.setattr(b, "DEVICE", "cpu")
    monkeypatch.setattr(b, "HEADLINE", (1, 64, 1, 32))
    monkeypatch.setattr(b, "SECOND", (1, 32, 1, 64))
    monkeypatch.setattr(b, "CONFIG4", ((1, 24, 1, 32), 4))
    monkeypatch.setattr(b, "CONFIG5", (1, 32, 1, 64))

    def run(*argv):
        monkeypatch.setattr(sys, "argv", ["bench.py"] + list(argv))
        capsys.readouterr()
        b.main()
        return json.loads(capsys.readouterr().out.strip().splitlines()[-1])

    out = run("--steps", "1", "--warmup", "0", "--skip-cpu")
    assert out["value"] > 0 and "error" not in out["sparse"] and "error" not in out["valu_probe"]
    assert out["sparse"]["config4_uni"]["edges"] > 0 and out["sparse"]["config5_bidi"]["edges"] > 0
    assert out["dense"]["backward_plan"]["step_loop_form"] == 0
    x = run("--extra")["extra"]
    for row in x["fused_forward"].values():
        assert row["max_rel_diff"] < 1e-5                      # fused against the composition, both on the kernels
    for row in x["fixed_point_forward"].values():
        assert row["max_rel_diff_to_fp32_kernel_batch0"] < 1e-5
    assert len(x["instruction_rates"]) == 4 and len(x["sparse_16bit"]) == 2


def test_smoke_on_the_emulated_library(on_the_emulated_library, monkeypatch, capsys):
    """__graft_entry__.smoke() as it is: dense, expandCoo, sparse and bidirectional against the oracle."""
    import __graft_entry__ as entry
    monkeypatch.setattr(torch.cuda, "is_available", lambda: True)
    monkeypatch.setattr(torch.cuda, "get_device_name", lambda *a: "host emulation")
    entry.smoke()
    assert "smoke ok" in capsys.readouterr().out


def test_late_gpu_tests_on_the_emulated_library(on_the_emulated_library):
    """tests/test_y_configs_gpu.py, the part that is small enough: the native-module stand-ins called the way the
    reference's autograd Functions call them, and (longer selection) the two model blocks, the sign-domain test and
    the training loop."""
    t = _load("test_y_configs_gpu")
    t.test_native_module_stand_ins_on_the_gpu()
    if FULL:
        t.test_model_blocks_on_the_gpu()
        t.test_sign_domain_of_the_fast_float32_backward()
        t.test_training_steps_on_the_gpu_operator_match_torch_autograd()
