"""CPU-only: bench.py walked from its command line to its JSON line without a GPU, so that a slip in the script
itself (a renamed key, a wrong argument, an import) shows here and not as a lost measurement on the GPU box.

The sizes are shrunk through the constants bench.py names them by, the device is the CPU, HIP events are wall-clock
stand-ins and the kernel drivers are the stand-ins of tests/test_wip_gpu_tests_dry_run_cpu.py (the CPU operator
package and closed forms).  The numbers that come out mean nothing; the shape of the output is what is checked."""
import json
import sys
import time

import pytest
import torch

from test_wip_gpu_tests_dry_run_cpu import cpu_stand_ins  # noqa: F401  (fixture)


class _Event(object):
    def __init__(self, enable_timing=False):
        self.t = None

    def record(self, stream=None):
        self.t = time.perf_counter()

    def elapsed_time(self, other):
        return max((other.t - self.t) * 1e3, 1e-6)


class _Lib(object):
    """Probes and column-rank entries: accept anything, report success."""
    def __getattr__(self, name):
        return lambda *a: 0


@pytest.fixture()
def bench(cpu_stand_ins, monkeypatch):  # noqa: F811
    import bench as b
    monkeypatch.setattr(torch.cuda, "is_available", lambda: True)
    monkeypatch.setattr(torch.cuda, "Event", _Event)
    for name in ("empty_cache", "reset_peak_memory_stats"):
        monkeypatch.setattr(torch.cuda, name, lambda *a, **k: None)
    for name in ("memory_allocated", "max_memory_allocated"):
        monkeypatch.setattr(torch.cuda, name, lambda *a, **k: 0)
    monkeypatch.setattr(cpu_stand_ins, "lib", lambda: _Lib())
    monkeypatch.setattr(cpu_stand_ins, "stream_of", lambda x: None)
    monkeypatch.setattr(b, "DEVICE", "cpu")
    monkeypatch.setattr(b, "HEADLINE", (2, 48, 2, 32))
    monkeypatch.setattr(b, "SECOND", (2, 40, 2, 64))
    monkeypatch.setattr(b, "CONFIG4", ((2, 96, 2, 32), 8))
    monkeypatch.setattr(b, "CONFIG5", (1, 256, 2, 64))
    monkeypatch.setattr(b, "CPU_SAMPLE", (1, 32, 2, 16))
    monkeypatch.setattr(b, "COPY_FLOATS", 1 << 10)
    monkeypatch.setattr(b, "SWEEP", {"B": 3, "H": 2, "T": (16, 32), "W": (16, 33)})
    return b


def _run(b, monkeypatch, capsys, *argv):
    monkeypatch.setattr(sys, "argv", ["bench.py"] + list(argv))
    capsys.readouterr()
    b.main()
    return [json.loads(line) for line in capsys.readouterr().out.splitlines() if line.strip()]


def test_default_run_prints_the_one_line(bench, monkeypatch, capsys):
    lines = _run(bench, monkeypatch, capsys, "--steps", "2", "--warmup", "1")
    assert len(lines) == 1
    out = lines[0]
    for key in ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step", "higher_is_better", "scaling",
                "vs_baseline", "dtype", "data", "config", "roofline", "cpu_baseline"):
        assert key in out, key
    assert out["n_gpus"] == 1 and out["steps"] == 2 and out["warmup"] == 1 and out["vs_baseline"] is None
    assert out["dtype"] == "f32" and out["value"] > 0 and "workload" in out["config"] and "model" not in out["config"]
    roof = out["roofline"]
    for key in ("bound", "achieved", "peak", "unit", "frac", "traffic"):
        assert key in roof, key
    assert abs(roof["frac"] - roof["achieved"] / roof["peak"]) < 1e-12 and roof["traffic_source"]["measured_in_this_run"] is False
    cpu = out["cpu_baseline"]
    for key in ("value", "unit", "cores", "kind", "sample"):
        assert key in cpu, key
    assert cpu["kind"] in ("reference", "port") and cpu["value"] > 0 and cpu["cpu_operator_package_fp32"]["value"] > 0
    assert "error" not in out["valu_probe"] and "error" not in out["sparse"]
    for name in ("config4_uni", "config5_bidi"):
        row = out["sparse"][name]
        assert row["edges"] > 0 and row["fwd_bwd_ms"] > 0 and row["bytes_alg"] > row["bytes_min"] > 0
    sp = cpu["sparse"]
    assert sp["cpu_operator_package_fp32"]["edges_per_s"] > 0 and sp["config5_bidi_cpu_operator_package_fp32"]["edges"] > 0
    assert (cpu["kind"] == "reference") == ("reference_fp64" in sp)


def test_side_flags(bench, monkeypatch, capsys):
    out, = _run(bench, monkeypatch, capsys, "--skip-sparse", "--skip-cpu", "--steps", "1", "--warmup", "0")
    assert "sparse" not in out and out["cpu_baseline"] is None
    for which in ("config4", "config5"):
        out, = _run(bench, monkeypatch, capsys, "--skip-dense", "--only", which)
        assert len(out["sparse"]) == 1 and next(iter(out["sparse"])).startswith(which)
    rows = _run(bench, monkeypatch, capsys, "--sweep")
    assert [(r["seq_length"], r["width"]) for r in rows] == [(16, 16), (16, 33), (32, 16), (32, 33)]
    assert all(r["avg_forward_ms"] > 0 and r["avg_backward_ms"] > 0 and r["batch_size"] == 3 for r in rows)
    out, = _run(bench, monkeypatch, capsys, "--copy-calibration")
    assert out["copies"] == 3 and out["copy_calibration_bytes_read"] == 4 << 10
    with pytest.raises(SystemExit) as e:
        _run(bench, monkeypatch, capsys, "--gpus", "2")
    assert e.value.code == 2


def test_extra_legs(bench, monkeypatch, capsys):
    out, = _run(bench, monkeypatch, capsys, "--extra")
    x = out["extra"]
    assert set(x) == {"fused_forward", "sparse_16bit", "fixed_point_forward", "instruction_rates", "column_ranks_B2_T48_H2_W32"}
    for row in x["fused_forward"].values():
        assert row["max_rel_diff"] < 1e-5 and set(row["fwd_bwd"]) == {"fused", "fused_pipelined", "composed"}
    for row in x["sparse_16bit"].values():
        assert all(row[dt + leg] > 0 for dt in ("float32", "float16", "bfloat16") for leg in ("_fwd_ms", "_fwd_bwd_ms"))
    assert len(x["instruction_rates"]) == 4


def test_without_a_gpu_it_says_so(monkeypatch, capsys):
    import bench as b
    monkeypatch.setattr(sys, "argv", ["bench.py"])
    monkeypatch.setattr(torch.cuda, "is_available", lambda: False)
    with pytest.raises(SystemExit) as e:
        b.main()
    assert e.value.code == 3 and "no GPU" in capsys.readouterr().err
