#!/usr/bin/env python3
"""Benchmark of the L1-attention hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--skip-sparse] [--skip-cpu]
    python bench.py --sweep                     # the reference's own timing grid (benchmark.py:57-66), one JSON line per cell
    python bench.py --skip-dense --only config4 # one sparse configuration per process (profiling aid)
    python bench.py --extra                     # opt-in legs: fused operator, 16-bit rows, fixed-point forward

A step is one dense L1Attn forward + backward (through the reference's Python API,
l1attn_cuda.L1AttnFn) over the headline configuration  q,k fp32 [B=8, T=4096, H=16, W=64],
upstream gradient dA fp32 [8,4096,4096,16] ~ N(0,1), all resident in HBM before the timed region.
Prints ONE JSON line: dense fwd+bwd throughput in GOP/s (algorithmic operations: 2 per
pair-element forward, 4 backward, N = B*T*T*H*W pair-elements), the roofline of the dominant
launch (the backward), the sparse / bidirectional-sparse / expandCoo figures of configurations 4
and 5, and a CPU baseline timed on this box's host cores on a bounded sample of the same workload.
Progress goes to stderr.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
for _p in (ROOT, os.path.join(ROOT, "l1-attention_amd"), os.path.join(ROOT, "tests")):
    if _p not in sys.path:
        sys.path.insert(0, _p)

# Where and on what the legs run.  The sizes are the benchmark's definition; they are names here only so that a
# walk-through of this file without a GPU (tests/test_bench_dry_run_cpu.py) can shrink them.
DEVICE = "cuda:0"
HEADLINE = (8, 4096, 16, 64)          # B, T, H, W of the headline dense configuration
SECOND = (16, 1024, 8, 64)            # the second dense configuration (extra legs)
CONFIG4 = ((4, 4096, 8, 32), 64)      # sparse: B, T, H, W; degrees uniform in 1..64
CONFIG5 = (1, 65536, 4, 64)           # bidirectional sparse, power-law degrees and self loops
CPU_SAMPLE = (1, 1024, 16, 64)        # the dense sample the host baseline is timed on
COPY_FLOATS = 1 << 28                 # 1 GiB: the copy the HBM counters are calibrated on
SWEEP = {"B": 512, "H": 8, "T": (16, 32, 64, 128, 256), "W": (16, 32, 33, 64, 65, 96, 97, 128)}

P_VALU_TOPS = 78.6     # 256 CU x 4 SIMD x 32 fp32 lanes/clk x 2.4 GHz; the 157.3 TFLOP/s datasheet figure counts FMA as 2
HBM_PEAK_GBS = 8000.0  # MI355X HBM3E

# HBM bytes per dense-backward launch (B=8,T=4096,H=16,W=64) from rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE
# (profiles/dense_B8_T4096_H16_W64_pmc_*.txt), scaled by what three 1 GiB device copies read on the same
# counters (profiles/copy_1GiB_pmc_*.txt: FETCH_SIZE 0.5 per KiB -> x2.0, WRITE_SIZE 1.0 per KiB -> x1.0).
# (Counters collected before the later tiles' partial rows became L2 adds: the 6 GiB of them that the
# workgroups read back are now read by the L2 instead; the total is unchanged to first order.)
# KiB per kernel, fetch / write: column ranks 149986 / 262144, main kernel 10683411 / 8652097,
# column-sum reduce 65547 / 2048, dk reduce 1050658 / 131072.
DENSE_BWD_TRAFFIC_BYTES = ((149986 + 10683411 + 65547 + 1050658) * 2 + 262144 + 8652097 + 2048 + 131072) * 1024
# The figure above is NOT measured by the run that prints it: it is read off committed counter summaries.
DENSE_BWD_TRAFFIC_SOURCE = {
    "measured_in_this_run": False,
    "files": ["profiles/dense_B8_T4096_H16_W64_pmc_fetch_size.txt", "profiles/dense_B8_T4096_H16_W64_pmc_write_size.txt",
              "profiles/copy_1GiB_pmc_fetch_size.txt", "profiles/copy_1GiB_pmc_write_size.txt"],
    "collected_at_commit": "65a21ba",
    "kernel_state": "one change before the current backward kernel: the later dst tiles of a workgroup then loaded, "
                    "added and stored their dk partial rows; they now send adds to the L2 instead",
}


def log(*a):
    print(*a, file=sys.stderr, flush=True)


def _shape_name(shape):
    return "B%d_T%d_H%d_W%d" % tuple(shape)


def dense_headline(steps, warmup):
    import torch
    import l1attn_cuda
    B, T, H, W = HEADLINE
    dev = torch.device(DEVICE)
    import workloads
    q, k, _ = workloads.dense_inputs(B, T, H, W, seed=1002)
    q, k = q.to(dev).requires_grad_(), k.to(dev).requires_grad_()
    gen = torch.Generator(device=dev).manual_seed(1002)
    dA = torch.empty(B, T, T, H, device=dev)
    for b in range(B):  # 8 GiB, generated on the device one batch at a time
        dA[b].normal_(generator=gen)
    N = B * T * T * H * W

    def step(ev=None):
        q.grad = None
        k.grad = None
        if ev:
            ev[0].record()
        a = l1attn_cuda.L1AttnFn.apply(q, k)
        if ev:
            ev[1].record()
        a.backward(dA)
        if ev:
            ev[2].record()
        del a

    for _ in range(warmup):
        step()
    torch.cuda.synchronize()
    evs = [[torch.cuda.Event(enable_timing=True) for _ in range(3)] for _ in range(steps)]
    t0 = time.perf_counter()
    for i in range(steps):
        step(evs[i])
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    fwd_ms = sum(e[0].elapsed_time(e[1]) for e in evs) / steps
    bwd_ms = sum(e[1].elapsed_time(e[2]) for e in evs) / steps
    ms_per_step = wall * 1e3 / steps
    out = {
        "B": B, "T": T, "H": H, "W": W, "pair_elements": N,
        "fwd_ms": fwd_ms, "bwd_ms": bwd_ms, "ms_per_step": ms_per_step,
        "fwd_tops": 2 * N / fwd_ms / 1e9, "bwd_tops": 4 * N / bwd_ms / 1e9,
        "fwd_bwd_gops": 6 * N / (ms_per_step * 1e-3) / 1e9,
    }
    out["frac_of_valu_peak"] = out["fwd_bwd_gops"] / 1e3 / P_VALU_TOPS
    # which forms of the backward this process ran (--bwd-form / --rank-sort; the default entry point without them)
    import _l1attn_hip as drv
    info = drv.dense_backward_plan(B, T, H, W)
    out["backward_plan"] = {"rank_form": int(info[2]), "branch_free": int(info[3]), "tiles_per_workgroup": int(info[9]),
                            "step_loop_form": int(info[14]),
                            "rank_sort": "merge" if (info[2] and drv._dense_bwd_form[1]) else "radix"}
    del dA, q, k
    torch.cuda.empty_cache()
    return out


def time_gpu(fn, iters, warm=2):
    import torch
    for _ in range(warm):
        fn()
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(iters):
        fn()
    e1.record()
    torch.cuda.synchronize()
    return e0.elapsed_time(e1) / iters


def sparse_configs(skip_cpu, only=None):
    """Configuration 4 (one-directional, B4 T4096 H8 W32, degree U{1..64}) and configuration 5
    (bidirectional, B1 T65536 H4 W64, Zipf degrees + self loops): fwd+bwd through the Python API.
    `only`: "config4" or "config5" runs that one alone, so that a profile of the process holds one configuration's
    launches and its kernel times and HBM counters can be read per configuration."""
    import torch
    import workloads
    import l1attn_sparse_cuda as sp
    import l1attn_sparse_bidi_cuda as bi
    from oracle import oracle
    dev = torch.device(DEVICE)
    res = {}
    for name, bidi, (B, T, H, W), co in (
            ("config4_uni", False, CONFIG4[0], lambda: workloads.uniform_degree_graph(CONFIG4[0][1], CONFIG4[1], seed=1004)),
            ("config5_bidi", True, CONFIG5, lambda: workloads.powerlaw_graph(CONFIG5[1], seed=1005))):
        if only and not name.startswith(only):
            continue
        co = co() if callable(co) else co
        E = co.shape[0]
        cod = co.to(dev)
        ms_expand = time_gpu(lambda: sp.expandCoo(cod, warn=False), 3, warm=1)
        coo, dmx, smx = sp.expandCoo(cod, warn=False)
        cpu_expand_ms = None
        if not skip_cpu:
            t0 = time.perf_counter()
            ocoo, odmx, osmx = oracle.expand_coo(co)
            cpu_expand_ms = (time.perf_counter() - t0) * 1e3
            assert torch.equal(coo.cpu(), ocoo) and (dmx, smx) == (odmx, osmx)
        x = [t.to(dev).requires_grad_() for t in workloads.sparse_inputs(B, T, H, W, seed=1004 + bidi, n=4)]
        dvo = torch.randn(B, T, H, W, device=dev)
        if bidi:
            m = bi.L1AttnSparseBidi()
            args = (x[0], x[1], x[2], x[3])
        else:
            m = sp.L1AttnSparse()
            args = (x[0], x[2], x[3])

        def fwd():
            return m(*args, coo, dmx)

        def fwdbwd():
            for t in x:
                t.grad = None
            fwd().backward(dvo)

        ms_fwd = time_gpu(fwd, 10)
        ms = time_gpu(fwdbwd, 10)
        r, g = B * H * W * 4, B * H * 4
        if bidi:
            bytes_alg = E * (8 * r + 7 * g + 64) + T * 11 * r
        else:
            bytes_alg = E * (6 * r + 5 * g + 48) + T * 8 * r
        bytes_min = 11 * T * r + 16 * E + 2 * g * E
        res[name] = {
            "B": B, "T": T, "H": H, "W": W, "edges": E, "dst_mxlen": dmx, "src_mxlen": smx,
            "fwd_ms": ms_fwd, "fwd_bwd_ms": ms,
            "edges_per_s": E / (ms * 1e-3), "edge_heads_per_s": E * B * H / (ms * 1e-3),
            "bytes_alg": bytes_alg, "alg_GBps": bytes_alg / (ms * 1e-3) / 1e9,
            "frac_of_hbm_peak": bytes_alg / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS,
            "bytes_min": bytes_min, "min_GBps": bytes_min / (ms * 1e-3) / 1e9,
            "frac_of_hbm_peak_bytes_min": bytes_min / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS,
            "working_set_bytes": 11 * T * r,
            "where_the_rows_live": "the eleven [B,T,H,W] tensors of a fwd+bwd are %.0f MiB: they stay in the L2s / the "
                                   "256 MiB Infinity Cache between gathers, so alg_GBps is a cache-bandwidth figure "
                                   "of the gather model, not HBM traffic; HBM sees about bytes_min per fwd+bwd"
                                   % (11 * T * r / 2.0 ** 20),
            "expand_coo_gpu_ms": ms_expand, "expand_coo_cpu_oracle_ms": cpu_expand_ms,
            "note": "plan build (two radix sorts) is cached per edge list and excluded from fwd/bwd time",
        }
        log(name, json.dumps(res[name]))
    return res


def extra_legs():
    """Opt-in (--extra): the two additions beyond the reference's operators, timed beside what they replace.
    Fused forward (logits, softmax over src with the no-op logit, value sum in one kernel) against the same
    result composed from L1Attn and torch's cat / softmax / einsum, at the second baseline configuration and
    the headline shape; sparse and bidirectional operators with float16 / bfloat16 rows against float32 rows at
    configurations 4 and 5 (forward, and forward + backward).  Prints its own JSON line; the default run does not come here."""
    import torch
    import workloads
    import l1attn_cuda
    import l1attn_sparse_cuda as sp
    import l1attn_sparse_bidi_cuda as bi
    import _l1attn_hip as drv
    drv.enable_experimental("fused", "rows16", "fixed")  # these legs exist to time exactly those paths
    dev = torch.device(DEVICE)
    res = {"fused_forward": {}, "sparse_16bit": {}}
    for name, (B, T, H, W) in ((_shape_name(SECOND), SECOND), (_shape_name(HEADLINE), HEADLINE)):
        q, k, v = (x.to(dev) for x in workloads.dense_inputs(B, T, H, W, seed=1002, with_v=True))
        fused, plain = l1attn_cuda.L1AttnFused(), l1attn_cuda.L1Attn()

        def composed():
            a = plain(q, k)
            a = torch.cat((a, torch.zeros(B, 1, T, H, device=dev)), 1)
            return torch.einsum("bsdh,bshw->bdhw", torch.softmax(a, 1)[:, :T], v)

        ms_f = time_gpu(lambda: fused(q, k, v), 5)
        ms_fp = time_gpu(lambda: drv.dense_fused_forward(q, k, v, pipelined=True), 5)
        big = B * T * T * H * 4 > (4 << 30)  # the composition holds three [B,T,T,H] tensors at once
        ms_c = time_gpu(composed, 2 if big else 5, warm=1)
        err = float((fused(q, k, v) - composed()).abs().max() / composed().abs().max())
        N = B * T * T * H * W
        # forward + backward, and the peak memory each route adds to the inputs
        x = [t.clone().requires_grad_() for t in (q, k, v)]
        dvo = torch.randn_like(v)

        def train(fn):
            for t in x:
                t.grad = None
            fn().backward(dvo)

        def fused_step():
            train(lambda: fused(*x))

        fused_piped = l1attn_cuda.L1AttnFused(pipelined=True)

        def fused_piped_step():
            train(lambda: fused_piped(*x))

        def composed_step():
            def f():
                a = plain(x[0], x[1])
                a = torch.cat((a, torch.zeros(B, 1, T, H, device=dev)), 1)
                return torch.einsum("bsdh,bshw->bdhw", torch.softmax(a, 1)[:, :T], x[2])
            train(f)

        steps = {}
        for label, fn in (("fused", fused_step), ("fused_pipelined", fused_piped_step), ("composed", composed_step)):
            torch.cuda.empty_cache()
            torch.cuda.reset_peak_memory_stats()
            base = torch.cuda.memory_allocated()
            ms = time_gpu(fn, 2 if big else 5, warm=1)
            steps[label] = {"fwd_bwd_ms": ms, "peak_extra_GiB": (torch.cuda.max_memory_allocated() - base) / 2.0 ** 30}
        del x, dvo
        res["fused_forward"][name] = {
            "fused_ms": ms_f, "fused_pipelined_ms": ms_fp, "composed_ms": ms_c, "speedup": ms_c / ms_f, "max_rel_diff": err,
            "fwd_bwd": steps,
            "fused_tops": 3 * N / ms_f / 1e9, "frac_of_valu_peak": 3 * N / ms_f / 1e9 / P_VALU_TOPS,
            "note": "3 algorithmic ops per pair-element (sub, abs-accumulate, multiply-accumulate)"}
        log(name, json.dumps(res["fused_forward"][name]))
        del q, k, v
        torch.cuda.empty_cache()
    for name, bidi, (B, T, H, W), co in (
            ("config4_uni", False, CONFIG4[0], workloads.uniform_degree_graph(CONFIG4[0][1], CONFIG4[1], seed=1004)),
            ("config5_bidi", True, CONFIG5, workloads.powerlaw_graph(CONFIG5[1], seed=1005))):
        coo, dmx, smx = sp.expandCoo(co.to(dev), warn=False)
        x32 = [t.to(dev) for t in workloads.sparse_inputs(B, T, H, W, seed=1004 + bidi, n=4)]
        m = bi.L1AttnSparseBidi() if bidi else sp.L1AttnSparse()
        row = {"edges": int(co.shape[0])}
        for dt in (torch.float32, torch.float16, torch.bfloat16):
            x = [t.to(dt) for t in x32]
            args = (x[0], x[1], x[2], x[3]) if bidi else (x[0], x[2], x[3])
            name_dt = str(dt).split(".")[1]
            row[name_dt + "_fwd_ms"] = time_gpu(lambda: m(*args, coo, dmx), 10)
            leaves = [t.clone().requires_grad_() for t in args]
            dvo = torch.randn(B, T, H, W, device=dev).to(dt)

            def fwdbwd():
                for t in leaves:
                    t.grad = None
                m(*leaves, coo, dmx).backward(dvo)

            row[name_dt + "_fwd_bwd_ms"] = time_gpu(fwdbwd, 10)
        res["sparse_16bit"][name] = row
        log(name, json.dumps(row))
    res["fixed_point_forward"] = {}
    for name, (B, T, H, W) in ((_shape_name(SECOND), SECOND), (_shape_name(HEADLINE), HEADLINE)):
        q, k, _ = workloads.dense_inputs(B, T, H, W, seed=1002)
        q, k = q.to(dev), k.to(dev)
        ms32 = time_gpu(lambda: drv.dense_forward(q, k), 5)
        msfx = time_gpu(lambda: drv.dense_forward_fixed(q, k), 5)
        a32, afx = drv.dense_forward(q, k)[0], drv.dense_forward_fixed(q, k)[0]
        diff = float((a32[0] - afx[0]).abs().max() / a32[0].abs().max())
        N = B * T * T * H * W
        res["fixed_point_forward"][name] = {
            "fp32_ms": ms32, "fixed_ms": msfx, "fixed_tops_algorithmic": 2 * N / msfx / 1e9,
            "max_rel_diff_to_fp32_kernel_batch0": diff,
            "note": "fixed_ms includes the two conversion pre-passes and the workspace allocation"}
        log(name, json.dumps(res["fixed_point_forward"][name]))
        del q, k, a32, afx
        torch.cuda.empty_cache()
    res["instruction_rates"] = instruction_rates()
    # column ranks of the long-sequence backward: library block radix sort against the merge sort of rank_sort.hip
    B, T, H, W = HEADLINE
    q, k, _ = workloads.dense_inputs(B, T, H, W, seed=1002)
    q, k = q.to(dev), k.to(dev)
    rq, rk = torch.empty_like(q), torch.empty_like(k)
    L, st = drv.lib(), drv.stream_of(q)
    res["column_ranks_" + _shape_name(HEADLINE)] = {
        "library_radix_sort_ms": time_gpu(lambda: L.l1attn_dense_column_ranks_f32(
            drv.ptr(q), drv.ptr(k), drv.ptr(rq), drv.ptr(rk), B, T, H, W, st), 10),
        "merge_sort_ms": time_gpu(lambda: L.l1attn_dense_column_ranks_merge_f32(
            drv.ptr(q), drv.ptr(k), drv.ptr(rq), drv.ptr(rk), B, T, H, W, st), 10)}
    log(json.dumps(res["column_ranks_" + _shape_name(HEADLINE)]))
    return res


def instruction_rates():
    """Issue rates of candidate instructions from the library's register-only probe (256 workgroups of 8 waves),
    in wave-instructions per SIMD and nanosecond and as lane-operations per second."""
    import torch
    import _l1attn_hip as drv
    L = drv.lib()
    blocks, iters = 256, 4000
    out = torch.empty(blocks * 512, dtype=torch.float32, device=DEVICE)
    st = drv.stream_of(out)
    names = {0: "v_fmac_f32", 1: "v_sad_u32 (VGPR operands)", 2: "v_sad_u32 (SGPR operand)",
             3: "v_sub_f32 + v_add_f32 |x| (two instructions per step)"}
    rates = {}
    for op, name in names.items():
        assert L.l1attn_probe_valu_op(drv.ptr(out), blocks, 100, op, st) == 0
        torch.cuda.synchronize()
        ev = [torch.cuda.Event(enable_timing=True) for _ in range(2)]
        ev[0].record()
        assert L.l1attn_probe_valu_op(drv.ptr(out), blocks, iters, op, st) == 0
        ev[1].record()
        torch.cuda.synchronize()
        ms = ev[0].elapsed_time(ev[1])
        steps = blocks * 8 * iters * 64
        rates[name] = {"ms": ms, "steps_per_simd_ns": steps / (256 * 4) / (ms * 1e6),
                       "lane_steps_tops": steps * 64 / (ms * 1e-3) / 1e12}
    return rates


def _l1attn_hip_setting(name):
    import _l1attn_hip
    return getattr(_l1attn_hip, name)


def reference_sweep(num_runs=10):
    """The reference's own timing grid (benchmark.py:57-66): B=512, H=8, T in {16,...,256}, W in
    {16,32,33,64,65,96,97,128}, forward and backward of L1AttnFn timed separately as averages over num_runs.
    Differences from that script, on purpose: HIP events on the stream instead of perf_counter around
    synchronize (its numbers at these sizes are mostly launch and sync latency), inputs made once per cell,
    and each cell also reports algorithmic Tops/s.  One JSON line per cell on stdout, and the list as return value."""
    import torch
    import l1attn_cuda
    dev = torch.device(DEVICE)
    B, H = SWEEP["B"], SWEEP["H"]
    rows = []
    for T in SWEEP["T"]:
        for W in SWEEP["W"]:
            g = torch.Generator(device=dev).manual_seed(1000 + T * 1000 + W)
            q = torch.randn(B, T, H, W, device=dev, generator=g).requires_grad_()
            k = torch.randn(B, T, H, W, device=dev, generator=g).requires_grad_()
            dA = torch.randn(B, T, T, H, device=dev, generator=g)
            attn = l1attn_cuda.L1AttnFn.apply(q, k)
            attn.backward(dA)  # warm-up of both launches (workspace allocation, plan choice)
            torch.cuda.synchronize()
            ev = [[torch.cuda.Event(enable_timing=True) for _ in range(3)] for _ in range(num_runs)]
            for e in ev:
                q.grad = None
                k.grad = None
                e[0].record()
                attn = l1attn_cuda.L1AttnFn.apply(q, k)
                e[1].record()
                attn.backward(dA)
                e[2].record()
            torch.cuda.synchronize()
            fwd_ms = sum(e[0].elapsed_time(e[1]) for e in ev) / num_runs
            bwd_ms = sum(e[1].elapsed_time(e[2]) for e in ev) / num_runs
            N = B * T * T * H * W
            row = {"sweep": "benchmark.py:57-66", "batch_size": B, "seq_length": T, "n_heads": H, "width": W,
                   "avg_forward_ms": fwd_ms, "avg_backward_ms": bwd_ms,
                   "fwd_tops": 2 * N / fwd_ms / 1e9, "bwd_tops": 4 * N / bwd_ms / 1e9,
                   "sign_range_checked": not _l1attn_hip_setting("_assume_sign_range")}
            print(json.dumps(row), flush=True)
            rows.append(row)
            del q, k, dA, attn
    return rows


def valu_probe():
    """What ordinary (non-packed) fp32 VALU code sustains on this GPU: the library's register-only probe on
    256 workgroups of 8 waves (two waves per SIMD on every CU), HIP events on the current stream."""
    import torch
    import _l1attn_hip as drv
    L = drv.lib()
    blocks, iters = 256, 4000
    out = torch.empty(blocks * 512, dtype=torch.float32, device=DEVICE)
    st = drv.stream_of(out)
    assert L.l1attn_probe_valu(drv.ptr(out), blocks, 100, st) == 0
    torch.cuda.synchronize()
    ev = [torch.cuda.Event(enable_timing=True) for _ in range(2)]
    ev[0].record()
    assert L.l1attn_probe_valu(drv.ptr(out), blocks, iters, st) == 0
    ev[1].record()
    torch.cuda.synchronize()
    ms = ev[0].elapsed_time(ev[1])
    lane_ops = blocks * 8 * iters * 64 * 64
    tops = lane_ops / (ms * 1e-3) / 1e12
    return {"kernel": "probe_valu_loop (independent v_fmac_f32, registers only, 2 waves per SIMD)",
            "lane_tops": tops, "frac_of_nominal_peak": tops / P_VALU_TOPS, "ms": ms}


def cpu_baseline_sparse(mods, ncores):
    """Configuration 4 in full (B4 T4096 H8 W32, about 133 k edges) on the host: the reference's own CPU extension
    (float64, one thread; its softmax Jacobian loop is O(dst_mxlen^2) per token and head) when oracle/_ref is
    there, and this repository's CPU operator package (float32, all cores).  Forward + backward, edges per second."""
    import torch
    import workloads
    import _l1attn_cpu
    (B, T, H, W), max_degree = CONFIG4
    co = workloads.uniform_degree_graph(T, max_degree, seed=1004)
    coo, dmx, _ = _l1attn_cpu.expand_coo(co)
    v, _, q, k = workloads.sparse_inputs(B, T, H, W, seed=1004, n=4)
    dvo = torch.randn(B, T, H, W, generator=torch.Generator().manual_seed(1))
    E = int(co.shape[0])
    out = {"edges": E}
    _l1attn_cpu.set_threads(ncores)
    _l1attn_cpu.sparse_forward(v, q, k, coo, dmx, True)
    t0 = time.perf_counter()
    vo, attn = _l1attn_cpu.sparse_forward(v, q, k, coo, dmx, True)
    _l1attn_cpu.sparse_backward(dvo, v, q, k, coo, attn, dmx, True)
    dt = time.perf_counter() - t0
    _l1attn_cpu.set_threads(0)
    out["cpu_operator_package_fp32"] = {"fwd_bwd_ms": dt * 1e3, "edges_per_s": E / dt, "cores": ncores}
    if mods is not None:
        d = [x.double() for x in (v, q, k, dvo)]
        t0 = time.perf_counter()
        vo, attn = mods["l1attn_sparse_drv"].forward(d[0], d[1], d[2], coo, dmx, True)
        mods["l1attn_sparse_drv"].backward(d[3], d[0], d[1], d[2], coo, attn, dmx, True)
        dt = time.perf_counter() - t0
        out["reference_fp64"] = {"fwd_bwd_ms": dt * 1e3, "edges_per_s": E / dt, "cores": 1, "kind": "reference"}
    # Configuration 5 (bidirectional, B1 T65536 H4 W64, about 1.08 M edges, longest dst segment 2049) on the CPU
    # operator package only: the reference's extension would walk its O(dst_mxlen^2) softmax Jacobian loop
    # (cpp/l1attn_sparse_bidi_drv.cpp:176-190) 65536 * 4 * 2049^2 = 1.1e12 times and hold 4.3 GB of float64 padding.
    B, T, H, W = CONFIG5
    co = workloads.powerlaw_graph(T, seed=1005)
    coo, dmx, _ = _l1attn_cpu.expand_coo(co)
    vf, vb, q, k = workloads.sparse_inputs(B, T, H, W, seed=1005, n=4)
    dvo = torch.randn(B, T, H, W, generator=torch.Generator().manual_seed(1))
    _l1attn_cpu.set_threads(ncores)
    t0 = time.perf_counter()
    vo, attn = _l1attn_cpu.bidi_forward(vf, vb, q, k, coo, dmx, True)
    _l1attn_cpu.bidi_backward(dvo, vf, vb, q, k, coo, attn, dmx, True)
    dt = time.perf_counter() - t0
    _l1attn_cpu.set_threads(0)
    out["config5_bidi_cpu_operator_package_fp32"] = {
        "edges": int(co.shape[0]), "fwd_bwd_ms": dt * 1e3, "edges_per_s": int(co.shape[0]) / dt, "cores": ncores,
        "note": "the reference's CPU extension is not timed here: O(dst_mxlen^2) Jacobian loop, 1.1e12 iterations"}
    return out


def cpu_baseline():
    """The reference's own CPU extension (oracle/_ref, fp64, one thread, scalar) when it was built and
    carried here, else the C restatement (oracle/liboracle.so, fp64, one thread), on a bounded sample
    of the headline workload: same H, W and input distribution, B=1 and T=1024 (1/128 of the pair-elements)."""
    import torch
    import workloads
    from oracle import oracle
    B, T, H, W = CPU_SAMPLE
    q, k, _ = workloads.dense_inputs(B, T, H, W, seed=1002)
    q, k = q.double(), k.double()
    dA = torch.randn(B, T, T, H, generator=torch.Generator().manual_seed(1002), dtype=torch.float64)
    N = B * T * T * H * W
    mods = None
    try:
        mods = oracle.ref_modules()
    except Exception as e:  # an _ref built against another torch would fail to import
        log("oracle/_ref not usable:", repr(e))
    torch.set_num_threads(1)
    oracle.set_threads(1)
    if mods is not None:
        kind = "reference"
        t0 = time.perf_counter()
        mods["l1attn_drv_cpp"].forward(q, k)
        mods["l1attn_drv_cpp"].backward(dA, q, k)
        dt = time.perf_counter() - t0
    else:
        kind = "port"
        t0 = time.perf_counter()
        oracle.dense_fwd(q, k)
        oracle.dense_bwd(dA, q, k)
        dt = time.perf_counter() - t0
    # the same sample on all host cores with the OpenMP build of the restatement (fp32)
    ncores = min(os.cpu_count() or 1, 16)
    oracle.set_threads(ncores)
    q32, k32, dA32 = q.float(), k.float(), dA.float()
    t0 = time.perf_counter()
    oracle.dense_fwd(q32, k32)
    oracle.dense_bwd(dA32, q32, k32)
    dt_mt = time.perf_counter() - t0
    oracle.set_threads(1)
    # this repository's own CPU operator package (l1attn_cpp over libl1attn_cpu.so; product code, not the baseline)
    pkg = None
    try:
        import _l1attn_cpu
        _l1attn_cpu.set_threads(ncores)
        _l1attn_cpu.dense_forward(q32, k32)
        t0 = time.perf_counter()
        _l1attn_cpu.dense_forward(q32, k32)
        _l1attn_cpu.dense_backward(dA32, q32, k32)
        dt_pkg = time.perf_counter() - t0
        _l1attn_cpu.set_threads(0)
        pkg = {"value": 6 * N / dt_pkg / 1e9, "unit": "GOP/s", "cores": ncores,
               "note": "l1attn_cpp (the CPU twin of the operators, fp32, OpenMP), same sample"}
    except Exception as e:
        log("CPU operator package not timed:", repr(e))
    sparse = None
    try:
        sparse = cpu_baseline_sparse(mods, ncores)
    except Exception as e:  # noqa: BLE001
        log("sparse CPU baseline not timed:", repr(e))
    return {
        "sparse": sparse,
        "cpu_operator_package_fp32": pkg,
        "value": 6 * N / dt / 1e9, "unit": "GOP/s", "cores": 1, "kind": kind,
        "sample": "dense fwd+bwd fp64, B=%d T=%d H=%d W=%d (1/%d of the headline pair-elements), %.1f s"
                  % (B, T, H, W, round(HEADLINE[0] * HEADLINE[1] ** 2 * HEADLINE[2] * HEADLINE[3] / N), dt),
        "port_fp32_openmp": {"value": 6 * N / dt_mt / 1e9, "unit": "GOP/s", "cores": ncores,
                             "note": "OpenMP over (batch, head) of the C restatement"},
    }


def _guarded(fn):
    try:
        return fn()
    except Exception as e:  # noqa: BLE001
        log("side measurement failed:", repr(e))
        return {"error": repr(e)}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=5)
    ap.add_argument("--warmup", type=int, default=2)
    ap.add_argument("--skip-sparse", action="store_true")
    ap.add_argument("--skip-cpu", action="store_true")
    ap.add_argument("--skip-dense", action="store_true", help="profiling aid: sparse legs only")
    ap.add_argument("--only", choices=("config4", "config5"), default=None,
                    help="with the sparse legs: run this configuration alone (one per process for profiles)")
    ap.add_argument("--sweep", action="store_true",
                    help="only run the reference's timing grid (benchmark.py:57-66), one JSON line per cell")
    ap.add_argument("--extra", action="store_true",
                    help="only time the fused forward and the 16-bit sparse forwards beside what they replace")
    ap.add_argument("--bwd-form", type=int, choices=(0, 1, 2), default=0,
                    help="A/B aid: step loop of the long-sequence dense backward (0 = the default entry point)")
    ap.add_argument("--rank-sort", choices=("radix", "merge"), default="radix",
                    help="A/B aid: sort behind the dense backward's column ranks (radix = the default entry point)")
    ap.add_argument("--assume-sign-range", action="store_true",
                    help="A/B aid: leave out the dense backward's sign-range check (the caller vouches for q and k); "
                         "matters for the short sequences of --sweep")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="profiling aid: only run three 1 GiB device-to-device copies, the known-size "
                         "kernel that rocprofv3 FETCH_SIZE / WRITE_SIZE readings are scaled by")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build measures one GPU only (the hot path does not communicate: batches and "
              "heads are independent, so more GPUs would each take a share of them); run with --gpus 1",
              file=sys.stderr)
        sys.exit(2)
    import torch
    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        sys.exit(3)
    import _l1attn_hip
    _l1attn_hip.lib()  # fail here, loudly, if the HIP library is not built
    if args.assume_sign_range:
        _l1attn_hip.assume_sign_range(True)
    if args.bwd_form or args.rank_sort == "merge":
        _l1attn_hip.enable_experimental(*([("bwd_pipe")] if args.bwd_form else []),
                                        *([("rank_merge")] if args.rank_sort == "merge" else []))
        _l1attn_hip.set_dense_backward_form(args.bwd_form, int(args.rank_sort == "merge"))

    if args.copy_calibration:
        src = torch.empty(COPY_FLOATS, dtype=torch.float32, device=DEVICE).normal_()
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)
        torch.cuda.synchronize()
        print(json.dumps({"copy_calibration_bytes_read": src.numel() * 4, "bytes_written": src.numel() * 4, "copies": 3}))
        return
    if args.skip_dense:
        print(json.dumps({"sparse": sparse_configs(True, args.only)}), flush=True)
        return
    if args.sweep:
        reference_sweep()
        return
    if args.extra:
        print(json.dumps({"extra": extra_legs()}), flush=True)
        return

    log("dense headline ...")
    d = dense_headline(args.steps, args.warmup)
    log(json.dumps(d))
    N = d["pair_elements"]
    roof = {
        "bound": "valu", "kernel": "dense_bwd_f32_fast (+ dense_column_ranks, dense_bwd_reduce_colsum, dense_bwd_reduce_dk: one backward launch)",
        "achieved": d["bwd_tops"], "peak": P_VALU_TOPS, "unit": "TFLOP/s",
        "frac": d["bwd_tops"] / P_VALU_TOPS,
        "traffic": DENSE_BWD_TRAFFIC_BYTES, "traffic_source": DENSE_BWD_TRAFFIC_SOURCE,
        "frac_of_datasheet_fp32": d["bwd_tops"] / 157.3,
        "flops_per_launch": 4 * N, "avg_launch_ms": d["bwd_ms"],
        "note": "algorithmic ops (4 per pair-element) over the HIP-event time of the backward launch; "
                "peak = nominal fp32 VALU issue rate (one wave64 instruction per SIMD every 2 cycles at "
                "2.4 GHz); traffic = HBM bytes of the launch against 8.5 GiB algorithmic (dA once + q,k,dq,dk): "
                "the rest is the dk partials (written and re-read by the four dst tiles of a workgroup, read by "
                "the reduction) and dA lines fetched by both column halves",
    }
    out = {
        "metric": "dense fwd+bwd GOP/s & % fp32 VALU peak; sparse fwd+bwd edges/s & HBM GB/s",
        "value": d["fwd_bwd_gops"], "unit": "GOP/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": d["ms_per_step"],
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f32", "data": "synthetic",
        "config": {"workload": "dense L1Attn fwd+bwd, q,k fp32 [B=%d,T=%d,H=%d,W=%d], dA [%d,%d,%d,%d] "
                               "(BASELINE.json configs[2], the headline dense configuration)"
                               % (d["B"], d["T"], d["H"], d["W"], d["B"], d["T"], d["T"], d["H"]),
                   "B": d["B"], "T": d["T"], "H": d["H"], "W": d["W"]},
        "frac_of_fp32_valu_peak": d["frac_of_valu_peak"],
        "valu_probe": _guarded(valu_probe),
        "dense": d,
        "roofline": roof,
    }
    # The headline figures above are complete; a failure in a side leg is reported inside the line instead of
    # taking the line with it.
    if not args.skip_sparse:
        log("sparse configurations ...")
        try:
            out["sparse"] = sparse_configs(args.skip_cpu, args.only)
        except Exception as e:  # noqa: BLE001
            import traceback
            log(traceback.format_exc())
            out["sparse"] = {"error": repr(e)}
    if not args.skip_cpu:
        log("cpu baseline ...")
        try:
            out["cpu_baseline"] = cpu_baseline()
        except Exception as e:  # noqa: BLE001
            import traceback
            log(traceback.format_exc())
            out["cpu_baseline"] = {"error": repr(e)}
    else:
        out["cpu_baseline"] = None
    print(json.dumps(out), flush=True)


if __name__ == "__main__":
    main()
