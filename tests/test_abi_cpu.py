"""CPU-only checks of the C ABI: the library loads, exports every function include/l1attn_hip.h
declares, and its host-side argument logic (no kernel launch) behaves as documented."""
import ctypes
import os
import re
import subprocess
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "l1attn_hip.h")
LIB = os.path.join(ROOT, "l1-attention_amd", "libl1attn_hip.so")


def _declared():
    src = open(HEADER).read()
    src = re.sub(r"/\*.*?\*/", "", src, flags=re.S)
    return sorted(set(re.findall(r"\b(l1attn_[a-z0-9_]+)\s*\(", src)))


@pytest.fixture(scope="module")
def lib():
    if not os.path.exists(LIB):
        import sys
        sys.path.insert(0, os.path.join(ROOT, "l1-attention_amd"))
        import build
        build.build()
    return ctypes.CDLL(LIB)


def test_every_declared_symbol_is_exported(lib):
    names = _declared()
    assert len(names) >= 20 and "l1attn_dense_fwd_f32" in names and "l1attn_expand_coo" in names
    for n in names:
        assert hasattr(lib, n), n


def test_header_compiles_as_c():
    import subprocess, tempfile
    with tempfile.TemporaryDirectory() as d:
        src = os.path.join(d, "t.c")
        open(src, "w").write('#include "l1attn_hip.h"\nint main(void){return L1ATTN_OK;}\n')
        subprocess.run(["gcc", "-std=c99", "-Wall", "-Werror", "-I", os.path.join(ROOT, "include"), "-c", src,
                        "-o", os.path.join(d, "t.o")], check=True)


def test_host_side_argument_logic(lib):
    i64, sz, vp = ctypes.c_int64, ctypes.c_size_t, ctypes.c_void_p
    assert lib.l1attn_version() >= 100
    lib.l1attn_dense_bwd_workspace_bytes.restype = sz
    lib.l1attn_dense_bwd_workspace_bytes.argtypes = [i64] * 4
    # one dst tile (T <= 32) needs the 256 bytes of the sign-domain flag only, the generic path no workspace
    assert lib.l1attn_dense_bwd_workspace_bytes(2, 32, 4, 32) == 256
    assert lib.l1attn_dense_bwd_workspace_bytes(2, 3, 16, 7) == 0
    # second baseline configuration (no column ranks): the flag, then 16 dk partials [T][HW] for each of the 16 batches
    assert lib.l1attn_dense_bwd_workspace_bytes(16, 1024, 8, 64) == 256 + 16 * 16 * 1024 * 512 * 4
    # headline config (column ranks, no flag): 64 dst tiles (64 tokens each) x 8 batches x T x H*W floats
    # per batch: 16 dk partials [T][HW] (64 dst tiles, four per workgroup), the two rank arrays [T][HW],
    # 64 + 1 column-sum arrays [T][H]
    assert lib.l1attn_dense_bwd_workspace_bytes(8, 4096, 16, 64) == 8 * 4 * ((16 + 2) * 4096 * 1024 + 65 * 4096 * 16)
    lib.l1attn_dense_fwd_f32.argtypes = [vp, vp, vp, i64, i64, i64, i64, vp]
    assert lib.l1attn_dense_fwd_f32(None, None, None, 1, 4, 2, 8, None) == -1      # null pointers
    assert lib.l1attn_dense_fwd_f32(None, None, None, 0, 4, 2, 8, None) == 0       # empty batch: nothing to do
    assert lib.l1attn_dense_fwd_f32(None, None, None, 1, 4, 2, -8, None) == -1     # negative size
    for n in ("l1attn_sparse_plan_bytes", "l1attn_sparse_plan_workspace_bytes"):
        getattr(lib, n).restype = sz
        getattr(lib, n).argtypes = [i64, i64]
    small, big = lib.l1attn_sparse_plan_bytes(10, 8), lib.l1attn_sparse_plan_bytes(100000, 4096)
    assert 0 < small < big and small % 256 == 0 and big % 256 == 0
    assert lib.l1attn_sparse_plan_workspace_bytes(100000, 4096) >= 7 * 100000 * 4  # 3 row arrays + 4 sort buffers
    lib.l1attn_expand_coo.argtypes = [vp, ctypes.c_int, i64, i64, vp, vp, vp, sz, vp]
    mx = (ctypes.c_int32 * 2)(7, 7)
    assert lib.l1attn_expand_coo(None, 64, 2, 0, None, mx, None, 0, None) == 0 and list(mx) == [1, 1]
    assert lib.l1attn_expand_coo(None, 16, 2, 5, None, mx, None, 0, None) == -1    # unsupported index width
    assert lib.l1attn_expand_coo(None, 64, 2, 5, None, mx, None, 0, None) == -1    # null list


def _plan(lib, B, T, H, W):
    lib.l1attn_dense_bwd_plan_info.argtypes = [ctypes.c_int64] * 4 + [ctypes.c_void_p]
    a = (ctypes.c_int64 * 16)()
    assert lib.l1attn_dense_bwd_plan_info(B, T, H, W, a) == 0
    keys = ("tiled", "wide", "rank", "branch_free", "threads", "n_cc", "n_tt", "tt_rows", "per", "group", "n_groups",
            "lds_bytes", "per_batch_bytes", "batches_per_launch", "deep", "flag_bytes")
    return dict(zip(keys, list(a)))


def test_dense_backward_plan_of_the_baseline_configurations(lib):
    """How the three dense configurations of BASELINE.json are tiled (host logic only, no GPU)."""
    c1 = _plan(lib, 2, 64, 4, 32)
    assert c1["tiled"] and not c1["wide"] and not c1["rank"] and (c1["tt_rows"], c1["n_tt"], c1["threads"]) == (32, 2, 128)
    c2 = _plan(lib, 16, 1024, 8, 64)
    assert c2["wide"] and not c2["rank"] and c2["branch_free"]            # T < 2048: sign from the scaled difference
    assert (c2["threads"], c2["n_cc"], c2["tt_rows"], c2["n_tt"], c2["group"]) == (512, 1, 64, 16, 1)  # 256 workgroups
    c3 = _plan(lib, 8, 4096, 16, 64)
    assert c3["wide"] and c3["rank"] and c3["branch_free"]
    assert (c3["threads"], c3["n_cc"], c3["tt_rows"], c3["n_tt"], c3["group"], c3["n_groups"]) == (512, 2, 64, 64, 4, 16)
    assert c3["batches_per_launch"] == 8 and c3["per"] == 4 and c3["lds_bytes"] == 4 * 8 * 68 * 4
    assert not (c1["deep"] or c2["deep"] or c3["deep"])                     # one step of prefetch distance unless asked
    # untiled shapes and empty problems
    assert not _plan(lib, 2, 3, 16, 7)["tiled"]
    assert _plan(lib, 0, 64, 4, 32) == {k: 0 for k in c1}
    a = (ctypes.c_int64 * 16)()
    assert lib.l1attn_dense_bwd_plan_info(1, -4, 2, 8, a) == -1 and lib.l1attn_dense_bwd_plan_info(1, 4, 2, 8, None) == -1


def test_dense_backward_plan_invariants_over_a_shape_grid(lib):
    """Every plan the host logic can produce on a grid of shapes must cover the problem exactly once and
    respect what the kernels assume (threads, LDS, staged values, tile grouping, workspace size)."""
    lib.l1attn_dense_bwd_workspace_bytes.restype = ctypes.c_size_t
    lib.l1attn_dense_bwd_workspace_bytes.argtypes = [ctypes.c_int64] * 4
    cdiv = lambda a, b: -(-a // b)
    seen = set()
    for B in (1, 2, 3, 8, 16, 33):
        for T in (16, 17, 64, 100, 512, 1000, 1024, 1536, 2048, 2100, 3000, 4096, 8192, 8200):
            for H in (1, 2, 3, 4, 8, 12, 16, 32):
                for W in (7, 16, 32, 33, 64, 96, 128):
                    p = _plan(lib, B, T, H, W)
                    HW = H * W
                    if not p["tiled"]:
                        assert T < 16 or HW < 32 or lib.l1attn_dense_bwd_workspace_bytes(B, T, H, W) == 0
                        continue
                    seen.add((p["wide"], p["rank"], p["branch_free"], p["group"] > 1))
                    th = p["threads"]
                    assert th % 64 == 0 and 64 <= th <= (512 if p["wide"] else 1024)
                    assert (p["n_cc"] - 1) * th < HW <= p["n_cc"] * th
                    assert p["n_tt"] == cdiv(T, p["tt_rows"]) and p["n_groups"] == cdiv(p["n_tt"], p["group"])
                    assert p["tt_rows"] in ((64, 72, 80, 88) if p["wide"] else (32,))
                    assert 0 < p["lds_bytes"] <= 64 * 1024 and 1 <= p["per"] <= (8 if p["wide"] else 16)
                    heads = max(min(HW, (c + 1) * th) // W - (c * th) // W + (1 if min(HW, (c + 1) * th) % W else 0)
                                for c in range(p["n_cc"]))
                    assert p["per"] * th >= 4 * p["tt_rows"] * heads          # every staged value has a thread
                    assert p["lds_bytes"] == 4 * heads * (p["tt_rows"] + 4) * 4
                    if p["rank"]:
                        assert p["wide"] and 2048 <= T <= 8192 and p["tt_rows"] <= 80 and 4 * heads * 16 <= th
                    if p["group"] > 1:
                        assert p["wide"] and p["tt_rows"] == 64 and p["per"] <= (4 if p["rank"] else 8)
                        assert p["branch_free"]                               # grouped tiles only in the branch-free form
                        assert B * p["n_cc"] * p["n_groups"] >= 256 * (512 // th)
                    if p["branch_free"]:
                        assert p["wide"] and p["tt_rows"] == 64 and T % 64 == 0 and HW % th == 0 and W == 64 and p["per"] == 4
                    partial = p["n_groups"] * T * HW * 4 if p["n_tt"] > 1 else 0
                    ranks = (2 * T * HW + (p["n_tt"] + 1) * T * H) * 4 if p["rank"] else 0
                    assert p["per_batch_bytes"] == partial + ranks
                    nb = min(B, cdiv(1024, p["n_groups"] * p["n_cc"])) if p["per_batch_bytes"] else B
                    assert p["batches_per_launch"] == nb
                    assert p["flag_bytes"] == (0 if p["rank"] else 256)       # the scaled-difference sign keeps a flag
                    assert lib.l1attn_dense_bwd_workspace_bytes(B, T, H, W) == p["flag_bytes"] + p["per_batch_bytes"] * nb
    # the grid reaches every family of instantiations: narrow, wide, ranks, branch-free, grouped
    assert (0, 0, 0, False) in seen and (1, 0, 0, False) in seen and (1, 1, 0, False) in seen
    assert (1, 1, 1, True) in seen and (1, 0, 1, True) in seen and (1, 1, 1, False) in seen and (1, 0, 1, False) in seen
    assert not any(grouped and not bf for (_, _, bf, grouped) in seen)


def test_dense_forward_workspace_follows_the_width(lib):
    """The forward needs scratch only for widths the tiled kernels cannot read directly: two zero-padded
    copies [B,T,H,WP] with WP the next multiple of 16 (128 above 96); nothing for multiples of 16, for
    widths above 128 or sequences below 32 tokens (generic kernels)."""
    lib.l1attn_dense_fwd_workspace_bytes.restype = ctypes.c_size_t
    lib.l1attn_dense_fwd_workspace_bytes.argtypes = [ctypes.c_int64] * 4
    B, T, H = 3, 100, 5
    for W, WP in [(16, 0), (32, 0), (64, 0), (96, 0), (128, 0), (1, 16), (7, 16), (17, 32), (33, 48), (65, 80), (81, 96),
                  (95, 96), (97, 128), (112, 0), (113, 128), (127, 128), (129, 0), (200, 0)]:
        assert lib.l1attn_dense_fwd_workspace_bytes(B, T, H, W) == 2 * B * T * H * WP * 4, W
    assert lib.l1attn_dense_fwd_workspace_bytes(B, 31, H, 33) == 0
    assert lib.l1attn_dense_fwd_workspace_bytes(0, T, H, 33) == 0 and lib.l1attn_dense_fwd_workspace_bytes(B, T, H, -1) == 0


def test_operator_modules_fail_loudly_without_library(monkeypatch):
    """No CPU or eager fallback: with the library missing the binding raises at first use."""
    import sys
    sys.path.insert(0, os.path.join(ROOT, "l1-attention_amd"))
    import _l1attn_hip as drv
    monkeypatch.setattr(drv, "_lib", None)
    monkeypatch.setattr(drv, "_LIB_PATH", os.path.join(ROOT, "does-not-exist.so"))
    with pytest.raises(RuntimeError, match="not built"):
        drv.lib()


def test_binding_rejects_cpu_tensors():
    import sys
    import torch
    sys.path.insert(0, os.path.join(ROOT, "l1-attention_amd"))
    import _l1attn_hip as drv
    q = torch.randn(1, 4, 2, 8)
    with pytest.raises(RuntimeError, match="q must be a CUDA tensor"):
        drv.dense_forward(q, q)
    with pytest.raises(RuntimeError, match="d_attn must be a CUDA tensor"):
        drv.dense_backward(torch.randn(1, 4, 4, 2), q, q)


def test_build_rejects_sgprs_touched_under_a_scalar_load_in_flight():
    """build.py's ISA check of the software-pipelined forward kernels: an SGPR spill between an
    inline-asm s_load and its wait must fail the build (such code faults on the GPU)."""
    import sys
    sys.path.insert(0, os.path.join(ROOT, "l1-attention_amd"))
    import build
    good = """
_ZN1_18dense_fwd_f32_pipeILi64EEEv: ; @k
	s_load_dwordx16 s[36:51], s[0:1], 0x0
	v_subrev_f32_e32 v1, s4, v2
	s_waitcnt lgkmcnt(0)
	v_subrev_f32_e32 v1, s36, v2
	s_endpgm
"""
    assert build.check_scalar_prefetch(good) == 1
    for bad_line in ("v_writelane_b32 v88, s40, 3", "v_readlane_b32 s51, v90, 11", "s_mov_b32 s36, s2",
                     "v_subrev_f32_e32 v1, s37, v2"):
        bad = good.replace("	v_subrev_f32_e32 v1, s4, v2", "	" + bad_line)
        with pytest.raises(RuntimeError, match="in flight"):
            build.check_scalar_prefetch(bad)
    with pytest.raises(RuntimeError, match="in flight"):
        build.check_scalar_prefetch(good.replace("	s_waitcnt lgkmcnt(0)\n", ""))
    # every kernel of a listing is walked, whatever its name; a set of names narrows the walk
    other = good.replace("dense_fwd_f32_pipe", "other_kernel")
    assert build.check_scalar_prefetch(other) == 1
    assert build.check_scalar_prefetch(other, {"_ZN1_18dense_fwd_f32_pipeILi64EEEv"}) == 0
    with pytest.raises(RuntimeError, match="in flight"):
        build.check_scalar_prefetch(other.replace("	v_subrev_f32_e32 v1, s4, v2", "	s_mov_b32 s36, s2"))


def test_scalar_prefetch_check_follows_branches_and_back_edges():
    """The in-flight SGPR set is carried along every branch edge to a fixed point: violations that only exist on a
    path through a loop's back edge, or in a block laid out after the exit, fail the build; a correct software
    pipeline (load in the latch, wait at the loop header) passes."""
    import sys
    sys.path.insert(0, os.path.join(ROOT, "l1-attention_amd"))
    import build
    pipeline = """
_Z4pipev: ; @k
	s_load_dwordx2 s[0:1], s[4:5], 0x0
	s_waitcnt lgkmcnt(0)
	s_load_dwordx4 s[8:11], s[0:1], 0x0
.LBB0_1:
	HEADER
	s_waitcnt lgkmcnt(0)
	v_add_f32_e32 v1, s8, v1
	s_mov_b32 s20, s9
	s_add_u32 s0, s0, 16
	s_load_dwordx4 s[8:11], s[0:1], 0x0
	s_cmp_lt_u32 s0, s12
	s_cbranch_scc1 .LBB0_1
	s_waitcnt lgkmcnt(0)
	s_endpgm
.Lfunc_end0:
"""
    good = pipeline.replace("	HEADER\n", "	v_mov_b32_e32 v2, s20\n")
    assert build.check_scalar_prefetch(good) == 3
    # a copy at the loop header of a register the latch loads: clean on the way in, in flight on the back edge
    for touch in ("s_mov_b32 s21, s8", "v_mov_b32_e32 v2, s11", "s_mov_b32 s10, 0"):
        with pytest.raises(RuntimeError, match="in flight.*\n.*" + re.escape(touch)):
            build.check_scalar_prefetch(pipeline.replace("HEADER", touch))
    # a second load into registers whose first load has not been waited for
    with pytest.raises(RuntimeError, match="in flight"):
        build.check_scalar_prefetch(pipeline.replace("HEADER", "s_load_dword s9, s[0:1], 0x40"))
    # the exit leaves the loop without its wait
    with pytest.raises(RuntimeError, match="s_endpgm with scalar loads in flight"):
        build.check_scalar_prefetch(good.replace("	s_waitcnt lgkmcnt(0)\n	s_endpgm", "	s_endpgm"))
    # the latch laid out after the exit: the header is reached from it by s_branch only
    rotated = """
_Z3rotv: ; @k
	s_load_dwordx2 s[0:1], s[4:5], 0x0
	s_waitcnt lgkmcnt(0)
	s_load_dwordx4 s[8:11], s[0:1], 0x0
	s_waitcnt lgkmcnt(0)
.LBB0_1:
	HEADER
	v_add_f32_e32 v1, s8, v1
	s_cmp_lt_u32 s0, s12
	s_cbranch_scc1 .LBB0_3
	s_endpgm
.LBB0_3:
	s_add_u32 s0, s0, 16
	s_load_dwordx4 s[8:11], s[0:1], 0x0
	s_branch .LBB0_1
.Lfunc_end0:
"""
    assert build.check_scalar_prefetch(rotated.replace("HEADER", "s_waitcnt lgkmcnt(0)")) == 3
    with pytest.raises(RuntimeError, match="in flight.*\n.*line 9: v_add_f32_e32 v1, s8, v1"):
        build.check_scalar_prefetch(rotated.replace("HEADER", "s_nop 0"))
    # a wait on one arm of a branch does not cover the other arm
    arms = """
_Z4armsv: ; @k
	s_load_dwordx2 s[2:3], s[4:5], 0x0
	s_cbranch_scc1 .LBB0_2
	s_waitcnt lgkmcnt(0)
.LBB0_2:
	s_mov_b32 s6, s2
	s_waitcnt lgkmcnt(0)
	s_endpgm
.Lfunc_end0:
"""
    with pytest.raises(RuntimeError, match="s_mov_b32 s6, s2"):
        build.check_scalar_prefetch(arms)
    assert build.check_scalar_prefetch(arms.replace("	s_cbranch_scc1 .LBB0_2\n	s_waitcnt", "	s_waitcnt lgkmcnt(0)\n	s_cbranch_scc1 .LBB0_2\n	s_waitcnt")) == 1
    with pytest.raises(RuntimeError, match="unknown label"):
        build.check_scalar_prefetch(arms.replace(".LBB0_2:", ".LBB0_9:"))
    # code no path reaches is not counted
    assert build.check_scalar_prefetch(arms.replace("	s_cbranch_scc1 .LBB0_2\n", "	s_waitcnt lgkmcnt(0)\n	s_endpgm\n")) == 1


def test_build_rejects_untracked_loads_in_inline_asm():
    """Loads whose result arrives later may not be issued from inline asm, in any kernel of any source: the
    compiler does not know the destination registers are still being written (a launch built that way took a GPU
    memory fault).  Checked on the listing (between the compiler's ASMSTART/ASMEND marks) and on the sources;
    scalar loads are allowed in the one helper and then verified instruction by instruction."""
    import sys
    sys.path.insert(0, os.path.join(ROOT, "l1-attention_amd"))
    import build
    listing = """
_Z5kern1v: ; @k
	buffer_load_dword v1, v0, s[0:3], 0 offen
	;;#ASMSTART
	v_fmac_f32 v1, v2, v3
	;;#ASMEND
	s_endpgm
_Z5kern2v: ; @k
	;;#ASMSTART
	s_load_dwordx16 s[36:51], s[0:1], 0x0
	;;#ASMEND
	;;#ASMSTART
	s_waitcnt lgkmcnt(0)
	;;#ASMEND
	s_endpgm
"""
    assert build.check_inline_asm_loads(listing) == {"_Z5kern2v"}
    for bad in ("buffer_load_dword v4, v0, s[0:3], 0 offen", "global_load_dwordx4 v[4:7], v[0:1], off",
                "flat_load_dword v4, v[0:1]", "ds_read_b128 v[4:7], v0", "scratch_load_dword v4, off, s0",
                "global_atomic_add_rtn_u32 v4, v[0:1], v2, off", "buffer_atomic_add_f32 v1, v0, s[0:3], 0 offen"):
        with pytest.raises(RuntimeError, match="does not track"):
            build.check_inline_asm_loads(listing.replace("	v_fmac_f32 v1, v2, v3", "	" + bad), "x.hip")
    # the shipped sources obey the rule; a second scalar-load site, or a vector load, in any file does not
    assert build.check_asm_sources() >= 10
    ok = {"sload.h": 'void sload32(int& a, const float* p)\n{\n\tasm volatile("s_load_dword %0, %1, 0x0" : "=&s"(a) : "s"(p));\n}\n'}
    assert build.check_asm_sources(ok) == 1
    with pytest.raises(RuntimeError, match="outside sload32"):
        build.check_asm_sources({"sparse.hip": ok["sload.h"]})
    with pytest.raises(RuntimeError, match="outside sload32"):
        build.check_asm_sources({"sload.h": ok["sload.h"].replace("sload32", "other")})
    with pytest.raises(RuntimeError, match="issues buffer_load_dword"):
        build.check_asm_sources({"dense.hip": 'void f()\n{\n\tasm volatile("v_nop\\n\\tbuffer_load_dword %0, %1, %2, 0 offen" : "=v"(x) : "v"(o), "s"(r));\n}\n'})
    with pytest.raises(RuntimeError, match="issues global_load_dword"):
        build.check_asm_sources({"coo.hip": 'void f()\n{\n\t__asm__ __volatile__("global_load_dword %0, %1, off" : "=v"(x) : "v"(a));\n}\n'})
    with pytest.raises(RuntimeError, match="issues ds_read_b32"):
        build.check_asm_sources({"fused.hip": 'void f()\n{\n\tasm("ds_read_b32 %0, %1" : "=v"(x) : "v"(o));\n}\n'})


def test_build_runs_where_the_forbidden_instruction_list_does_not_travel(monkeypatch, capsys, tmp_path):
    """isa_checks.py names instructions and stays on the build machine; build() must still import and run its
    other checks without it.  hipcc is replaced by a stand-in that fails at once, so only the start is walked."""
    import builtins
    import sys
    sys.path.insert(0, os.path.join(ROOT, "l1-attention_amd"))
    import build
    real_import = builtins.__import__

    def no_isa_checks(name, *a, **kw):
        if name == "isa_checks":
            raise ImportError("No module named 'isa_checks'")
        return real_import(name, *a, **kw)
    monkeypatch.delitem(sys.modules, "isa_checks", raising=False)
    monkeypatch.setattr(builtins, "__import__", no_isa_checks)
    monkeypatch.setenv("HIPCC", "/bin/false")
    # a failed build removes the library it would have replaced: point it at a stand-in file, not the real one
    stale = tmp_path / "libl1attn_hip.so"
    stale.write_bytes(b"left over from an earlier build")
    monkeypatch.setattr(build, "LIB", str(stale))
    with pytest.raises(RuntimeError, match="hipcc failed"):
        build.build()
    assert "forbidden instructions is skipped" in capsys.readouterr().err
    assert not stale.exists()


def test_build_rejects_spills_in_the_hot_kernels():
    """build.py reads registers and scratch of every dense kernel from the code-object metadata and fails
    the build when a kernel of the headline path spills; the table of the last build is kept beside the
    objects."""
    import sys
    sys.path.insert(0, os.path.join(ROOT, "l1-attention_amd"))
    import build
    meta = """
amdhsa.kernels:
  - .args:
      - .offset: 0
    .group_segment_fixed_size: 40960
    .name:           _ZN1_18dense_fwd_f32_pipeILi64EEEv
    .private_segment_fixed_size: 0
    .sgpr_count:     100
    .sgpr_spill_count: 1
    .vgpr_count:     95
    .vgpr_spill_count: 0
  - .args:           []
    .group_segment_fixed_size: 0
    .name:           other_kernel
    .private_segment_fixed_size: 344
    .sgpr_count:     20
    .vgpr_count:     128
    .vgpr_spill_count: 12
amdhsa.target:   amdgcn-amd-amdhsa--gfx950
"""
    res = build.kernel_resources(meta)
    assert res["_ZN1_18dense_fwd_f32_pipeILi64EEEv"] == {"lds_bytes": 40960, "scratch_bytes": 0, "sgpr": 100,
                                                         "sgpr_spills": 1, "vgpr": 95, "vgpr_spills": 0}
    assert res["other_kernel"]["scratch_bytes"] == 344 and res["other_kernel"]["vgpr_spills"] == 12
    full = {"k_dense_fwd_f32_pipeILi64E": dict(vgpr=95, scratch_bytes=0, vgpr_spills=0),
            "k_dense_fwd_f32_pipeILi32E": dict(vgpr=70, scratch_bytes=0, vgpr_spills=0),
            "k_dense_bwd_f32_fastILi64ELi512ELi4ELb1ELb1ELb1E": dict(vgpr=218, scratch_bytes=0, vgpr_spills=0),
            "k_dense_bwd_f32_fastILi64ELi512ELi4ELb0ELb0ELb1E": dict(vgpr=190, scratch_bytes=0, vgpr_spills=0),
            "k_dense_bwd_f32_fastILi64ELi512ELi4ELb1ELb0ELb1E": dict(vgpr=220, scratch_bytes=0, vgpr_spills=0),
            "k_dense_bwd_f32_fastILi64ELi512ELi4ELb0ELb1ELb1E": dict(vgpr=187, scratch_bytes=0, vgpr_spills=0),
            "k_dense_bwd_reduce_dkILb1ELb1E": dict(vgpr=20, scratch_bytes=0, vgpr_spills=0)}
    build.check_hot_kernels(full)
    for name, change in [("k_dense_fwd_f32_pipeILi64E", dict(vgpr=130)),              # three waves per SIMD only
                         ("k_dense_bwd_f32_fastILi64ELi512ELi4ELb1ELb1ELb1E", dict(scratch_bytes=64)),
                         ("k_dense_bwd_reduce_dkILb1ELb1E", dict(vgpr_spills=3))]:
        bad = {k: dict(v) for k, v in full.items()}
        bad[name].update(change)
        with pytest.raises(RuntimeError, match="must not spill"):
            build.check_hot_kernels(bad)
    with pytest.raises(RuntimeError, match="no kernel matches"):
        build.check_hot_kernels({k: v for k, v in full.items() if "reduce" not in k})
    table = os.path.join(ROOT, "l1-attention_amd", "build", "dense_kernel_resources.txt")
    if os.path.exists(table):  # written by the build that made the library under test
        rows = open(table).read().splitlines()
        assert any("dense_fwd_f32_pipeILi64E" in r and "scratch_bytes=0" in r for r in rows)


class _FakeLib(object):
    """Stands in for the loaded library: every entry point reports success without doing anything, after
    checking the call against the header's prototype (argument count; a pointer where a pointer is declared,
    an integer where an integer is).  `calls` lists the names looked up, in order."""
    calls = []
    _protos = None

    @classmethod
    def _check(cls, name, args):
        if cls._protos is None:
            import test_abi_signatures_cpu as sig
            cls._protos = sig._prototypes(open(os.path.join(ROOT, "include", "l1attn_hip.h")).read(), ";")
        ret, params = cls._protos[name]
        assert len(args) == len(params), "%s called with %d arguments, declared with %d" % (name, len(args), len(params))
        for i, (a, p) in enumerate(zip(args, params)):
            if p == "ptr":
                ok = a is None or isinstance(a, (ctypes.c_void_p, ctypes.Array))
            else:
                ok = isinstance(a, int)
            assert ok, "%s argument %d: %r where the header declares %s" % (name, i, a, p)

    def __getattr__(self, name):
        _FakeLib.calls.append(name)

        def call(*a):
            _FakeLib._check(name, a)
            if name.endswith("_bytes"):
                return 256
            if name == "l1attn_sparse_plan_check":
                a[3][4], a[3][5] = 3, 2
            return 0
        return call


def test_driver_control_flow_without_a_gpu(monkeypatch):
    """The Python drivers' argument checks, allocations and call sequences, walked on CPU tensors with the
    library, the device checks and the stream lookup replaced by stand-ins (no kernel runs, no result is
    looked at): a typing slip in a driver shows here and not only on the GPU box."""
    import contextlib
    import sys
    import torch
    sys.path.insert(0, os.path.join(ROOT, "l1-attention_amd"))
    import _l1attn_hip as drv
    monkeypatch.setattr(drv, "lib", lambda: _FakeLib())
    monkeypatch.setattr(drv, "check_input", lambda x, name: None)
    monkeypatch.setattr(drv, "stream_of", lambda x: None)
    monkeypatch.setattr(torch.cuda, "device", lambda d: contextlib.nullcontext())
    B, T, H, W, Wv, E = 2, 6, 3, 8, 4, 7
    q, k = torch.zeros(B, T, H, W), torch.zeros(B, T, H, W)
    v, vb = torch.zeros(B, T, H, Wv), torch.zeros(B, T, H, Wv)
    coo = torch.zeros(E, 4, dtype=torch.int32)
    # paths that have not passed on a GPU yet are closed unless asked for by name
    monkeypatch.setattr(drv, "_enabled", set())
    with pytest.raises(RuntimeError, match="experimental"):
        drv.dense_fused_forward(q, k, v)
    with pytest.raises(RuntimeError, match="experimental"):
        drv.dense_forward_fixed(q, k)
    with pytest.raises(RuntimeError, match="experimental.*rows16"):
        drv.sparse_forward(v.half(), q.half(), k.half(), coo, 3, True)
    with pytest.raises(RuntimeError, match="experimental.*rows16"):
        drv.bidi_backward(v.bfloat16(), v.bfloat16(), vb.bfloat16(), q.bfloat16(), k.bfloat16(), coo,
                          torch.zeros(B, E, H), 3, True)
    with pytest.raises(ValueError, match="unknown experimental"):
        drv.enable_experimental("everything")
    assert drv.enable_experimental("rows16", "fused", "fixed") == frozenset(("rows16", "fused", "fixed"))
    a, = drv.dense_forward(q, k)
    assert a.shape == (B, T, T, H)
    a, = drv.dense_forward_fixed(q, k)
    assert a.shape == (B, T, T, H) and _FakeLib.calls[-2:] == ["l1attn_dense_fwd_fixed_workspace_bytes", "l1attn_dense_fwd_fixed_f32"]
    dq, dk = drv.dense_backward(torch.zeros(B, T, T, H), q, k)
    assert dq.shape == q.shape and dk.shape == k.shape and _FakeLib.calls[-1] == "l1attn_dense_bwd_f32"
    # a caller that vouches for the sign range, or selects a non-default form, goes through the _ex entry point
    # (its argument list is checked against the header by the stand-in library)
    monkeypatch.setattr(drv, "_assume_sign_range", False)
    assert drv.assume_sign_range() is False
    drv.dense_backward(torch.zeros(B, T, T, H), q, k)
    assert _FakeLib.calls[-1] == "l1attn_dense_bwd_ex_f32" and drv.assume_sign_range(False) is True
    drv.dense_backward(torch.zeros(B, T, T, H).double(), q.double(), k.double())
    assert _FakeLib.calls[-1] == "l1attn_dense_bwd_f64"
    with pytest.raises(RuntimeError, match="d_attn must be"):
        drv.dense_backward(torch.zeros(B, T, T, H + 1), q, k)
    with pytest.raises(RuntimeError, match="one shape"):
        drv.dense_backward(torch.zeros(B, T, T, H), q, torch.zeros(B, T, H, W + 1))
    vo, lse = drv.dense_fused_forward(q, k, v, want_lse=True)
    assert vo.shape == v.shape and lse.shape == (B, T, H) and _FakeLib.calls[-1] == "l1attn_fused_fwd_f32"
    assert drv.dense_fused_forward(q.double(), k.double(), v.double())[1] is None
    drv.dense_fused_forward(q, k, v, pipelined=True)
    assert _FakeLib.calls[-1] == "l1attn_fused_fwd_pipe_f32"
    drv.dense_fused_forward(q.double(), k.double(), v.double(), pipelined=True)   # float64 has one entry
    assert _FakeLib.calls[-1] == "l1attn_fused_fwd_f64"
    with pytest.raises(RuntimeError, match="equal leading dims"):
        drv.dense_fused_forward(q, k, torch.zeros(B, T + 1, H, Wv))
    with pytest.raises(RuntimeError, match="share dtype"):
        drv.dense_fused_forward(q, k, v.double())
    grads = drv.dense_fused_backward(torch.zeros_like(v), q, k, v, vo, lse)
    assert [g.shape for g in grads] == [q.shape, k.shape, v.shape]
    assert "l1attn_fused_bwd_stage_f32" in _FakeLib.calls and "l1attn_fused_bwd_stage_pipe_f32" not in _FakeLib.calls
    drv.dense_fused_backward(torch.zeros_like(v), q, k, v, vo, lse, pipelined=True)
    assert "l1attn_fused_bwd_stage_pipe_f32" in _FakeLib.calls
    drv.dense_fused_backward(torch.zeros_like(v).double(), q.double(), k.double(), v.double(), vo.double(), lse.double(),
                             pipelined=True)                                          # float64 has one entry
    assert _FakeLib.calls[-1].startswith("l1attn_dense_bwd") and "l1attn_fused_bwd_stage_f64" in _FakeLib.calls
    with pytest.raises(RuntimeError, match="lse must be"):
        drv.dense_fused_backward(torch.zeros_like(v), q, k, v, vo, lse[:, :-1])
    with pytest.raises(RuntimeError, match="dvo must have"):
        drv.dense_fused_backward(torch.zeros(B, T, H, Wv + 1), q, k, v, vo, lse)
    plan = drv.plan_for(coo, T)
    assert (plan.E, plan.T, plan.max_dst_deg, plan.max_src_deg) == (E, T, 3, 2)
    assert drv.plan_for(coo, T) is plan                      # cached on the tensor
    coo[0, 0] = 1
    assert drv.plan_for(coo, T) is not plan                  # in-place write invalidates
    vo, P = drv.sparse_forward(v, q, k, coo, 3, True)
    assert vo.shape == v.shape and P.shape == (B, E, H)
    dv, dq, dk = drv.sparse_backward(torch.zeros_like(v), v, q, k, coo, P, 3, True)
    assert dv.shape == v.shape and dq.shape == q.shape and dk.shape == k.shape
    with pytest.raises(RuntimeError, match="dvo must have"):
        drv.sparse_backward(torch.zeros(B, T, H, Wv + 1), v, q, k, coo, P, 3, True)
    with pytest.raises(RuntimeError, match="attn must be"):
        drv.sparse_backward(torch.zeros_like(v), v, q, k, coo, P[:, :-1], 3, True)
    vo, P = drv.bidi_forward(v, vb, q, k, coo, 3, False)
    assert vo.shape == v.shape and P.shape == (B, E, H)
    grads = drv.bidi_backward(torch.zeros_like(v), v, vb, q, k, coo, P, 3, False)
    assert [g.shape for g in grads] == [v.shape, vb.shape, q.shape, k.shape]
    with pytest.raises(RuntimeError, match="vb must have"):
        drv.bidi_forward(v, torch.zeros(B, T, H, Wv + 2), q, k, coo, 3, True)
    with pytest.raises(RuntimeError, match="equal leading dims"):
        drv.sparse_forward(torch.zeros(B, T + 1, H, Wv), q, k, coo, 3, True)
    with pytest.raises(RuntimeError, match="only float32 and float64"):
        drv.dense_forward(q.half(), k.half())
    # 16-bit rows: fp32 edge weights, entry points named after the storage type
    for dt, sfx in ((torch.float16, "f16"), (torch.bfloat16, "bf16")):
        v16, vb16, q16, k16 = (x.to(dt) for x in (v, vb, q, k))
        del _FakeLib.calls[:]
        vo, P = drv.sparse_forward(v16, q16, k16, coo, 3, True)
        assert _FakeLib.calls[-1] == "l1attn_sparse_fwd_" + sfx
        assert vo.dtype == dt and vo.shape == v.shape and P.dtype == torch.float32 and P.shape == (B, E, H)
        vo, P = drv.bidi_forward(v16, vb16, q16, k16, coo, 3, False)
        assert _FakeLib.calls[-1] == "l1attn_sparse_bidi_fwd_" + sfx
        assert vo.dtype == dt and P.dtype == torch.float32
        grads = drv.sparse_backward(torch.zeros_like(v16), v16, q16, k16, coo, P, 3, True)
        assert _FakeLib.calls[-1] == "l1attn_sparse_bwd_" + sfx and all(g_.dtype == dt for g_ in grads)
        grads = drv.bidi_backward(torch.zeros_like(v16), v16, vb16, q16, k16, coo, P, 3, True)
        assert _FakeLib.calls[-1] == "l1attn_sparse_bidi_bwd_" + sfx and len(grads) == 4
        with pytest.raises(RuntimeError, match="attn must be"):  # the weights of a 16-bit call are fp32
            drv.sparse_backward(torch.zeros_like(v16), v16, q16, k16, coo, P.to(dt), 3, True)
        with pytest.raises(RuntimeError, match="share dtype"):
            drv.sparse_forward(v, q16, k16, coo, 3, True)


def test_operator_modules_autograd_plumbing_without_a_gpu(monkeypatch):
    """The three drop-in modules under autograd with the stand-in library: which tensors are saved, which
    gradients come back (None for coo and the integers), five- and six-argument calls of the sparse module."""
    import contextlib
    import sys
    import torch
    sys.path.insert(0, os.path.join(ROOT, "l1-attention_amd"))
    import _l1attn_hip as drv
    import l1attn_cuda, l1attn_sparse_cuda, l1attn_sparse_bidi_cuda
    monkeypatch.setattr(drv, "lib", lambda: _FakeLib())
    monkeypatch.setattr(drv, "check_input", lambda x, name: None)
    monkeypatch.setattr(drv, "stream_of", lambda x: None)
    monkeypatch.setattr(torch.cuda, "device", lambda d: contextlib.nullcontext())
    monkeypatch.setattr(drv, "_enabled", {"fused"})
    B, T, H, W, E = 2, 5, 3, 8, 6
    mk = lambda *s: torch.zeros(*s, requires_grad=True)
    q, k = mk(B, T, H, W), mk(B, T, H, W)
    a = l1attn_cuda.L1Attn()(q, k)
    assert a.shape == (B, T, T, H)
    a.sum().backward()
    assert q.grad.shape == q.shape and k.grad.shape == k.shape
    coo = torch.zeros(E, 4, dtype=torch.int32)
    v, q, k = mk(B, T, H, W), mk(B, T, H, W), mk(B, T, H, W)
    m = l1attn_sparse_cuda.L1AttnSparse()
    vo = m(v, q, k, coo, 2)                 # README form
    vo2 = m(v, q, k, coo, 2, False)         # wrapper form
    (vo.sum() + vo2.sum()).backward()
    assert all(t.grad is not None and t.grad.shape == t.shape for t in (v, q, k))
    vf, vb, q, k = mk(B, T, H, W), mk(B, T, H, W), mk(B, T, H, W), mk(B, T, H, W)
    vo = l1attn_sparse_bidi_cuda.L1AttnSparseBidi()(vf, vb, q, k, coo, 2, True)
    vo.sum().backward()
    assert all(t.grad is not None and t.grad.shape == t.shape for t in (vf, vb, q, k))
    # the fused operator: forward saves vo and lse, backward returns three gradients
    q, k, v = mk(B, T, H, W), mk(B, T, H, W), mk(B, T, H, W)
    del _FakeLib.calls[:]
    vo = l1attn_cuda.L1AttnFused()(q, k, v)
    assert vo.shape == v.shape
    vo.sum().backward()
    assert all(t.grad is not None and t.grad.shape == t.shape for t in (q, k, v))
    assert [c for c in _FakeLib.calls if not c.endswith("_bytes")] == \
        ["l1attn_fused_fwd_f32", "l1attn_fused_bwd_stage_f32", "l1attn_dense_bwd_f32"]


def test_native_module_stand_ins_without_a_gpu(monkeypatch):
    """The three modules named like the reference's pybind11 drivers (cuda/l1attn_cuda_drv.cpp:106-109,
    cuda/l1attn_sparse_cuda_drv.cpp:71-74, cuda/l1attn_sparse_bidi_cuda_drv.cpp:77-80): forward/backward with the
    reference's argument order and list returns, called the way the reference's own autograd Functions call them
    (saved dst_mxlen / use_softmax come back as .item() values: cuda/l1attn_sparse_cuda.py:16, :42-46)."""
    import contextlib
    import sys
    import torch
    sys.path.insert(0, os.path.join(ROOT, "l1-attention_amd"))
    import _l1attn_hip as drv
    import l1attn_cuda_drv, l1attn_sparse_cuda_drv, l1attn_sparse_bidi_cuda_drv
    for m in (l1attn_cuda_drv, l1attn_sparse_cuda_drv, l1attn_sparse_bidi_cuda_drv):
        assert callable(m.forward) and callable(m.backward)
    q = torch.randn(1, 4, 2, 8)
    with pytest.raises(RuntimeError, match="q must be a CUDA tensor"):      # CHECK_INPUT, library not needed
        l1attn_cuda_drv.forward(q, q)
    with pytest.raises(RuntimeError, match="v must be a CUDA tensor"):
        l1attn_sparse_cuda_drv.forward(q, q, q, torch.zeros(3, 4, dtype=torch.int32), 2, True)
    with pytest.raises(RuntimeError, match="dvo must be a CUDA tensor"):
        l1attn_sparse_bidi_cuda_drv.backward(q, q, q, q, q, torch.zeros(3, 4, dtype=torch.int32), q, 2, True)
    monkeypatch.setattr(drv, "lib", lambda: _FakeLib())
    monkeypatch.setattr(drv, "check_input", lambda x, name: None)
    monkeypatch.setattr(drv, "stream_of", lambda x: None)
    monkeypatch.setattr(torch.cuda, "device", lambda d: contextlib.nullcontext())
    B, T, H, W, E = 2, 5, 3, 8, 6
    q, k, v, vb = (torch.zeros(B, T, H, W) for _ in range(4))
    coo = torch.zeros(E, 4, dtype=torch.int32)
    attn = l1attn_cuda_drv.forward(q, k)
    assert isinstance(attn, list) and attn[0].shape == (B, T, T, H)
    d_q, d_k = l1attn_cuda_drv.backward(torch.zeros(B, T, T, H), q, k)
    assert d_q.shape == q.shape and d_k.shape == k.shape
    dmx, sm = torch.tensor(3), torch.tensor(True)
    vo, attn = l1attn_sparse_cuda_drv.forward(v, q, k, coo, 3, True)
    d_v, d_q, d_k = l1attn_sparse_cuda_drv.backward(torch.zeros_like(vo), v, q, k, coo, attn, dmx.item(), sm.item())
    assert vo.shape == v.shape and [g.shape for g in (d_v, d_q, d_k)] == [v.shape, q.shape, k.shape]
    vo, attn = l1attn_sparse_bidi_cuda_drv.forward(v, vb, q, k, coo, 3, False)
    grads = l1attn_sparse_bidi_cuda_drv.backward(torch.zeros_like(vo), v, vb, q, k, coo, attn, dmx.item(), False)
    assert len(grads) == 4 and all(g.shape == v.shape for g in grads)


def test_build_checks_the_instruction_density_of_the_hot_loops():
    """build.py counts the vector-ALU instructions of the headline kernels' loops on the listing and fails when a
    loop spends more per pair-element than accepted (the algorithm itself: 2 forward, 3 backward)."""
    import sys
    sys.path.insert(0, os.path.join(ROOT, "l1-attention_amd"))
    import build
    body = "\n".join(["\tv_subrev_f32_e32 v1, s4, v2", "\tv_add_f32_e64 v3, v3, |v1|"] * 8)
    listing = """
_Z4kernv: ; @k
	s_load_dwordx2 s[0:1], s[4:5], 0x0
.LBB0_1: ; %loop
""" + body + """
	s_add_u32 s2, s2, 1
	s_waitcnt lgkmcnt(0)
	ds_read_b32 v9, v8
	s_cbranch_scc1 .LBB0_1
	s_endpgm
.Lfunc_end0:
"""
    (loop,) = build.loop_profiles(listing, "kern")
    assert (loop["valu"], loop["salu"], loop["waitcnt"], loop["lds"], loop["smem"]) == (16, 2, 1, 1, 0)
    assert build.check_hot_loops(listing, (("kernv", 8, 2, 2.0),)) == {"kernv": 2.0}
    with pytest.raises(RuntimeError, match="2.00 vector instructions per pair-element"):
        build.check_hot_loops(listing, (("kernv", 8, 2, 1.9),))
    with pytest.raises(RuntimeError, match="no loop"):
        build.check_hot_loops(listing, (("kernv", 16, 2, 4.0),))


def test_backward_variants_are_chosen_by_argument_only(lib):
    """loop_form 1 / 2 of l1attn_dense_bwd_plan_info_ex turn the branch-free plans into their pipelined forms (two
    steps of prefetch distance; the same with two LDS planes, hence twice the LDS) and change nothing else.  The
    library reads no environment variable: a process started with the old switches set plans as any other."""
    shapes = ((2, 64, 4, 32), (16, 1024, 8, 64), (8, 4096, 16, 64), (8, 4100, 16, 64), (2, 3, 16, 7))
    lib.l1attn_dense_bwd_plan_info.argtypes = [ctypes.c_int64] * 4 + [ctypes.c_void_p]
    lib.l1attn_dense_bwd_plan_info_ex.argtypes = [ctypes.c_int64] * 4 + [ctypes.c_int, ctypes.c_void_p]

    def plans(form):
        out = []
        for s in shapes:
            a = (ctypes.c_int64 * 16)()
            rc = lib.l1attn_dense_bwd_plan_info(*s, a) if form is None else lib.l1attn_dense_bwd_plan_info_ex(*s, form, a)
            assert rc == 0
            out.append(list(a))
        return out
    runs = {f: plans(f) for f in (None, 0, 1, 2)}
    assert runs[None] == runs[0] and all(p[14] == 0 for p in runs[0])
    a = (ctypes.c_int64 * 16)()
    assert lib.l1attn_dense_bwd_plan_info_ex(*shapes[1], 3, a) == -1 and lib.l1attn_dense_bwd_plan_info_ex(*shapes[1], -1, a) == -1
    for form in (1, 2):
        for one, two in zip(runs[0], runs[form]):
            assert two[14] == form * one[3]                                      # exactly the branch-free plans change
            assert two[11] == one[11] * (2 if two[14] == 2 else 1)               # LDS: two planes in form 2
            assert one[:11] + one[12:14] == two[:11] + two[12:14]                # and nothing else
    assert [p[14] for p in runs[2]] == [0, 2, 2, 0, 0]
    import _l1attn_hip as drv
    code = ("import ctypes, sys; L = ctypes.CDLL(sys.argv[1]);"
            "L.l1attn_dense_bwd_plan_info.argtypes = [ctypes.c_int64] * 4 + [ctypes.c_void_p];"
            "a = (ctypes.c_int64 * 16)(); assert L.l1attn_dense_bwd_plan_info(8, 4096, 16, 64, a) == 0; print(list(a))")
    env = dict(os.environ, L1ATTN_BWD_PREFETCH="3", L1ATTN_RANK_SORT="merge")
    r = subprocess.run([sys.executable, "-c", code, drv._LIB_PATH], env=env, capture_output=True, text=True, check=True)
    assert eval(r.stdout) == runs[0][2]
    with open(os.path.join(os.path.dirname(drv._LIB_PATH), "csrc", "dense.hip")) as f:
        assert "getenv" not in f.read()


def test_non_default_backward_forms_need_an_opt_in_by_name(monkeypatch):
    import _l1attn_hip as drv
    monkeypatch.setattr(drv, "_enabled", set())
    monkeypatch.setattr(drv, "_dense_bwd_form", (0, 0))
    with pytest.raises(RuntimeError, match="bwd_pipe"):
        drv.set_dense_backward_form(loop_form=1)
    with pytest.raises(RuntimeError, match="rank_merge"):
        drv.set_dense_backward_form(rank_sort=1)
    with pytest.raises(ValueError):
        drv.set_dense_backward_form(loop_form=3)
    assert drv.set_dense_backward_form(0, 0) == (0, 0)
    drv.enable_experimental("bwd_pipe", "rank_merge")
    with pytest.warns(RuntimeWarning, match="loop_form=2, rank_sort=1"):   # said once per change, never silently
        assert drv.set_dense_backward_form(2, 1) == (0, 0) and drv._dense_bwd_form == (2, 1)
    assert drv.dense_backward_plan(8, 4096, 16, 64)[14] == 2 and drv.dense_backward_plan(8, 4096, 16, 64, 0)[14] == 0
    assert drv.set_dense_backward_form() == (2, 1)
