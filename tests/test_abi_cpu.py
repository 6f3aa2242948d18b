"""CPU-only checks of the C ABI: the library loads, exports every function include/l1attn_hip.h
declares, and its host-side argument logic (no kernel launch) behaves as documented."""
import ctypes
import os
import re

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
    # one dst tile (T <= 32) or the generic path needs no workspace
    assert lib.l1attn_dense_bwd_workspace_bytes(2, 32, 4, 32) == 0
    assert lib.l1attn_dense_bwd_workspace_bytes(2, 3, 16, 7) == 0
    # headline config: 64 dst tiles (64 tokens each) x 8 batches x T x H*W floats
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
    # kernels without the prefetch idiom are not inspected
    assert build.check_scalar_prefetch(good.replace("dense_fwd_f32_pipe", "other_kernel")) == 0
