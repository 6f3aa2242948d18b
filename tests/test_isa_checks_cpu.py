"""CPU-only: the build's look-out for instructions the device code must not contain."""
import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, os.path.join(ROOT, "l1-attention_amd"))


def test_build_rejects_forbidden_instructions():
    import isa_checks
    ok = """
k:
	v_fmac_f32_e32 v1, v2, v3
	v_pk_mul_lo_u16 v4, v5, v6
	s_load_dwordx4 s[0:3], s[4:5], 0x0
	buffer_store_dword v1, v0, s[0:3], 0 offen
	global_atomic_add_f32 v0, v1, s[2:3]
	s_endpgm
"""
    isa_checks.check_forbidden(ok)
    for line in ("v_pk_fma_f32 v[0:1], v[2:3], v[4:5], v[6:7]", "v_pk_add_f32 v[0:1], v[2:3], v[4:5]",
                 "v_pk_mul_f32 v[0:1], v[2:3], v[4:5]", "s_store_dword s0, s[2:3], 0x0",
                 "s_buffer_store_dwordx2 s[0:1], s[4:7], 0x0", "s_atomic_add s0, s[2:3], 0x0", "s_dcache_wb"):
        with pytest.raises(RuntimeError, match="forbidden instruction"):
            isa_checks.check_forbidden(ok.replace("\tv_fmac_f32_e32 v1, v2, v3", "\t" + line), "x.hip")
