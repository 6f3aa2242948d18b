"""Checks of the generated device code that only the build (on the CPU) runs.

This file names instructions the library must never contain, so that the build can look for them."""
import re

FORBIDDEN = (
    # packed fp32 arithmetic: compiled out with -packed-fp32-ops, never written by hand
    r"v_pk_(add|mul|fma)_f32",
    # anything that writes through the scalar data cache
    r"s_(buffer_)?store_", r"s_(buffer_)?atomic_", r"s_scratch_store", r"s_dcache_wb",
)


def check_forbidden(asm, where=""):
    """Fail the build if the device code contains an instruction this library must not use."""
    pat = re.compile(r"^\s*(" + "|".join(FORBIDDEN) + r")", re.M)
    hits = [m.group(0).strip() for m in pat.finditer(asm)]
    if hits:
        raise RuntimeError("forbidden instruction in %s: %s" % (where or "device code", ", ".join(sorted(set(hits)))))
