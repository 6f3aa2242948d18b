"""CPU-only: the hand-written instruction sequences of csrc/gfx950.h and csrc/sload.h, read off the headers and
executed by a small interpreter of the few instructions they use, against the host stand-ins the kernel emulation
runs in their place (tests/cpu_emu/emu_gfx950.h, emu_sload.h).

The kernel emulation replaces these two headers by "what the instructions compute".  This file checks that claim
from the other side: the asm templates themselves -- operand numbers, negations, the order of the instructions --
compute what the stand-ins compute, on random values bit for bit; and their operand constraints obey the rule whose
violation is invisible to any host run: an output that is written before the last input has been read must be
early-clobber ("=&") or tied ("+"), or the compiler may give it an input's register.  (That the instructions
assemble for gfx950 is the build's business: hipcc assembles every template.)
"""
import os
import re
import struct
import subprocess
from fractions import Fraction

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CSRC = os.path.join(ROOT, "l1-attention_amd", "csrc")
EMU = os.path.join(ROOT, "tests", "cpu_emu")
CLANG = "/opt/rocm/llvm/bin/clang++"
CXX = CLANG if os.path.exists(CLANG) else "g++"


@pytest.fixture(scope="module")
def headers():
    """gfx950.h (which includes sload.h) after the preprocessor, so that operand macros are expanded."""
    r = subprocess.run([CXX, "-E", "-P", "-x", "c++", "-std=c++20", "-I", EMU, "-I", CSRC, "-D__device__=",
                        "-D__forceinline__=inline", os.path.join(CSRC, "gfx950.h")], capture_output=True, text=True)
    assert r.returncode == 0, r.stderr[-2000:]
    return r.stdout


def _split_top(text, sep):
    """Split at `sep` outside parentheses and string literals."""
    parts, depth, cur, i, in_str = [], 0, "", 0, False
    while i < len(text):
        c = text[i]
        if in_str:
            cur += c
            if c == "\\":
                cur += text[i + 1]
                i += 1
            elif c == '"':
                in_str = False
        elif c == '"':
            in_str = True
            cur += c
        elif c in "([":
            depth += 1
            cur += c
        elif c in ")]":
            depth -= 1
            cur += c
        elif c == sep and depth == 0:
            parts.append(cur)
            cur = ""
        else:
            cur += c
        i += 1
    parts.append(cur)
    return parts


def asm_of(text, func):
    """-> (instructions, outputs, inputs) of the asm statement in `func`; operands as (constraint, C expression)."""
    m = re.search(r"inline void %s\(" % re.escape(func), text)
    assert m, func
    return _asm_at(text, text.index("asm volatile(", m.end()) + len("asm volatile("))


def _asm_at(text, start):
    depth, i = 1, start
    while depth:
        depth += {"(": 1, ")": -1}.get(text[i], 0)
        i += 1
    sections = _split_top(text[start:i - 1], ":")
    template = "".join(re.findall(r'"((?:[^"\\]|\\.)*)"', sections[0]))
    instrs = [x.strip() for x in template.replace("\\t", " ").split("\\n") if x.strip()]

    def operands(sec):
        out = []
        for item in _split_top(sec, ","):
            item = item.strip()
            if item:
                mm = re.match(r'"([^"]*)"\s*\((.*)\)$', item, re.S)
                assert mm, item
                out.append((mm.group(1), " ".join(mm.group(2).split())))
        return out
    outs = operands(sections[1]) if len(sections) > 1 else []
    ins = operands(sections[2]) if len(sections) > 2 else []
    return instrs, outs, ins


def _f32(x):
    return np.float32(x)


def _round_f32(r):
    """Fraction -> float32, round to nearest even (what a fused multiply-add delivers)."""
    x = np.float32(float(r))
    best = None
    for c in (np.nextafter(x, np.float32(-np.inf)), x, np.nextafter(x, np.float32(np.inf))):
        if not np.isfinite(c):
            continue
        err = abs(Fraction(float(c)) - r)
        even = (struct.unpack("<I", struct.pack("<f", float(c)))[0] & 1) == 0
        if best is None or err < best[0] or (err == best[0] and even):
            best = (err, c)
    return np.float32(best[1])


def run_template(instrs, regs):
    """Execute the instructions on `regs` {operand number: np.float32 | int (an unsigned 32-bit value)}."""
    def src(tok):
        tok = tok.strip()
        neg = tok.startswith("-%")
        if tok.startswith("%") or neg:
            v = regs[int(tok.lstrip("-%"))]
            return -v if neg else v
        return _f32(float(tok))
    for ins in instrs:
        op, _, rest = ins.partition(" ")
        clamp = rest.endswith(" clamp")
        args = [a.strip() for a in (rest[:-6] if clamp else rest).split(",")]
        assert args[0].startswith("%"), ins
        d = int(args[0][1:])
        if op in ("v_sub_f32", "v_sub_f32_e64"):
            r = _f32(src(args[1]) - src(args[2]))
            regs[d] = _f32(min(max(r, _f32(0)), _f32(1))) if clamp else r
        elif op == "v_med3_f32":
            regs[d] = sorted([src(a) for a in args[1:4]])[1]
        elif op == "v_fmac_f32":
            regs[d] = _round_f32(Fraction(float(src(args[1]))) * Fraction(float(src(args[2]))) + Fraction(float(regs[d])))
        elif op == "v_fma_f32":
            regs[d] = _round_f32(Fraction(float(src(args[1]))) * Fraction(float(src(args[2]))) + Fraction(float(src(args[3]))))
        elif op == "v_sad_u32":
            a, b, c = (int(regs[int(t.strip()[1:])]) for t in args[1:4])
            regs[d] = (abs(a - b) + c) & 0xFFFFFFFF
        else:
            raise AssertionError("instruction the interpreter does not know: " + ins)
    return regs


def check_constraints(instrs, outs, ins):
    """Operand numbers exist and are all used; an output written while an input is still to be read is '&' or '+'."""
    n_out, n = len(outs), len(outs) + len(ins)
    used = set()
    last_input_read, first_write = -1, {}
    for i, text in enumerate(instrs):
        toks = [int(t) for t in re.findall(r"%(\d+)", text)]
        assert all(t < n for t in toks), text
        used.update(toks)
        first = re.match(r"\S+\s+%(\d+)", text)
        if first and not text.startswith("s_waitcnt"):
            first_write.setdefault(int(first.group(1)), i)
        reads = toks[1:] if first else toks
        if any(t >= n_out for t in reads):
            last_input_read = i
    # (a template that names no operand at all only pins registers for the compiler: swait32, the empty statements)
    assert used == set(range(n)) or not used, (sorted(set(range(n)) - used), "operands never used")
    for o, (constraint, _) in enumerate(outs):
        assert constraint[0] in "=+", constraint
        if constraint.startswith("=") and "&" not in constraint and o in first_write:
            assert first_write[o] >= last_input_read, "output %d written before the last input is read needs '=&'" % o


HARNESS = r"""
#include "emu_gfx950.h"
#include <stdio.h>
int main()
{
	int mode;
	while (scanf("%d", &mode) == 1) {
		if (mode == 2) {
			unsigned au, q[8], k[8];
			scanf("%u", &au);
			for (int i = 0; i < 8; i++) scanf("%u", &q[i]);
			for (int i = 0; i < 8; i++) scanf("%u", &k[i]);
			float qv[8];
			f32x16 kv;
			for (int i = 0; i < 16; i++) kv.a[i] = 0;
			for (int i = 0; i < 8; i++) { qv[i] = __uint_as_float(q[i]); kv.a[4 + i] = __uint_as_float(k[i]); }
			sad8(au, qv, kv, 4);
			printf("%u\n", au);
			continue;
		}
		float qc[4], kc, g[4], dq[4], dk;
		for (int i = 0; i < 4; i++) scanf("%a", &qc[i]);
		scanf("%a", &kc);
		for (int i = 0; i < 4; i++) scanf("%a", &g[i]);
		for (int i = 0; i < 4; i++) scanf("%a", &dq[i]);
		scanf("%a", &dk);
		const float4 gg = {g[0], g[1], g[2], g[3]};
		if (mode == 0) pair_step4(qc, kc, gg, dq, dk); else pair_step4_rank(qc, kc, gg, dq, dk);
		printf("%a %a %a %a %a\n", dq[0], dq[1], dq[2], dq[3], dk);
	}
	return 0;
}
"""


@pytest.fixture(scope="module")
def stand_ins(tmp_path_factory):
    d = tmp_path_factory.mktemp("asm_harness")
    src, exe = str(d / "h.cpp"), str(d / "h")
    open(src, "w").write(HARNESS)
    subprocess.run(["g++", "-std=c++20", "-O1", "-pthread", "-ffp-contract=off", "-I", EMU, src, "-o", exe], check=True)

    def call(lines):
        r = subprocess.run([exe], input="\n".join(lines) + "\n", capture_output=True, text=True, check=True)
        return r.stdout.split("\n")[:-1]
    return call


@pytest.mark.parametrize("func,mode", [("pair_step4", 0), ("pair_step4_rank", 1)])
def test_backward_pair_steps_compute_what_their_stand_ins_compute(headers, stand_ins, func, mode):
    instrs, outs, ins = asm_of(headers, func)
    check_constraints(instrs, outs, ins)
    assert [e for _, e in outs] == ["e0", "e1", "dq[0]", "dq[1]", "dq[2]", "dq[3]", "dk"]
    assert [e for _, e in ins] == ["qc[0]", "qc[1]", "qc[2]", "qc[3]", "kc", "g.x", "g.y", "g.z", "g.w"]
    assert all(c == "v" for c, _ in ins) and [c for c, _ in outs] == ["=&v", "=&v"] + ["+v"] * 5
    rng = np.random.default_rng(5 + mode)
    cases, lines = [], []
    for n in range(400):
        if mode == 0:    # differences of values scaled by 2^64: huge, zero, or of magnitude at least 1; some fractional
            qc = rng.standard_normal(4).astype(np.float32) * np.float32(2.0 ** rng.integers(-3, 70))
            kc = np.float32(qc[rng.integers(4)] if n % 3 == 0 else rng.standard_normal() * 2.0 ** rng.integers(-3, 70))
        else:            # ranks: whole numbers against a whole number minus one half
            qc = rng.integers(-1, 60, 4).astype(np.float32) * 2
            kc = np.float32(2 * rng.integers(0, 60) - 0.5)
        g, dq = rng.standard_normal(4).astype(np.float32), rng.standard_normal(4).astype(np.float32)
        dk = np.float32(rng.standard_normal())
        cases.append((qc, kc, g, dq, dk))
        lines.append("%d " % mode + " ".join(float(x).hex() for x in list(qc) + [kc] + list(g) + list(dq) + [dk]))
    want = stand_ins(lines)
    for (qc, kc, g, dq, dk), line in zip(cases, want):
        regs = {0: _f32(0), 1: _f32(0), 6: dk, 11: kc}
        regs.update({2 + i: dq[i] for i in range(4)})
        regs.update({7 + i: qc[i] for i in range(4)})
        regs.update({12 + i: g[i] for i in range(4)})
        run_template(instrs, regs)
        got = [regs[2], regs[3], regs[4], regs[5], regs[6]]
        ref = [np.float32(float.fromhex(x)) for x in line.split()]
        assert all(a == b for a, b in zip(got, ref)), (func, qc, kc, got, ref)


def test_fixed_point_block_computes_what_its_stand_in_computes(headers, stand_ins):
    instrs, outs, ins = asm_of(headers, "sad8")
    check_constraints(instrs, outs, ins)
    assert outs == [("+v", "au")] and len(ins) == 16
    # the eight q operands are VGPRs from qv[0..8), the eight k operands SGPRs from kv[i0 .. i0+8), in this order
    assert [e for _, e in ins[:8]] == ["__float_as_uint(qv[%d])" % i for i in range(8)]
    assert [e for _, e in ins[8:]] == ["__float_as_uint(kv[i0 + %d])" % i for i in range(8)]
    assert [c for c, _ in ins] == ["v"] * 8 + ["s"] * 8
    rng = np.random.default_rng(9)
    cases, lines = [], []
    for _ in range(300):
        au = int(rng.integers(0, 2 ** 31))
        q = [int(x) for x in rng.integers(0, 2 ** 32, 8)]
        k = [int(x) for x in rng.integers(0, 2 ** 32, 8)]
        cases.append((au, q, k))
        lines.append("2 %d " % au + " ".join(str(x) for x in q + k))
    for (au, q, k), line in zip(cases, stand_ins(lines)):
        regs = {0: au}
        regs.update({1 + i: q[i] for i in range(8)})
        regs.update({9 + i: k[i] for i in range(8)})
        assert run_template(instrs, regs)[0] == int(line)


def test_scalar_prefetch_helpers_load_what_their_stand_ins_deliver(headers):
    """sload32: sixteen floats at p into `lo`, the next sixteen (byte offset 0x40) into `hi`, both destinations
    early-clobber so that the second load still finds the pointer; sload32_at<BYTES> the same from p + BYTES;
    swait32 waits for everything outstanding and names both buffers as read and written, which is what keeps the
    compiler from using them across it.  emu_sload.h: memcpy(lo, p, 64); memcpy(hi, p + 16, 64) at the wait."""
    instrs, outs, ins = asm_of(headers, "sload32")
    check_constraints(instrs, outs, ins)
    assert instrs == ["s_load_dwordx16 %0, %2, 0x0", "s_load_dwordx16 %1, %2, 0x40"]
    assert outs == [("=&s", "lo"), ("=&s", "hi")] and ins == [("s", "p")]
    instrs, outs, ins = asm_of(headers, "sload32_at")
    check_constraints(instrs, outs, ins)
    assert instrs == ["s_load_dwordx16 %0, %2, %3", "s_load_dwordx16 %1, %2, %4"]
    assert outs == [("=&s", "lo"), ("=&s", "hi")] and ins == [("s", "p"), ("n", "BYTES"), ("n", "BYTES + 0x40")]
    instrs, outs, ins = asm_of(headers, "swait32")
    assert instrs == ["s_waitcnt lgkmcnt(0)"] and outs == [("+s", "lo"), ("+s", "hi")] and ins == []
    instrs, outs, ins = asm_of(headers, "lds_barrier")
    assert instrs == ["s_waitcnt lgkmcnt(0)", "s_barrier"] and outs == [] and ins == []
    stand_in = open(os.path.join(EMU, "emu_sload.h")).read()
    assert "memcpy(x.lo->a, x.p, 64);" in stand_in and "memcpy(x.hi->a, x.p + 16, 64);" in stand_in
    assert "sload32(lo, hi, p + BYTES / 4);" in stand_in


def test_the_constraint_rule_catches_a_missing_early_clobber():
    instrs = ["v_sub_f32 %0, %2, %3", "v_fmac_f32 %1, %0, %4"]
    ok = ([("=&v", "e"), ("+v", "acc")], [("v", "a"), ("v", "b"), ("v", "g")])
    check_constraints(instrs, *ok)
    with pytest.raises(AssertionError, match="needs '=&'"):
        check_constraints(instrs, [("=v", "e"), ("+v", "acc")], ok[1])
    with pytest.raises(AssertionError, match="never used"):
        check_constraints(instrs, ok[0], ok[1] + [("v", "spare")])
    with pytest.raises(AssertionError):
        check_constraints(["v_sub_f32 %0, %2, %9"], *ok)


def test_every_asm_statement_of_the_sources_obeys_the_constraint_rule():
    """All `asm volatile(...)` statements under csrc/ (the instruction-rate probes of version.hip included): operand
    numbers exist, every operand is used, outputs written before the last input is read are '=&' or '+'.  Empty
    templates (register pins for the scheduler) only name operands."""
    import glob
    n = 0
    for path in sorted(glob.glob(os.path.join(CSRC, "*"))):
        text = open(path).read()
        text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
        text = re.sub(r"//[^\n]*", "", text)
        if "L1_QU(" in text:  # the one operand list written with macros: the preprocessed text is checked above
            continue
        for m in re.finditer(r"asm volatile\(", text):
            instrs, outs, ins = _asm_at(text, m.end())
            check_constraints(instrs, outs, ins)
            n += 1
    assert n >= 20
