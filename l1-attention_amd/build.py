"""Compile the HIP sources under csrc/ into libl1attn_hip.so, and the host-CPU twin under csrc_cpu/ into
libl1attn_cpu.so, next to this file.

    python build.py            # hipcc --offload-arch=gfx950 and g++, in-tree output

hipcc cross-compiles without a GPU.  Packed fp32 instructions are disabled for all device
code (-packed-fp32-ops): the kernels issue scalar-per-lane fp32 VALU operations only.
"""
import glob
import os
import re
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
LIB = os.path.join(HERE, "libl1attn_hip.so")
CPU_LIB = os.path.join(HERE, "libl1attn_cpu.so")
ARCH = "gfx950"


def sources():
    return sorted(glob.glob(os.path.join(HERE, "csrc", "*.hip")))


def _sregs(tok):
    m = re.match(r"s\[(\d+):(\d+)\]$", tok)
    if m:
        return set(range(int(m.group(1)), int(m.group(2)) + 1))
    m = re.match(r"s(\d+)$", tok)
    return {int(m.group(1))} if m else set()


_VMEM_LOAD = re.compile(r"^(buffer_load|global_load|flat_load|scratch_load|tbuffer_load|ds_read|ds_load|"
                        r"buffer_atomic|global_atomic|flat_atomic|ds_\w+_rtn)")


def _walk_kernels(asm_text):
    """(kernel, line number, instruction text, inside an inline-asm block) for every instruction of a device
    listing.  The compiler brackets inline asm with `;;#ASMSTART` / `;;#ASMEND` comment lines."""
    cur, in_asm = None, False
    for ln, line in enumerate(asm_text.split("\n"), 1):
        l = line.strip()
        if l.startswith(";;#ASMSTART"):
            in_asm = True
            continue
        if l.startswith(";;#ASMEND"):
            in_asm = False
            continue
        if l.startswith("_Z") and ":" in l.split(";")[0]:
            cur, in_asm = l.split(":")[0], False
            continue
        if l.startswith(".Lfunc_end"):  # what follows the last function of a listing is metadata, not code
            cur = None
            continue
        if cur is None or not l or l[0] in ";.":
            continue
        l = l.split(";")[0].strip()
        if l:
            yield cur, ln, l, in_asm


def check_inline_asm_loads(asm_text, where=""):
    """No inline-asm block of any kernel may issue a load whose result arrives later (vector memory, LDS, or an
    atomic that returns a value): the compiler does not know that the destination registers are still being
    written, is free to move or reuse them before the hand-placed wait, and the late data then lands in whatever
    lives there (an address, an exec mask) -- a memory fault on the GPU.  Loads of that kind go through builtins
    or plain C++, which the compiler tracks.  The one exception, scalar loads, is checked instruction by
    instruction in check_scalar_prefetch.  Returns the set of kernels whose inline asm issues scalar loads."""
    problems, with_sload = [], set()
    for kern, ln, l, in_asm in _walk_kernels(asm_text):
        if not in_asm:
            continue
        op = l.split()[0]
        if _VMEM_LOAD.match(op):
            problems.append("%s line %d: %s" % (kern, ln, l))
        elif op.startswith("s_load_") or op.startswith("s_buffer_load"):
            with_sload.add(kern)
    if problems:
        raise RuntimeError("inline asm issues loads the compiler does not track (%s):\n%s"
                           % (where or "device code", "\n".join(problems[:10])))
    return with_sload


def _kernel_bodies(asm_text):
    """(kernel, [(line number, instruction text)], {label: index of the instruction it precedes}) for every
    function of a device listing."""
    cur, ins, labels = None, [], {}
    for ln, line in enumerate(asm_text.split("\n"), 1):
        l = line.strip()
        if l.startswith("_Z") and ":" in l.split(";")[0]:
            if cur is not None:
                yield cur, ins, labels
            cur, ins, labels = l.split(":")[0], [], {}
            continue
        if cur is None:
            continue
        if l.startswith(".Lfunc_end"):
            yield cur, ins, labels
            cur = None
            continue
        l = l.split(";")[0].strip()
        m = re.match(r"^([.\w$]+):$", l)
        if m:
            labels[m.group(1)] = len(ins)
        elif l and l[0] != ".":
            ins.append((ln, l))
    if cur is not None:
        yield cur, ins, labels


def _scalar_prefetch_step(l, inflight):
    """One instruction against the SGPRs that still have a scalar load in flight before it:
    (in-flight set after it, problem text or None, is a scalar load)."""
    op = l.split()[0]
    toks = re.findall(r"s\[\d+:\d+\]|s\d+", l)
    used = set()
    for t in toks:
        used |= _sregs(t)
    if op.startswith("s_load_dword") or op.startswith("s_buffer_load"):
        # neither the address nor the destination may be in flight: two loads into one register complete in
        # either order
        bad = l if used & inflight else None
        return inflight | (_sregs(toks[0]) if toks else set()), bad, True
    if op == "s_waitcnt" and "lgkmcnt(0)" in l:
        return frozenset(), None, False
    if op == "s_endpgm":
        return frozenset(), ("s_endpgm with scalar loads in flight" if inflight else None), False
    if op in ("s_setpc_b64", "s_swappc_b64") and inflight:
        return inflight, "indirect jump with scalar loads in flight: " + l, False
    return inflight, (l if used & inflight else None), False


def check_scalar_prefetch(asm_text, kernels=None):
    """Static check of the scalar loads in the generated ISA of the kernels that issue them from inline asm.

    The pipelined kernels issue `s_load_dwordx16` from inline asm and wait for it one chunk of math later.
    The compiler does not know that the destination SGPRs are written asynchronously: if register
    pressure makes it spill, copy or reuse them between the load and the next `s_waitcnt lgkmcnt(0)`,
    the late-arriving data lands in whatever lives there by then (a pointer, an exec mask) and the
    kernel faults.  This takes the kernels in `kernels` (a set of mangled names: build() passes every kernel
    whose inline asm issues a scalar load, whatever its name or source file; None takes all) and follows their
    control flow: the set of SGPRs with a load in flight is carried along the fall-through and along every
    `s_branch` / `s_cbranch_*` edge, back edges included, joined by union where paths meet, until nothing
    changes.  The build fails if on any path an instruction reads or writes an SGPR that is still in flight
    (a second load into it included), or if the kernel can end with one in flight.
    Returns the number of scalar loads checked."""
    n_loads, problems = 0, []
    for kern, ins, labels in _kernel_bodies(asm_text):
        if (kernels is not None and kern not in kernels) or not ins:
            continue
        n = len(ins)

        def successors(i):
            op = ins[i][1].split()[0]
            if op == "s_endpgm":
                return []
            m = re.match(r"s_c?branch\w*\s+([.\w$]+)", ins[i][1])
            out = []
            if m:
                if m.group(1) not in labels:
                    raise RuntimeError("scalar-prefetch check: %s line %d branches to an unknown label %s"
                                       % (kern, ins[i][0], m.group(1)))
                out.append(labels[m.group(1)])
            if op != "s_branch" and i + 1 < n:
                out.append(i + 1)
            return out

        state = [None] * n  # in-flight SGPRs before each instruction; None: not reached
        state[0] = frozenset()
        work = [0]
        while work:
            i = work.pop()
            after = frozenset(_scalar_prefetch_step(ins[i][1], state[i])[0])
            for s_ in successors(i):
                joined = after if state[s_] is None else state[s_] | after
                if joined != state[s_]:
                    state[s_] = joined
                    work.append(s_)
        for i, (ln, l) in enumerate(ins):
            if state[i] is None:
                continue
            _, bad, is_load = _scalar_prefetch_step(l, state[i])
            n_loads += is_load
            if bad:
                problems.append((kern, ln, bad))
    if problems:
        msg = "\n".join("%s line %d: %s" % p for p in problems[:10])
        raise RuntimeError("scalar-prefetch check failed: SGPRs touched while their s_load is in flight\n" + msg)
    return n_loads


_ASM_STMT = re.compile(r"(?:\b|__)asm(?:__)?\s*(?:(?:volatile|__volatile__|goto)\s*)*\(")  # asm, __asm__, __asm
SCALAR_LOAD_HELPER = ("sload.h", "sload32")  # the one header, and the name its loading helpers start with


def check_asm_sources(files=None):
    """Source-level twin of check_inline_asm_loads, so that the rule also covers templates nobody instantiates
    yet: no `asm` statement under csrc/ may contain a vector-memory, LDS or returning-atomic load, and `s_load`
    may appear only in the helpers of the one header named above.  `files`: {name: text}, default csrc/*."""
    if files is None:
        files = {}
        for path in sorted(glob.glob(os.path.join(HERE, "csrc", "*"))):
            if path.endswith((".hip", ".h")):
                with open(path) as f:
                    files[os.path.basename(path)] = f.read()
    problems = []
    for name, text in sorted(files.items()):
        # comments out (line breaks kept for the line numbers): prose must not look like code to the scan below
        text = re.sub(r"/\*.*?\*/", lambda c: "\n" * c.group(0).count("\n"), text, flags=re.S)
        text = re.sub(r"//[^\n]*", "", text)
        for m in _ASM_STMT.finditer(text):
            depth, i = 1, m.end()
            while i < len(text) and depth:  # the statement up to its closing parenthesis
                depth += {"(": 1, ")": -1}.get(text[i], 0)
                i += 1
            body = " ".join(re.findall(r'"((?:[^"\\]|\\.)*)"', text[m.end():i]))
            line = text.count("\n", 0, m.start()) + 1
            for ins in re.split(r"\\n|\\t|;", body):
                op = ins.strip().split(" ")[0]
                if _VMEM_LOAD.match(op):
                    problems.append("%s:%d: inline asm issues %s" % (name, line, op))
                elif op.startswith("s_load_") or op.startswith("s_buffer_load"):
                    # the enclosing function: the last definition header before the statement
                    heads = re.findall(r"\b(\w+)\s*\([^;{}]*\)\s*\{", text[:m.start()])
                    if name != SCALAR_LOAD_HELPER[0] or not (heads and heads[-1].startswith(SCALAR_LOAD_HELPER[1])):
                        problems.append("%s:%d: %s outside %s()" % (name, line, op, SCALAR_LOAD_HELPER[1]))
    if problems:
        raise RuntimeError("inline asm may not issue loads the compiler does not track:\n" + "\n".join(problems))
    return len(files)


def kernarg_sgprs(asm_text):
    """{kernel: first SGPR of the pair that holds the kernel-argument pointer at entry}, from the kernel
    descriptors of a listing (user SGPRs are handed out in a fixed order: private segment buffer, dispatch
    pointer, queue pointer, kernel-argument pointer)."""
    out, cur, base = {}, None, 0
    for raw in asm_text.split("\n"):
        l = raw.strip()
        if l.startswith(".amdhsa_kernel "):
            cur, base = l.split()[1], 0
        elif cur and l.startswith(".amdhsa_user_sgpr_"):
            key, _, val = l.partition(" ")
            width = {".amdhsa_user_sgpr_private_segment_buffer": 4, ".amdhsa_user_sgpr_dispatch_ptr": 2,
                     ".amdhsa_user_sgpr_queue_ptr": 2}.get(key)
            if width:
                base += width * int(val)
            elif key == ".amdhsa_user_sgpr_kernarg_segment_ptr" and int(val):
                out[cur] = base
        elif l.startswith(".end_amdhsa_kernel"):
            cur = None
    return out


def isa_digests(asm_text, mask_kernarg_offsets=False):
    """{kernel: (sha256 of its instruction stream, number of instructions)} for a device listing: the instructions
    with their operands, in order, without comments, labels and directives.  Two builds whose digests agree run
    the same machine code for that kernel.  mask_kernarg_offsets: the immediate offset of every scalar load from
    the kernel-argument pointer is left out of the digest, so that two kernels whose argument lists are laid out
    differently and whose code is otherwise the same agree (runs of adjacent argument loads are compared in
    sorted order)."""
    import hashlib
    streams = {}
    karg = kernarg_sgprs(asm_text) if mask_kernarg_offsets else {}
    overwritten = set()
    for kern, _, l, _ in _walk_kernels(asm_text):
        if re.match(r"^[\w.$]+:$", l):  # a label
            continue
        # branch targets carry the function's ordinal in the file (.LBB<ordinal>_<block>): drop the ordinal, so
        # that adding a kernel to a source does not change the digests of the others
        l = re.sub(r"\.LBB\d+_", ".LBB_", " ".join(l.split()))
        if kern in karg and kern not in overwritten:
            l = re.sub(r"^(s_load_dword\w* \S+ s\[%d:%d\],) \S+" % (karg[kern], karg[kern] + 1), r"\1 KERNARG_OFFSET", l)
            # the pair holds the argument pointer until the first instruction (in layout order) that names it as
            # its destination; what is loaded through it afterwards is not a kernel argument
            m = re.match(r"(?!s_cmp|s_bitcmp|s_cbranch)\S+ (s\[\d+:\d+\]|s\d+)\b", l)
            if m and _sregs(m.group(1)) & {karg[kern], karg[kern] + 1}:
                overwritten.add(kern)
        streams.setdefault(kern, []).append(l)
    if mask_kernarg_offsets:
        # adjacent argument loads are independent of each other (each waits at its first use): their order in the
        # listing follows the argument layout too, so a run of them is compared as a set
        for v in streams.values():
            i = 0
            while i < len(v):
                j = i
                while j < len(v) and v[j].endswith(" KERNARG_OFFSET"):
                    j += 1
                v[i:j] = sorted(v[i:j])
                i = j + 1
    return {k: (hashlib.sha256("\n".join(v).encode()).hexdigest()[:16], len(v)) for k, v in streams.items()}


def kernel_resources(asm):
    """Registers, scratch and LDS of every kernel in a device ISA listing, from its code-object metadata:
    {mangled name: {"vgpr", "sgpr", "scratch_bytes", "lds_bytes", "vgpr_spills", "sgpr_spills"}}."""
    fields = {".vgpr_count": "vgpr", ".sgpr_count": "sgpr", ".private_segment_fixed_size": "scratch_bytes",
              ".group_segment_fixed_size": "lds_bytes", ".vgpr_spill_count": "vgpr_spills",
              ".sgpr_spill_count": "sgpr_spills"}
    out, cur = {}, {}
    in_meta = False
    for raw in asm.splitlines():
        l = raw.strip()
        if l.startswith("amdhsa.kernels:"):
            in_meta = True
            continue
        if not in_meta:
            continue
        if l.startswith("- .") or l.startswith("amdhsa."):  # next kernel record, or the end of the list
            if "name" in cur:
                out[cur.pop("name")] = cur
            cur = {}
            l = l[2:] if l.startswith("- ") else l
        key, _, val = l.partition(":")
        key, val = key.strip(), val.strip()
        if key == ".name":
            cur["name"] = val
        elif key in fields:
            cur[fields[key]] = int(val)
    if "name" in cur:
        out[cur.pop("name")] = cur
    return out


def check_hot_kernels(res):
    """The kernels of the headline path must run from registers: no scratch memory, no spilled VGPRs, and
    a register count that leaves the waves per SIMD their launch geometry assumes."""
    want = {  # substring of the mangled name -> most VGPRs per lane
        "dense_fwd_f32_pipeILi64E": 128,                              # 1024 threads: four waves per SIMD
        "dense_fwd_f32_pipeILi32E": 128,
        "dense_bwd_f32_fastILi64ELi512ELi4ELb1ELb1ELb1E": 256,        # 512 threads: two waves per SIMD (all loop forms)
        "dense_bwd_f32_fastILi64ELi512ELi4ELb1ELb0ELb1E": 256,
        "dense_bwd_f32_fastILi64ELi512ELi4ELb0ELb1ELb1E": 256,
        "dense_bwd_f32_fastILi64ELi512ELi4ELb0ELb0ELb1E": 256,
        "dense_bwd_reduce_dkILb1ELb1E": 64,
    }
    problems = []
    for sub, max_vgpr in want.items():
        hits = [(n, r) for n, r in res.items() if sub in n]
        if not hits:
            problems.append("no kernel matches %s" % sub)
        for n, r in hits:
            if r.get("scratch_bytes", 0) or r.get("vgpr_spills", 0) or r.get("vgpr", 0) > max_vgpr:
                problems.append("%s: %s" % (n, r))
    if problems:
        raise RuntimeError("hot-path kernels must not spill:\n" + "\n".join(problems))


def loop_profiles(asm_text, kernel_substr):
    """Instruction mix of every loop (a branch back to an earlier label) of the kernels whose mangled name contains
    kernel_substr: [{"kernel", "first", "last", "valu", "salu", "smem", "lds", "vmem", "waitcnt", "other"}]."""
    out = []
    lines = asm_text.split("\n")
    i = 0
    while i < len(lines):
        l = lines[i]
        if l.startswith("_Z") and kernel_substr in l and ":" in l.split(";")[0]:
            name = l.split(":")[0]
            ins, labels = [], {}
            i += 1
            while i < len(lines) and not lines[i].strip().startswith(".Lfunc_end"):
                t = lines[i].split(";")[0].strip()
                i += 1
                m = re.match(r"^(\.LBB\d+_\d+):", t)
                if m:
                    labels[m.group(1)] = len(ins)
                elif t and t[0] not in ".;" and not t.endswith(":"):
                    ins.append(t)
            for n, t in enumerate(ins):
                m = re.search(r"s_c?branch\w* (\.LBB\d+_\d+)", t)
                if m and labels.get(m.group(1), n + 1) <= n:
                    mix = dict(kernel=name, first=labels[m.group(1)], last=n, valu=0, salu=0, smem=0, lds=0, vmem=0,
                               waitcnt=0, other=0)
                    for u in ins[labels[m.group(1)]:n + 1]:
                        op = u.split()[0]
                        kind = ("valu" if op.startswith("v_") else "waitcnt" if op.startswith("s_waitcnt") else
                                "smem" if op.startswith(("s_load", "s_buffer_load")) else "salu" if op.startswith("s_") else
                                "lds" if op.startswith("ds_") else
                                "vmem" if op.startswith(("buffer_", "global_", "flat_", "scratch_")) else "other")
                        mix[kind] += 1
                    out.append(mix)
        else:
            i += 1
    return out


# The loops that carry the headline path: kernel, pair-elements a lane finishes per iteration, vector-ALU
# instructions the kernel's formulation needs per pair-element, and the most the build accepts (what is above the
# formulation's own count is loop overhead the compiler adds: address arithmetic, staging, the flush).
HOT_LOOPS = (
    ("dense_fwd_f32_pipeILi64ELb0E", 8 * 64, 2, 2.30),                    # eight src rows of 64 columns per lane
    ("dense_fwd_f32_pipeILi32ELb0E", 8 * 32, 2, 2.55),
    ("dense_bwd_f32_fastILi64ELi512ELi4ELb1ELb1ELb1ELi0E", 4 * 64, 3, 3.20),  # four src rows against 64 dst tokens, ranks
    ("dense_bwd_f32_fastILi64ELi512ELi4ELb0ELb0ELb1ELi0E", 4 * 64, 4, 4.25),  # the same with the sign from the difference
    # the pipelined forms of the same loops: two steps per iteration
    ("dense_bwd_f32_fastILi64ELi512ELi4ELb1ELb1ELb1ELi1E", 8 * 64, 3, 3.20),
    ("dense_bwd_f32_fastILi64ELi512ELi4ELb1ELb1ELb1ELi2E", 8 * 64, 3, 3.20),
    ("dense_bwd_f32_fastILi64ELi512ELi4ELb0ELb0ELb1ELi1E", 8 * 64, 4, 4.25),
    ("dense_bwd_f32_fastILi64ELi512ELi4ELb0ELb0ELb1ELi2E", 8 * 64, 4, 4.25),
)


def check_hot_loops(asm_text, table=HOT_LOOPS):
    """Vector-ALU instructions per pair-element in the loops of the headline kernels, from the listing: the loop taken
    for a kernel is the smallest one that holds at least the algorithm's own instructions.  A compiler that starts
    to spend more than the accepted overhead there fails the build instead of showing up as a slower benchmark.
    Returns {kernel substring: instructions per pair-element}."""
    found = {}
    for sub, pairs, own, most in table:
        need = pairs * own
        loops = [p for p in loop_profiles(asm_text, sub) if p["valu"] >= need]
        if not loops:
            raise RuntimeError("hot-loop check: no loop of %s holds %d vector instructions" % (sub, need))
        per = min(p["valu"] for p in loops) / float(pairs)
        if per > most:
            raise RuntimeError("hot-loop check: %s spends %.2f vector instructions per pair-element (accepted: %.2f)"
                               % (sub, per, most))
        found[sub] = per
    return found


def build(verbose=False):
    """Compile, check, link.  A build that fails a compile or a check leaves NO library behind: one from an
    earlier build would no longer match the sources, and none that has not passed the checks may run."""
    try:
        return _build(verbose)
    except BaseException:
        if os.path.exists(LIB):
            os.remove(LIB)
        raise


def _build(verbose):
    sys.path.insert(0, HERE)
    try:
        from isa_checks import check_forbidden  # travels with the sources on the build machine only
    except ImportError:
        print("build: isa_checks.py is not here, the scan for forbidden instructions is skipped "
              "(the inline-asm, scalar-prefetch and spill checks still run)", file=sys.stderr)

        def check_forbidden(text, where=""):
            return None
    check_asm_sources()
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    objs = []
    procs = []
    os.makedirs(os.path.join(HERE, "build"), exist_ok=True)
    for src in sources():
        obj = os.path.join(HERE, "build", os.path.basename(src) + ".o")
        cmd = [hipcc, "--offload-arch=" + ARCH, "-O3", "-std=c++17", "-fPIC",
               "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
               "-I", os.path.join(HERE, "csrc"), "-c", src, "-o", obj]
        if verbose:
            print(" ".join(cmd))
        procs.append((src, subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)))
        objs.append(obj)
    # device ISA listings of every source, for the checks below (in parallel with the compiles)
    listings = []
    for src in sources():
        cmd = [hipcc, "--offload-arch=" + ARCH, "-O3", "-std=c++17", "-Xclang", "-target-feature", "-Xclang",
               "-packed-fp32-ops", "-I", os.path.join(HERE, "csrc"), "-S", "--cuda-device-only", src, "-o", "-"]
        listings.append((src, subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.DEVNULL, text=True)))
    for src, p in procs:
        out, _ = p.communicate()
        # the host pass warns that it does not know the packed-fp32 feature; that is expected
        out = "\n".join(l for l in out.splitlines() if "packed-fp32-ops" not in l)
        if p.returncode != 0:
            raise RuntimeError("hipcc failed on %s:\n%s" % (src, out))
        if verbose and out.strip():
            print(out)
    asm, n, digests = None, 0, []
    for src, p in listings:
        text, _ = p.communicate()
        if p.returncode != 0:
            raise RuntimeError("hipcc -S failed on %s" % src)
        check_forbidden(text, os.path.basename(src))
        # ISA-level safety checks, every kernel of every source: no untracked load from inline asm, and in
        # every kernel whose inline asm issues scalar loads no instruction touches an SGPR still in flight
        prefetchers = check_inline_asm_loads(text, os.path.basename(src))
        n += check_scalar_prefetch(text, prefetchers)
        masked = isa_digests(text, mask_kernarg_offsets=True)
        for kname, (h, cnt) in sorted(isa_digests(text).items()):
            digests.append("%s %s %s %d %s" % (os.path.basename(src), kname, h, cnt, masked[kname][0]))
        if os.path.basename(src) == "dense.hip":
            asm = text
            if not any("dense_fwd_f32_pipe" in kname for kname in prefetchers):
                raise RuntimeError("scalar-prefetch check found no pipelined forward kernel to verify")
    if n < 8:
        raise RuntimeError("scalar-prefetch check verified only %d loads" % n)
    if verbose:
        print("scalar-prefetch check: %d loads verified" % n)
    res = kernel_resources(asm)
    check_hot_kernels(res)
    per_pair = check_hot_loops(asm)
    if verbose:
        print("vector instructions per pair-element:", per_pair)
    with open(os.path.join(HERE, "build", "dense_kernel_resources.txt"), "w") as f:
        for name in sorted(res):
            f.write("%s %s\n" % (name, " ".join("%s=%d" % kv for kv in sorted(res[name].items()))))
    # one line per kernel: source, mangled name, digest of its instruction stream, instruction count, the digest
    # without the offsets of its kernel-argument loads.  Kept under
    # version control, so that the history shows which commits changed which kernel's machine code.
    with open(os.path.join(HERE, "isa_digests.txt"), "w") as f:
        f.write("\n".join(digests) + "\n")
    cmd = [hipcc, "--offload-arch=" + ARCH, "-shared", "-fPIC", "-o", LIB] + objs
    if verbose:
        print(" ".join(cmd))
    subprocess.run(cmd, check=True)
    return LIB


def build_cpu(verbose=False):
    """libl1attn_cpu.so: the API file once, the kernels twice (baseline x86-64 and AVX2 + FMA; the library picks
    the copy the processor supports when it is loaded)."""
    cxx = os.environ.get("CXX", "g++")
    src = os.path.join(HERE, "csrc_cpu")
    out = os.path.join(HERE, "build")
    os.makedirs(out, exist_ok=True)
    common = [cxx, "-O3", "-std=c++17", "-fPIC", "-fopenmp", "-fno-fast-math", "-Wall"]
    jobs = [
        (common + ["-c", os.path.join(src, "l1attn_cpu.cpp")], "l1attn_cpu.o"),
        (common + ["-ffp-contract=off", "-DL1CPU_NS=l1cpu_generic", "-c", os.path.join(src, "l1attn_cpu_kernels.cpp")],
         "l1attn_cpu_kernels_generic.o"),
        (common + ["-mavx2", "-mfma", "-DL1CPU_NS=l1cpu_avx2", "-c", os.path.join(src, "l1attn_cpu_kernels.cpp")],
         "l1attn_cpu_kernels_avx2.o"),
    ]
    procs = []
    for cmd, obj in jobs:
        cmd = cmd + ["-o", os.path.join(out, obj)]
        if verbose:
            print(" ".join(cmd))
        procs.append((cmd, subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)))
    for cmd, p in procs:
        text, _ = p.communicate()
        if p.returncode != 0:
            raise RuntimeError("%s failed:\n%s" % (" ".join(cmd), text))
        if verbose and text.strip():
            print(text)
    subprocess.run([cxx, "-shared", "-fopenmp", "-o", CPU_LIB] + [os.path.join(out, obj) for _, obj in jobs], check=True)
    return CPU_LIB


if __name__ == "__main__":
    print(build(verbose="-v" in sys.argv))
    print(build_cpu(verbose="-v" in sys.argv))
