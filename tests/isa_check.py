"""Checks the generated gfx950 assembly for hazards the compiler does not cover.

The GEMM kernels issue their global->LDS loads from asm statements (the compiler has no
way to express "do not wait for this load before the next LDS read").  The compiler
inserts the wait states the hardware needs between dependent instructions it generates
itself, but it does not look inside an asm statement.  Two requirements of gfx9-family
hardware are therefore checked on the compiler's output:

* a vector instruction that writes a scalar register (v_readfirstlane_b32, v_readlane_b32,
  a compare that writes a scalar pair) must be followed by at least five wait states before
  a vector memory instruction reads that register (here: as part of its buffer descriptor);
* a write of M0 must be followed by at least one wait state before a memory instruction
  that uses M0 as its LDS address.

``scan(text)`` returns a list of human-readable findings (empty when clean);
``compile_to_isa(source)`` produces the text to scan.

A third check concerns speed, not correctness.  The streaming kernels keep several
independent loads in flight per lane.  When each load sits in its own divergent branch
("if this vector is inside the row"), the compiler cannot prove that the load of the
previous loop iteration into the same registers was consumed, and puts ``s_waitcnt
vmcnt(0)`` in front of every load: the loads then run one after the other (the cast kernel
lost 12 % that way, the cast with amax 23 %).  ``memory_order(text)`` lists, per kernel, the
order of loads (L), stores (S), full waits (W) and counted waits (w), so that a test can
require the loads of a kernel to be issued back to back.
"""
import os
import re
import subprocess

HERE = os.path.dirname(os.path.abspath(__file__))

_SGPR = re.compile(r"\bs(\d+)\b|\bs\[(\d+):(\d+)\]")
_MEM = re.compile(r"^\s*(buffer_|global_|flat_|scratch_)")


def _sgprs(text):
    regs = set()
    for m in _SGPR.finditer(text):
        if m.group(1) is not None:
            regs.add(int(m.group(1)))
        else:
            regs.update(range(int(m.group(2)), int(m.group(3)) + 1))
    return regs


def _is_instruction(line):
    s = line.strip()
    return bool(s) and not s.startswith((";", ".", "//")) and not s.endswith(":")


def _wait_states(line):
    m = re.match(r"\s*s_nop\s+(\d+)", line)
    return int(m.group(1)) + 1 if m else 1


def _valu_scalar_dest(line):
    """Scalar registers written by a vector instruction, or an empty set."""
    s = line.strip()
    if not s.startswith("v_"):
        return set()
    ops = s.split(None, 1)
    if len(ops) < 2:
        return set()
    dest = ops[1].split(",")[0]
    if s.startswith(("v_readfirstlane_b32", "v_readlane_b32")) or re.match(r"v_cmp\w*_e64", s) or "_e64" in ops[0]:
        return _sgprs(dest)
    return set()


def scan(text):
    lines = text.splitlines()
    findings = []
    i = 0
    while i < len(lines):
        if "#ASMSTART" not in lines[i]:
            i += 1
            continue
        start = i
        j = i + 1
        while j < len(lines) and "#ASMEND" not in lines[j]:
            j += 1
        block = [l for l in lines[start + 1:j] if _is_instruction(l)]
        i = j + 1
        # wait states inside the block before its first memory instruction, M0 rule on the way
        waited = 0
        m0_age = None
        for l in block:
            if _MEM.match(l):
                used = _sgprs(l)
                if " lds" in l and m0_age is not None and m0_age < 1:
                    findings.append(f"line {start + 1}: M0 written {m0_age} wait states before '{l.strip()}'")
                # look back over the compiler's instructions
                need = 5 - waited
                k = start - 1
                seen = 0
                while k >= 0 and seen < need:
                    if _is_instruction(lines[k]) and "#ASM" not in lines[k]:
                        hit = _valu_scalar_dest(lines[k]) & used
                        if hit:
                            findings.append(
                                f"line {k + 1}: '{lines[k].strip()}' writes s{sorted(hit)} {seen + waited} wait states "
                                f"before '{l.strip()}' (line {start + 1}) reads it; 5 are required")
                        seen += _wait_states(lines[k])
                    k -= 1
                break
            if re.match(r"\s*s_mov_b32\s+m0\b", l):
                m0_age = 0
            else:
                if m0_age is not None:
                    m0_age += _wait_states(l)
            waited += _wait_states(l)
    return findings


def scratch_bytes(text):
    """Kernels of a compiled source that use scratch memory (register spills): {mangled name: bytes per lane}."""
    out = {}
    for m in re.finditer(r"\.amdhsa_kernel (\S+)(.*?)\.end_amdhsa_kernel", text, re.S):
        n = int(re.search(r"private_segment_fixed_size (\d+)", m.group(2)).group(1))
        if n:
            out[m.group(1)] = n
    return out


def m0_sharing(text):
    """Global -> LDS loads that take the m0 a previous asm statement wrote (four loads of a group share one write, their
    immediate offsets tell the regions apart): between such a load and the write of m0 it relies on there must be no
    label (another path could arrive with another m0) and no other write of m0, and the write must be one of ours
    (inside an asm statement).  Returns (number of loads that share, findings)."""
    lines = text.splitlines()
    findings, shared = [], 0
    in_asm = False
    block_writes_m0 = False
    for n, l in enumerate(lines):
        if "#ASMSTART" in l:
            in_asm, block_writes_m0 = True, False
            continue
        if "#ASMEND" in l:
            in_asm = False
            continue
        if not in_asm or not _is_instruction(l):
            continue
        if re.match(r"\s*s_mov_b32\s+m0\b", l):
            block_writes_m0 = True
        if _MEM.match(l) and " lds" in l and not block_writes_m0:
            shared += 1
            k = n - 1
            inside = False
            while k >= 0:
                t = lines[k]
                if "#ASMEND" in t:
                    inside = True
                elif "#ASMSTART" in t:
                    inside = False
                elif re.match(r"\s*\.?[A-Za-z_][\w.$]*:", t):
                    findings.append(f"line {n + 1}: '{l.strip()}' takes m0 from before the label at line {k + 1}")
                    break
                elif _is_instruction(t) and re.match(r"\s*s_\w+\s+m0\b", t):
                    if not (inside and re.match(r"\s*s_mov_b32\s+m0\b", t)):
                        findings.append(f"line {n + 1}: '{l.strip()}' takes m0 from '{t.strip()}' (line {k + 1}), not from an asm statement")
                    break
                k -= 1
            else:
                findings.append(f"line {n + 1}: '{l.strip()}' has no write of m0 before it")
    return shared, findings


def memory_order(text):
    """{kernel symbol: string over L, S, W (s_waitcnt vmcnt(0)), w (s_waitcnt vmcnt(n > 0)), A (atomic)}"""
    out = {}
    for m in re.finditer(r"^(_Z\w+):\s*(?:;.*)?$", text, re.M):
        end = text.find(".Lfunc_end", m.end())
        if end < 0:
            continue
        seq = []
        for line in text[m.end():end].splitlines():
            t = line.strip()
            if not _is_instruction(line):
                continue
            if re.match(r"(global|buffer|flat)_load", t):
                seq.append("L")
            elif re.match(r"(global|buffer|flat)_store", t):
                seq.append("S")
            elif re.match(r"(global|buffer|flat)_atomic", t):
                seq.append("A")
            elif t.startswith("s_waitcnt") and "vmcnt(0)" in t:
                seq.append("W")
            elif t.startswith("s_waitcnt") and "vmcnt(" in t:
                seq.append("w")
        out[m.group(1)] = "".join(seq)
    return out


def compile_to_isa(source, extra_flags=()):
    """Device-only assembly of one HIP source of csrc/ with the build's flags."""
    import importlib.util  # noqa: PLC0415
    spec = importlib.util.spec_from_file_location("_mi355q_build_flags", os.path.join(os.path.dirname(HERE), "gaudi-pytorch-bridge_amd", "build.py"))
    build = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(build)
    HIPCC_FLAGS, CSRC = build.HIPCC_FLAGS, build.CSRC
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    cmd = [hipcc] + [f for f in HIPCC_FLAGS if f != "-fPIC"] + list(extra_flags) + \
          ["--cuda-device-only", "-S", "-x", "hip", os.path.join(CSRC, source), "-o", "-"]
    r = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True)
    if r.returncode != 0:
        raise RuntimeError("hipcc failed: " + r.stderr[-2000:])
    return r.stdout


def exchange_order(text):
    """{kernel symbol: string} for kernels that draw a ticket (global_atomic_add), over
    S / L (global store / load with the sc1 bit, what a device-scope atomic access compiles to), A (the atomic),
    W (s_waitcnt vmcnt(0)), B (s_barrier, runs merged) and F (a cache-wide write-back or invalidate)."""
    out = {}
    for m in re.finditer(r"^(_Z\w+):\s*(?:;.*)?$", text, re.M):
        end = text.find(".Lfunc_end", m.end())
        if end < 0:
            continue
        body = text[m.end():end]
        if "global_atomic_add" not in body:
            continue
        ev = []
        for line in body.splitlines():
            t = line.strip()
            if not _is_instruction(line):
                continue
            if re.match(r"global_store\w*\s.*\bsc1\b", t):
                ev.append("S")
            elif re.match(r"global_load\w*\s.*\bsc1\b", t):
                ev.append("L")
            elif t.startswith("global_atomic_add"):
                ev.append("A")
            elif t.startswith("s_barrier"):
                ev.append("B")
            elif t.startswith("s_waitcnt") and "vmcnt(0)" in t:
                ev.append("W")
            elif re.match(r"buffer_wbl2|buffer_inv|global_wb|global_inv", t):
                ev.append("F")
        out[m.group(1)] = re.sub(r"B+", "B", "".join(ev))
    return out
