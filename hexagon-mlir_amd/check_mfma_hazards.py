"""Check the compiled kernels for register hazards that the compiler cannot see through inline assembly, and for
register spills where the code cannot afford them.

    python hexagon-mlir_amd/check_mfma_hazards.py            # compiles the sources below to gfx950 assembly
                                                             # and scans it

1. Reads of an accumulator too soon after an inline-assembly MFMA. The 16x16x32 MFMAs of the paired-slab GEMM are
`asm volatile` (the accumulator is tied to the destination), so the compiler's hazard recogniser does not see them
and inserts no wait states between such an MFMA and a later read of its result (`v_accvgpr_read`, a store from an
AGPR, ...). The kernel spends the wait states itself at the end of its K loop; `scan` verifies, on the assembly the
compiler actually produced, that every instruction that reads an accumulator register is at least NEED wait states
behind the last assembly MFMA in layout order (`s_nop k` counts k + 1, every other instruction 1; an unconditional
branch ends the fall-through).

2. A matrix instruction that reads a register too soon after a vector instruction wrote it, where one of the two is
inline assembly. A matrix instruction must not read a vector register in the two issue slots after a vector
instruction wrote it; the compiler keeps that distance for the pairs it can see, but it sees neither the writes of
the SDWA int8 -> fp16 conversions (hexmi_common.h) nor the reads of an assembly MFMA. One slot was enough wherever
the matrix pipe was idle and lost the last converted byte where the pipe was still busy with the MFMA before.
`scan_conversions` verifies that no such pair is closer than CVT_NEED slots.

Exit status 1 lists offenders.
"""
import os
import re
import subprocess
import sys
import tempfile

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, HERE)
import build as _build  # noqa: E402  (the compiler and flags the library is built with)

NEED = 19          # wait states before a VALU read of the result of the longest (16-pass) matrix instruction


def scan(asm_path):
    name, since, in_asm, bad = None, 10 ** 9, False, {}
    with open(asm_path) as f:
        for line in f:
            t = line.strip()
            m = re.match(r"^(_Z\S+):", line)
            if m:
                name, since = m.group(1), 10 ** 9
                continue
            if t.startswith(";;#ASMSTART"):
                in_asm = True
                continue
            if t.startswith(";;#ASMEND"):
                in_asm = False
                continue
            if not t or t[0] in ";." or t.endswith(":"):
                continue
            op = t.split()[0]
            if op.startswith("v_mfma"):
                if in_asm:
                    since = 0
                continue
            if op in ("s_branch", "s_endpgm", "s_setpc_b64"):
                since = 10 ** 9
                continue
            if op == "s_nop":
                since += int(t.split()[1]) + 1
                continue
            sources = t.split(None, 1)[1].split(",", 1)[1] if "," in t else ""
            if re.search(r"\ba\[?\d", sources) and since < NEED:
                bad.setdefault(name, []).append((since, t))
            since += 1
    return bad


CVT_NEED = 2       # issue slots between a vector write of a register and a matrix instruction that reads it
_MFMA_SRC = re.compile(r"v_mfma\S+ \S+, v\[(\d+):(\d+)\], v\[(\d+):(\d+)\]")
_VALU_DST = re.compile(r"(v_\w+) v(?:\[(\d+):(\d+)\]|(\d+))\b")


def scan_conversions(asm_path):
    """{kernel: [(slots, assembly line)]}: a matrix instruction reads a vector register fewer than CVT_NEED issue
    slots after a vector instruction wrote it, where one of the two sits inside an asm statement (the compiler
    spaces the pairs it can see)."""
    with open(asm_path) as f:
        lines = f.read().split("\n")
    name, in_asm, bad = None, False, {}
    recent = []                                             # (slots ago is implied by position) [(lo, hi, hidden, line)]
    for i, line in enumerate(lines):
        t = line.strip()
        m = re.match(r"^(_Z\S+):", line)
        if m:
            name, recent = m.group(1), []
            continue
        if t.startswith(";;#ASMSTART"):
            in_asm = True
            continue
        if t.startswith(";;#ASMEND"):
            in_asm = False
            continue
        if not t or t[0] in ";.":
            continue
        if t.endswith(":"):
            recent = []                                     # a label: other paths arrive here, no distance to measure
            continue
        op = t.split()[0]
        if op.startswith("v_mfma"):
            mm = _MFMA_SRC.match(t)
            if mm:
                a0, a1, b0, b1 = map(int, mm.groups())
                for age, (lo, hi, hidden, at) in enumerate(reversed(recent)):
                    if age >= CVT_NEED:
                        break
                    if lo is not None and (hidden or in_asm) and (lo <= a1 and hi >= a0 or lo <= b1 and hi >= b0):
                        bad.setdefault(name, []).append((age, at))
            recent.append((None, None, False, i + 1))
        elif op == "s_nop":
            recent += [(None, None, False, i + 1)] * (int(t.split()[1]) + 1)
        elif op in ("s_branch", "s_endpgm", "s_setpc_b64") or op.startswith("s_cbranch"):
            recent = []
        else:
            md = _VALU_DST.match(t)
            if md and not md.group(1).startswith("v_accvgpr_write"):
                lo = int(md.group(2) if md.group(2) is not None else md.group(4))
                hi = int(md.group(3) if md.group(3) is not None else md.group(4))
                recent.append((lo, hi, in_asm, i + 1))
            else:
                recent.append((None, None, False, i + 1))
        recent = recent[-4:]
    return bad


# 3. Register spills in kernels whose waits are counted by hand. These kernels wait for their global -> LDS copies
# with `s_waitcnt vmcnt(n)` immediates that assume every outstanding vector-memory operation is one of those copies; a
# spilled register is reloaded with a vector-memory operation of its own, the count is off by one from then on and
# a wave reads a stage before its data is there (seen: 192 bytes of scratch in one variant, wrong sums).
COUNTED_WAITS = ("w8a16_mid_kernel", "w8a16_split_kernel", "w8a16_persist_kernel", "gemm_kernel_k64")


def scan_scratch(asm_path):
    """{kernel: [assembly lines]} for kernels of COUNTED_WAITS with a scratch access between their first and their
    last global -> LDS copy in layout order (before the first and behind the last, a spill disturbs no count)."""
    bad, name, copies, scratch = {}, None, [], []

    def close():
        if name and copies and any(k in name for k in COUNTED_WAITS):
            inside = [n for n in scratch if copies[0] < n < copies[-1]]
            if inside:
                bad[name] = inside

    with open(asm_path) as f:
        for n, line in enumerate(f, 1):
            m = re.match(r"^(_Z\S+):", line)
            if m:
                close()
                name, copies, scratch = m.group(1), [], []
                continue
            t = line.strip()
            if re.match(r"(global_load_lds|buffer_load\S*)\b.*\blds\b", t) or t.startswith("global_load_lds"):
                copies.append(n)
            elif t.startswith("scratch_"):
                scratch.append(n)
    close()
    return bad


SOURCES = ("gemm.hip", "calibrate.hip")      # the files with MFMAs written as inline assembly
CVT_SOURCES = ("gemm.hip", "calibrate.hip", "w8a16.hip", "w8a16_split.hip")   # asm conversions or asm MFMAs


def _assembly(name, tmp):
    out = os.path.join(tmp, name[:-4] + ".s")
    cmd = [_build.HIPCC] + _build.flags_for(name) + ["--cuda-device-only", "-S", os.path.join(_build.CSRC, name), "-o", out]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        sys.exit("hipcc failed:\n" + r.stderr)
    return out


def main():
    import concurrent.futures
    bad, bad_cvt, bad_scratch = {}, {}, {}
    names = sorted(set(SOURCES) | set(CVT_SOURCES))
    with tempfile.TemporaryDirectory() as tmp:
        with concurrent.futures.ThreadPoolExecutor(max_workers=len(names)) as ex:
            outs = dict(zip(names, ex.map(lambda n: _assembly(n, tmp), names)))
        for name in SOURCES:
            bad.update(scan(outs[name]))
        for name in CVT_SOURCES:
            bad_cvt.update(scan_conversions(outs[name]))
        for name in names:
            bad_scratch.update(scan_scratch(outs[name]))
    for k, v in bad.items():
        print("%s: %d accumulator reads too close to an assembly MFMA, first: %d wait states before `%s`"
              % (k, len(v), v[0][0], v[0][1]))
    for k, v in bad_cvt.items():
        print("%s: %d vector writes too close to the MFMA that reads them, first: %d slot(s), assembly line %d"
              % (k, len(v), v[0][0], v[0][1]))
    for k, v in bad_scratch.items():
        print("%s: %d scratch accesses among the copies of a kernel that counts its vector-memory operations by "
              "hand, first at assembly line %d" % (k, len(v), v[0]))
    print("kernels with accumulator reads too close to an assembly MFMA: %d" % len(bad))
    print("kernels with a vector write too close to the MFMA that reads it: %d" % len(bad_cvt))
    print("kernels with counted waits that spill registers: %d" % len(bad_scratch))
    return 1 if bad or bad_cvt or bad_scratch else 0


if __name__ == "__main__":
    sys.exit(main())
