"""Check the compiled kernels for reads of an accumulator too soon after an inline-assembly MFMA.

    python hexagon-mlir_amd/check_mfma_hazards.py            # compiles csrc/gemm.hip and csrc/calibrate.hip to gfx950
                                                             # assembly and scans it

The 16x16x32 MFMAs of the paired-slab GEMM are `asm volatile` (the accumulator is tied to the destination), so the
compiler's hazard recogniser does not see them and inserts no wait states between such an MFMA and a later read of
its result (`v_accvgpr_read`, a store from an AGPR, ...). The kernel spends the wait states itself at the end of its
K loop; this script verifies, on the assembly the compiler actually produced, that every instruction that reads an
accumulator register is at least NEED wait states behind the last assembly MFMA in layout order (`s_nop k` counts
k + 1, every other instruction 1; an unconditional branch ends the fall-through). Exit status 1 lists offenders.
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


SOURCES = ("gemm.hip", "calibrate.hip")      # the files with MFMAs written as inline assembly


def main():
    bad = {}
    with tempfile.TemporaryDirectory() as tmp:
        for name in SOURCES:
            out = os.path.join(tmp, name[:-4] + ".s")
            cmd = [_build.HIPCC] + _build.FLAGS + ["--cuda-device-only", "-S", os.path.join(_build.CSRC, name), "-o", out]
            r = subprocess.run(cmd, capture_output=True, text=True)
            if r.returncode != 0:
                sys.exit("hipcc failed:\n" + r.stderr)
            bad.update(scan(out))
    for k, v in bad.items():
        print("%s: %d accumulator reads too close to an assembly MFMA, first: %d wait states before `%s`"
              % (k, len(v), v[0][0], v[0][1]))
    print("kernels with accumulator reads too close to an assembly MFMA: %d" % len(bad))
    return 1 if bad else 0


if __name__ == "__main__":
    sys.exit(main())
