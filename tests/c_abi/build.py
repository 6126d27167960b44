"""Compile the C++ callers of the C ABI (tests/c_abi/*.cpp) against include/hexmi.h and libhexmi.so.

    python tests/c_abi/build.py

hipcc is used as the host C++ compiler (the programs hold no device code: they call the HIP runtime for memory and a
stream, and libhexmi.so for the operators). Binaries go to tests/c_abi/bin/ and find the library through a
relative run path, so the tree can be moved.
"""
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
INCLUDE = os.path.join(ROOT, "include")
LIB_DIR = os.path.join(ROOT, "hexagon-mlir_amd", "hexmi")
BIN_DIR = os.path.join(HERE, "bin")
HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
PROGRAMS = ("matmul_caller", "attention_caller")


def binary(name):
    return os.path.join(BIN_DIR, name)


def build(force=False):
    os.makedirs(BIN_DIR, exist_ok=True)
    for name in PROGRAMS:
        src, out = os.path.join(HERE, name + ".cpp"), binary(name)
        deps = [src, os.path.join(HERE, "tensor_io.h"), os.path.join(INCLUDE, "hexmi.h")]
        if not force and os.path.exists(out) and os.path.getmtime(out) > max(os.path.getmtime(d) for d in deps):
            continue
        cmd = [HIPCC, "-O2", "-std=c++17", "--offload-arch=gfx950", "-I", INCLUDE, "-I", HERE, src, "-o", out,
               "-L", LIB_DIR, "-lhexmi", "-Wl,-rpath,$ORIGIN/../../../hexagon-mlir_amd/hexmi"]
        r = subprocess.run(cmd, capture_output=True, text=True)
        if r.returncode != 0:
            raise RuntimeError("hipcc failed for %s:\n%s\n%s" % (name, r.stdout, r.stderr))
    return [binary(n) for n in PROGRAMS]


if __name__ == "__main__":
    for path in build(force="--force" in sys.argv):
        print(path)
