"""Build libhexmi.so (HIP kernels + C ABI) for gfx950, in-tree.

    python hexagon-mlir_amd/build.py            # incremental
    python hexagon-mlir_amd/build.py --force    # recompile everything

hipcc cross-compiles without a GPU. Objects go to csrc/build/, the library to
hexagon-mlir_amd/hexmi/libhexmi.so (next to the Python loader).
"""
import concurrent.futures
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
INCLUDE = os.path.join(os.path.dirname(HERE), "include")
OUT_LIB = os.path.join(HERE, "hexmi", "libhexmi.so")
OBJ_DIR = os.path.join(CSRC, "build")

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
# -packed-fp32-ops off: hipcc must not form v_pk_*_f32 from float code.
FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument", "-Wno-unknown-warning-option",
    "-I", INCLUDE, "-I", CSRC,
]


# amdgpu-kernarg-preload-count: the kernel arguments arrive in scalar registers when a wave starts instead of being
# loaded by its first instructions. About 0.1 us per launch for the W8A16 kernels (9.19 -> 9.08 us at one row,
# 11.8 -> 11.7 at sixteen, A/B under graph replay); the row kernels, which start tens of thousands of waves, lose by
# it (softmax fp32 [4096, 1024] 6.55 -> 6.89 us), so it is set per file.
EXTRA_FLAGS = {
    "w8a16.hip": ["-mllvm", "-amdgpu-kernarg-preload-count=16"],
    "w8a16_split.hip": ["-mllvm", "-amdgpu-kernarg-preload-count=16"],
}


def flags_for(src):
    return FLAGS + EXTRA_FLAGS.get(src, [])


def _sources():
    return sorted(f for f in os.listdir(CSRC) if f.endswith(".hip"))


def _headers_mtime():
    hs = [os.path.join(CSRC, f) for f in os.listdir(CSRC) if f.endswith(".h")]
    hs += [os.path.join(INCLUDE, f) for f in os.listdir(INCLUDE) if f.endswith(".h")]
    return max(os.path.getmtime(h) for h in hs)


def _compile(src, force, hdr_mtime):
    obj = os.path.join(OBJ_DIR, src[:-4] + ".o")
    path = os.path.join(CSRC, src)
    if (not force and os.path.exists(obj)
            and os.path.getmtime(obj) > max(os.path.getmtime(path), hdr_mtime)):
        return obj, False
    cmd = [HIPCC] + flags_for(src) + ["-c", path, "-o", obj]
    # hipcc reads the source once for the device pass and again for the host pass: a file saved in between gives an
    # object whose launch stubs name kernels its code object does not hold (the first such launch aborts the process)
    for _ in range(3):
        before = os.path.getmtime(path)
        r = subprocess.run(cmd, capture_output=True, text=True)
        if os.path.getmtime(path) == before:
            break
    else:
        raise RuntimeError("%s kept changing while it was compiled" % src)
    if r.returncode != 0:
        raise RuntimeError("hipcc failed for %s:\n%s\n%s" % (src, r.stdout, r.stderr))
    return obj, True


def build(force=False, verbose=True):
    os.makedirs(OBJ_DIR, exist_ok=True)
    hdr = _headers_mtime()
    srcs = _sources()
    with concurrent.futures.ThreadPoolExecutor(max_workers=min(8, len(srcs))) as ex:
        results = list(ex.map(lambda s: _compile(s, force, hdr), srcs))
    objs = [o for o, _ in results]
    rebuilt = any(c for _, c in results)
    if rebuilt or force or not os.path.exists(OUT_LIB):
        cmd = [HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", OUT_LIB] + objs
        r = subprocess.run(cmd, capture_output=True, text=True)
        if r.returncode != 0:
            raise RuntimeError("link failed:\n%s\n%s" % (r.stdout, r.stderr))
    if verbose:
        print("libhexmi.so: %d sources, %s" % (len(srcs), "rebuilt" if rebuilt else "up to date"))
    return OUT_LIB


if __name__ == "__main__":
    build(force="--force" in sys.argv)
