"""Builds libgnnhip.so (the gfx950 HIP kernels + C ABI) in-tree with hipcc.

Usage: python -m graphnn_amd.build [--force]
The library is written to graphnn_amd/lib/libgnnhip.so.  hipcc cross-compiles
for gfx950 without a GPU present.
"""
import os
import shutil
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
CSRC = os.path.join(HERE, "csrc")
LIBDIR = os.path.join(HERE, "lib")
OBJDIR = os.path.join(LIBDIR, "obj")
LIB = os.path.join(LIBDIR, "libgnnhip.so")

ARCH = "gfx950"
# packed-fp32 ops are switched off: hipcc would otherwise form v_pk_*_f32 from plain float code.
HIPCC_FLAGS = [
    "--offload-arch=" + ARCH, "-O3", "-std=c++17", "-fPIC",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall", "-Wno-unused-function",
    "-I", os.path.join(ROOT, "include"), "-I", CSRC,
]


def _hipcc():
    exe = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(exe):
        raise RuntimeError("hipcc not found; the gnnhip library cannot be built")
    return exe


def sources():
    return sorted(os.path.join(CSRC, f) for f in os.listdir(CSRC) if f.endswith(".hip"))


def _compile_one(args):
    hipcc, src, obj = args
    cmd = [hipcc] + HIPCC_FLAGS + ["-c", src, "-o", obj]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError("hipcc failed on %s:\n%s\n%s" % (src, r.stdout, r.stderr))
    return r.stderr


def build(force=True, verbose=True, jobs=8):
    """Compile every .hip source and link libgnnhip.so.  Returns the library path."""
    hipcc = _hipcc()
    os.makedirs(OBJDIR, exist_ok=True)
    srcs = sources()
    headers = [os.path.join(CSRC, f) for f in os.listdir(CSRC) if f.endswith(".h")]
    headers.append(os.path.join(ROOT, "include", "gnnhip.h"))
    newest_header = max(os.path.getmtime(h) for h in headers)
    todo = []
    objs = []
    for s in srcs:
        o = os.path.join(OBJDIR, os.path.basename(s)[:-4] + ".o")
        objs.append(o)
        stale = (not os.path.exists(o)) or os.path.getmtime(o) < max(os.path.getmtime(s), newest_header)
        if force or stale:
            todo.append((hipcc, s, o))
    with ThreadPoolExecutor(max_workers=max(1, min(jobs, len(todo) or 1))) as ex:
        for warn in ex.map(_compile_one, todo):
            if verbose and warn.strip():
                # the host pass does not know the packed-fp32 target feature; that warning is expected
                lines = [l for l in warn.splitlines() if "packed-fp32-ops" not in l and l.strip()]
                if lines:
                    print("\n".join(lines), file=sys.stderr)
    if todo or not os.path.exists(LIB):
        cmd = [hipcc, "--offload-arch=" + ARCH, "-shared", "-fPIC", "-o", LIB] + objs
        r = subprocess.run(cmd, capture_output=True, text=True)
        if r.returncode != 0:
            raise RuntimeError("link failed:\n%s\n%s" % (r.stdout, r.stderr))
    if verbose:
        print("built %s (%d sources compiled)" % (LIB, len(todo)))
    return LIB


if __name__ == "__main__":
    build(force="--force" in sys.argv)
