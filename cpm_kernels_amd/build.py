"""Build libcpmk_hip.so (hand-written HIP kernels + C ABI) for gfx950 with hipcc.

    python -m cpm_kernels_amd.build          # compile every csrc/*.hip and link

The library is built in-tree (cpm_kernels_amd/lib/) so that it travels with the source
tree; hipcc cross-compiles for gfx950 without a GPU being present.
"""
import os
import shutil
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
BENCH_SRC = os.path.join(HERE, "bench")       # yardstick kernels for bench.py; a library of their own
LIBDIR = os.path.join(HERE, "lib")
LIBNAME = "libcpmk_hip.so"
BENCH_LIBNAME = "libcpmk_ceilings.so"
ARCH = "gfx950"

# No fast-math: correctly rounded fp32 divide is part of the rounding contract.
# Packed fp32 VALU ops are switched off for all device code.
HIPCC_FLAGS = [
    "--offload-arch=" + ARCH, "-O3", "-fPIC", "-std=c++17", "-Wall", "-Wno-unused-function",
    "-Wno-pass-failed", "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
]


def find_hipcc():
    for cand in (os.environ.get("HIPCC"), shutil.which("hipcc"),
                 os.path.join(os.environ.get("ROCM_PATH", "/opt/rocm"), "bin", "hipcc")):
        if cand and os.path.exists(cand):
            return cand
    raise RuntimeError("hipcc not found (set HIPCC or ROCM_PATH)")


def sources():
    return sorted(f for f in os.listdir(CSRC) if f.endswith(".hip"))


def library_path():
    return os.path.join(LIBDIR, LIBNAME)


def bench_library_path():
    return os.path.join(LIBDIR, BENCH_LIBNAME)


def _run(cmd):
    p = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    out = "\n".join(l for l in p.stdout.splitlines()
                    if "packed-fp32-ops" not in l and "warning generated" not in l)
    if p.returncode != 0:
        raise RuntimeError("command failed: %s\n%s" % (" ".join(cmd), out))
    return out


def build_library(verbose=True, jobs=None):
    """Compile every kernel file and link the shared library; always recompiles."""
    hipcc = find_hipcc()
    objdir = os.path.join(LIBDIR, "obj")
    os.makedirs(objdir, exist_ok=True)
    srcs = sources()
    objs = [os.path.join(objdir, s[:-4] + ".o") for s in srcs]

    def compile_one(pair):
        src, obj = pair
        out = _run([hipcc] + HIPCC_FLAGS + ["-c", os.path.join(CSRC, src), "-o", obj])
        if verbose:
            print("[cpmk build] %s%s" % (src, ("\n" + out) if out.strip() else ""), flush=True)

    jobs = jobs or min(8, os.cpu_count() or 1)
    with ThreadPoolExecutor(max_workers=jobs) as ex:
        list(ex.map(compile_one, zip(srcs, objs)))
    tmp = library_path() + ".tmp"
    _run([hipcc, "--offload-arch=" + ARCH, "-shared", "-fPIC", "-o", tmp] + objs)
    os.replace(tmp, library_path())
    if verbose:
        print("[cpmk build] linked %s" % library_path(), flush=True)
    build_bench_library(verbose)
    return library_path()


def build_bench_library(verbose=True):
    """The yardstick kernels bench.py measures beside the library's own (not part of the product)."""
    hipcc = find_hipcc()
    os.makedirs(LIBDIR, exist_ok=True)
    srcs = sorted(os.path.join(BENCH_SRC, f) for f in os.listdir(BENCH_SRC) if f.endswith(".hip"))
    tmp = bench_library_path() + ".tmp"
    _run([hipcc] + HIPCC_FLAGS + ["-shared", "-o", tmp] + srcs)
    os.replace(tmp, bench_library_path())
    if verbose:
        print("[cpmk build] linked %s" % bench_library_path(), flush=True)
    return bench_library_path()


if __name__ == "__main__":
    build_library()
    sys.exit(0)
