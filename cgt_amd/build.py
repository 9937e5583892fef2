"""Builds libcgt_amd.so (the HIP kernels + C ABI) for gfx950, in-tree.

    python -m cgt_amd.build            # compile every source, link
    python -m cgt_amd.build --if-missing

hipcc cross-compiles without a GPU.  The library lands in cgt_amd/lib/ so it
travels with the source tree; it is never installed elsewhere.
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
LIBPATH = os.path.join(LIBDIR, "libcgt_amd.so")
RT_LIBPATH = os.path.join(LIBDIR, "libcgt_rt.so")
RT_INCLUDE = os.path.join(CSRC, "include")
CXX = os.environ.get("CXX", "g++")
# flags of the reference's native-compile step for host code (cgt/compilation.py:688)
CPP_FLAGS = ["-fvisibility=hidden", "-std=c++11", "-fPIC", "-O3", "-DNDEBUG"]
INCLUDE = os.path.join(ROOT, "include")

SOURCES = ["runtime.hip", "im2col.hip", "pool.hip", "lrn.hip", "gemm.hip", "glue.hip", "elwise.hip", "conv.hip"]

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
ARCH = "gfx950"
# packed fp32 ops are switched off for all device code on this target
HIP_FLAGS = ["--offload-arch=" + ARCH, "-O3", "-std=c++17", "-fPIC", "-fvisibility=hidden",
             "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
             "-Wno-unused-command-line-argument",
             "-I" + INCLUDE, "-I" + CSRC]


def _run(cmd):
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if proc.returncode != 0:
        raise RuntimeError("command failed: %s\n%s" % (" ".join(cmd), proc.stdout))
    # the host pass warns that it does not know the packed-fp32 feature: harmless
    lines = [ln for ln in proc.stdout.splitlines()
             if ln.strip() and "packed-fp32-ops" not in ln and "is not a recognized feature" not in ln]
    return "\n".join(lines)


def _compile(src):
    obj = os.path.join(OBJDIR, os.path.splitext(src)[0] + ".o")
    out = _run([HIPCC] + HIP_FLAGS + ["-c", os.path.join(CSRC, src), "-o", obj])
    return obj, out


def build(verbose=True):
    """Compile every source for gfx950 and link libcgt_amd.so."""
    if not os.path.exists(HIPCC) and shutil.which("hipcc") is None:
        raise RuntimeError("hipcc not found")
    os.makedirs(OBJDIR, exist_ok=True)
    with ThreadPoolExecutor(max_workers=min(8, len(SOURCES))) as ex:
        results = list(ex.map(_compile, SOURCES))
    for (_obj, out) in results:
        if verbose and out:
            print(out)
    objs = [r[0] for r in results]
    tmp = LIBPATH + ".tmp"
    _run([HIPCC, "--offload-arch=" + ARCH, "-shared", "-fPIC", "-o", tmp] + objs)
    os.replace(tmp, LIBPATH)
    if verbose:
        print("built", LIBPATH)
    build_runtime(verbose)
    return LIBPATH


def build_runtime(verbose=True):
    """Host runtime (object model, C API for the host language, interpreter): plain g++."""
    tmp = RT_LIBPATH + ".tmp"
    _run([CXX] + CPP_FLAGS + ["-I" + INCLUDE, "-I" + RT_INCLUDE, os.path.join(CSRC, "cgt_runtime.cpp"),
                              "-shared", "-o", tmp, "-L" + LIBDIR, "-lcgt_amd", "-Wl,-rpath,$ORIGIN"])
    os.replace(tmp, RT_LIBPATH)
    if verbose:
        print("built", RT_LIBPATH)
    return RT_LIBPATH


def main(argv):
    if "--if-missing" in argv and os.path.exists(LIBPATH):
        return 0
    build()
    return 0


if __name__ == "__main__":
    sys.exit(main(sys.argv[1:]))
