"""Build libcxgnn_hip.so (hand-written HIP kernels for gfx950) with hipcc.

Usage: python build.py [--force]
Every csrc/*.hip file is compiled to an object and the objects are linked into
lib/libcxgnn_hip.so.  Objects newer than their sources are reused unless
--force is given.
"""
import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
OBJ = os.path.join(HERE, "build")
LIB = os.path.join(HERE, "lib", "libcxgnn_hip.so")
HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
FLAGS = [
    "-O3", "-std=c++17", "-fPIC", "--offload-arch=gfx950",
    # packed-fp32 instructions are switched off for every kernel in this library
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall", "-Wno-unused-function", "-Wno-unused-variable",
    "-I" + os.path.join(HERE, "..", "include"),
]


def _headers_mtime():
    newest = 0.0
    for d in (CSRC, os.path.join(HERE, "..", "include")):
        for f in os.listdir(d):
            if f.endswith((".h", ".hpp")):
                newest = max(newest, os.path.getmtime(os.path.join(d, f)))
    return newest


def build(force=False, jobs=None, verbose=True):
    os.makedirs(OBJ, exist_ok=True)
    os.makedirs(os.path.dirname(LIB), exist_ok=True)
    srcs = sorted(f for f in os.listdir(CSRC) if f.endswith(".hip"))
    hdr_time = _headers_mtime()
    todo = []
    objs = []
    for s in srcs:
        src = os.path.join(CSRC, s)
        obj = os.path.join(OBJ, s[:-4] + ".o")
        objs.append(obj)
        if force or not os.path.exists(obj) or os.path.getmtime(obj) < max(os.path.getmtime(src), hdr_time):
            todo.append((src, obj))

    def compile_one(pair):
        src, obj = pair
        cmd = [HIPCC] + FLAGS + ["-c", src, "-o", obj]
        if verbose:
            print("[build]", os.path.basename(src), flush=True)
        r = subprocess.run(cmd, capture_output=True, text=True)
        out = "\n".join(l for l in (r.stdout + r.stderr).splitlines()
                        if "packed-fp32-ops" not in l)
        if r.returncode != 0:
            raise RuntimeError("hipcc failed for %s:\n%s" % (src, out))
        if out.strip() and verbose:
            print(out)

    jobs = jobs or min(8, max(1, len(todo)))
    with ThreadPoolExecutor(max_workers=jobs) as ex:
        list(ex.map(compile_one, todo))
    if todo or force or not os.path.exists(LIB):
        cmd = [HIPCC, "-shared", "-fPIC", "--offload-arch=gfx950", "-o", LIB] + objs
        r = subprocess.run(cmd, capture_output=True, text=True)
        if r.returncode != 0:
            raise RuntimeError("link failed:\n" + r.stdout + r.stderr)
        if verbose:
            print("[build] linked", LIB, flush=True)
    return LIB


EXT_SRC = os.path.join(HERE, "csrc_ext", "backend_ext.cpp")
EXT_OUT = os.path.join(HERE, "cxgnncomp_backend", "_C.so")


def build_ext(force=False, verbose=True):
    """Compile cxgnncomp_backend/_C.so: the pybind11 / torch C++ host layer (csrc_ext/backend_ext.cpp)
    over libcxgnn_hip.so.  Host code only, built with g++ against the installed torch."""
    import sysconfig
    import torch
    deps = [EXT_SRC, os.path.join(HERE, "..", "include", "cxgnn_hip.h")]
    if not force and os.path.exists(EXT_OUT) and os.path.getmtime(EXT_OUT) >= max(os.path.getmtime(d) for d in deps):
        return EXT_OUT
    tdir = os.path.dirname(torch.__file__)
    cxx = os.environ.get("CXX", "g++")
    cmd = [cxx, "-O2", "-std=c++17", "-fPIC", "-shared", "-Wall", "-Wno-unused-function",
           "-D__HIP_PLATFORM_AMD__=1", "-DUSE_ROCM=1", "-DTORCH_EXTENSION_NAME=_C", "-DTORCH_API_INCLUDE_EXTENSION_H",
           "-D_GLIBCXX_USE_CXX11_ABI=%d" % int(torch._C._GLIBCXX_USE_CXX11_ABI),
           "-I" + os.path.join(tdir, "include"), "-I" + os.path.join(tdir, "include", "torch", "csrc", "api", "include"),
           "-I/opt/rocm/include", "-I" + sysconfig.get_paths()["include"], "-I" + os.path.join(HERE, "..", "include"),
           EXT_SRC, "-o", EXT_OUT,
           "-L" + os.path.join(tdir, "lib"), "-lc10", "-lc10_hip", "-ltorch", "-ltorch_cpu", "-ltorch_hip", "-ltorch_python",
           "-L" + os.path.dirname(LIB), "-lcxgnn_hip",
           "-Wl,-rpath,$ORIGIN/../lib", "-Wl,-rpath," + os.path.join(tdir, "lib")]
    if verbose:
        print("[build] csrc_ext/backend_ext.cpp", flush=True)
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError("compiling the host extension failed:\n" + r.stdout + r.stderr)
    if r.stderr.strip() and verbose:
        print(r.stderr)
    return EXT_OUT


if __name__ == "__main__":
    build(force="--force" in sys.argv)
    build_ext(force="--force" in sys.argv)
