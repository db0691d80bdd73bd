"""Builds the native libraries in-tree.

  libbr_hip.so       HIP kernels + C ABI (hipcc, gfx950 only)
  libblackriver.so   C++ host runtime: operator API, tensors, word VM
                     (g++, links libbr_hip.so; never includes a HIP header)
  libbr_probe.so     the bare-MFMA calibration loop bench.py reports beside
                     the GEMM figures (measurement aid; the product never
                     loads it)

``python -m blackriver_amd.build --sanitize`` builds, into lib/sanitize/, the
host runtime and the CPU oracle with AddressSanitizer + UBSan (host code only;
the kernel library is linked as built) for running the CPU test suite under
the sanitizers:
    LD_PRELOAD="$(gcc -print-file-name=libasan.so) $(gcc -print-file-name=libstdc++.so)" \
        BR_SANITIZE=1 ASAN_OPTIONS=detect_leaks=0 python -m pytest tests -m "not gpu"
(libstdc++ is preloaded with libasan so that the interceptor of C++ throws finds
the real function inside an interpreter that is not linked against it.)

Run as ``python -m blackriver_amd.build``.  hipcc cross-compiles for gfx950
without a GPU, so this works on a CPU-only machine.
"""
from __future__ import annotations

import concurrent.futures
import os
import subprocess
import sys

PKG = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(PKG)
INCLUDE = os.path.join(ROOT, "include")
KERNEL_DIR = os.path.join(PKG, "csrc", "kernels")
HOST_DIR = os.path.join(PKG, "csrc", "host")
LIB_DIR = os.path.join(PKG, "lib")
OBJ_DIR = os.path.join(PKG, "build")

BENCH_DIR = os.path.join(PKG, "csrc", "bench")
PROBE_LIB = os.path.join(LIB_DIR, "libbr_probe.so")
SAN_DIR = os.path.join(LIB_DIR, "sanitize")
SAN_FLAGS = ["-fsanitize=address,undefined", "-fno-omit-frame-pointer", "-g", "-O1"]
HIP_LIB = os.path.join(LIB_DIR, "libbr_hip.so")
HOST_LIB = os.path.join(LIB_DIR, "libblackriver.so")

HIPCC_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-I" + INCLUDE, "-I" + KERNEL_DIR,
    # keep the compiler from forming packed-fp32 instructions
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
] + os.environ.get("BR_HIPCC_EXTRA", "").split()   # e.g. BR_HIPCC_EXTRA="-DBR_STREAM=0" for an A/B build
CXX_FLAGS = ["-O2", "-std=c++17", "-fPIC", "-Wall", "-Wno-maybe-uninitialized", "-I" + INCLUDE, "-I" + HOST_DIR]


def _run(cmd):
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    out = "\n".join(l for l in proc.stdout.splitlines()
                    if "is not a recognized feature for this target" not in l)
    if proc.returncode != 0:
        raise RuntimeError("command failed: %s\n%s" % (" ".join(cmd), out))
    return out


def _sources(folder, ext):
    return sorted(os.path.join(folder, f) for f in os.listdir(folder) if f.endswith(ext))


def _stale(obj, src, folder):
    """True when obj is older than src or than any header next to it / in include/."""
    if not os.path.exists(obj):
        return True
    t = os.path.getmtime(obj)
    deps = [src] + _sources(folder, ".hpp") + _sources(INCLUDE, ".h")
    return any(os.path.getmtime(d) > t for d in deps)


def build_kernels(verbose=True, force=True):
    os.makedirs(LIB_DIR, exist_ok=True)
    os.makedirs(OBJ_DIR, exist_ok=True)
    srcs = _sources(KERNEL_DIR, ".hip")
    objs = [os.path.join(OBJ_DIR, os.path.basename(s)[:-4] + ".o") for s in srcs]

    def one(pair):
        src, obj = pair
        if not force and not _stale(obj, src, KERNEL_DIR):
            return ""
        return _run(["hipcc"] + HIPCC_FLAGS + ["-c", src, "-o", obj])

    with concurrent.futures.ThreadPoolExecutor(max_workers=min(8, len(srcs))) as pool:
        for out in pool.map(one, zip(srcs, objs)):
            if verbose and out.strip():
                print(out)
    _run(["hipcc", "--offload-arch=gfx950", "-shared", "-fPIC", "-o", HIP_LIB] + objs)
    if verbose:
        print("built", HIP_LIB)
    return HIP_LIB


def build_host(verbose=True, force=True):
    srcs = _sources(HOST_DIR, ".cpp") if os.path.isdir(HOST_DIR) else []
    if not srcs:
        return None
    os.makedirs(LIB_DIR, exist_ok=True)
    os.makedirs(OBJ_DIR, exist_ok=True)
    objs = [os.path.join(OBJ_DIR, "host_" + os.path.basename(s)[:-4] + ".o") for s in srcs]

    def one(pair):
        src, obj = pair
        if not force and not _stale(obj, src, HOST_DIR):
            return ""
        return _run(["g++"] + CXX_FLAGS + ["-c", src, "-o", obj])

    with concurrent.futures.ThreadPoolExecutor(max_workers=min(8, len(srcs))) as pool:
        for out in pool.map(one, zip(srcs, objs)):
            if verbose and out.strip():
                print(out)
    _run(["g++", "-shared", "-fPIC", "-o", HOST_LIB] + objs +
         ["-L" + LIB_DIR, "-lbr_hip", "-Wl,-rpath,$ORIGIN"])
    if verbose:
        print("built", HOST_LIB)
    return HOST_LIB


def build_probe(verbose=True):
    """The calibration loop of bench.py: its own small library."""
    src = os.path.join(BENCH_DIR, "probe.hip")
    _run(["hipcc"] + HIPCC_FLAGS + ["-shared", "-o", PROBE_LIB, src])
    if verbose:
        print("built", PROBE_LIB)
    return PROBE_LIB


def build_sanitized(verbose=True):
    """Host runtime and CPU oracle with ASan + UBSan (host compilers only)."""
    os.makedirs(SAN_DIR, exist_ok=True)
    srcs = _sources(HOST_DIR, ".cpp")
    host = os.path.join(SAN_DIR, "libblackriver.so")
    _run(["g++"] + CXX_FLAGS + SAN_FLAGS + ["-shared", "-o", host] + srcs +
         ["-L" + LIB_DIR, "-lbr_hip", "-Wl,-rpath,$ORIGIN/.."])
    oracle = os.path.join(SAN_DIR, "libbr_oracle.so")
    _run(["gcc", "-fopenmp", "-march=x86-64-v3", "-fPIC", "-std=c11", "-Wall", "-Wextra"] + SAN_FLAGS +
         ["-shared", "-o", oracle, os.path.join(ROOT, "oracle", "br_oracle.c"), "-lm"])
    if verbose:
        print("built", host)
        print("built", oracle)
    return host, oracle


def build_all(verbose=True, force=True):
    build_kernels(verbose, force)
    build_host(verbose, force)
    build_probe(verbose)


if __name__ == "__main__":
    # `--incremental` recompiles only sources that changed since the last build
    if "--sanitize" in sys.argv:
        if not os.path.exists(HIP_LIB):
            build_kernels()
        build_sanitized()
    else:
        build_all(force="--incremental" not in sys.argv)
    sys.exit(0)
