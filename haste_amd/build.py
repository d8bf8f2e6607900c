"""Builds libhaste_hip.so (the C-ABI library) from haste_amd/csrc/*.hip with hipcc for gfx950.

Usage: python -m haste_amd.build [--force]
"""
import concurrent.futures
import glob
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
OBJ_DIR = os.path.join(HERE, "_obj")
LIB_PATH = os.path.join(HERE, "libhaste_hip.so")

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument", "-Wno-unknown-warning-option",
]


def _compile(src):
    obj = os.path.join(OBJ_DIR, os.path.basename(src) + ".o")
    cmd = [HIPCC] + FLAGS + ["-c", src, "-o", obj]
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError("hipcc failed for %s:\n%s\n%s" % (src, res.stdout, res.stderr))
    return obj


def build(force=True, verbose=False):
    """Compiles every HIP source and links the shared library. Returns its path."""
    sources = sorted(glob.glob(os.path.join(CSRC, "*.hip")))
    if not sources:
        raise RuntimeError("no HIP sources under " + CSRC)
    if not force and os.path.exists(LIB_PATH):
        newest = max(os.path.getmtime(p) for p in glob.glob(os.path.join(CSRC, "*")))
        if os.path.getmtime(LIB_PATH) >= newest:
            return LIB_PATH
    os.makedirs(OBJ_DIR, exist_ok=True)
    with concurrent.futures.ThreadPoolExecutor(max_workers=min(8, len(sources))) as pool:
        objs = list(pool.map(_compile, sources))
    cmd = [HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB_PATH] + objs
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError("link failed:\n%s\n%s" % (res.stdout, res.stderr))
    if verbose:
        print("built", LIB_PATH)
    return LIB_PATH


def build_cpp_api_check(verbose=False):
    """Compiles tests/cpp/api_check.cpp, a C++ caller of include/haste.h, against the library."""
    root = os.path.dirname(HERE)
    src = os.path.join(root, "tests", "cpp", "api_check.cpp")
    out = os.path.join(root, "tests", "cpp", "api_check")
    cmd = [HIPCC, "-O2", "-std=c++17", "-I" + os.path.join(root, "include"), src, "-o", out,
           "-L" + HERE, "-lhaste_hip", "-Wl,-rpath,$ORIGIN/../../haste_amd"]
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError("api_check build failed:\n%s\n%s" % (res.stdout, res.stderr))
    if verbose:
        print("built", out)
    return out


if __name__ == "__main__":
    build(force=True, verbose=True)
    build_cpp_api_check(verbose=True)
