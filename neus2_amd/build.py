"""Builds libneus2_amd.so (HIP kernels + C ABI) for gfx950 with hipcc, in-tree.

    python -m neus2_amd.build            # incremental
    python -m neus2_amd.build --force    # rebuild everything
"""
import concurrent.futures as cf
import glob
import os
import subprocess
import sys

PKG = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(PKG)
CSRC = os.path.join(PKG, "csrc")
OBJ = os.path.join(CSRC, "build")
LIB = os.path.join(PKG, "libneus2_amd.so")

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-fvisibility=hidden",
    # packed fp32 VALU ops are kept out of the device code on purpose
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-I", os.path.join(ROOT, "include"), "-I", CSRC,
    "-Wall", "-Wno-unused-function",
]


def _newer(src_files, target):
    if not os.path.exists(target):
        return True
    t = os.path.getmtime(target)
    return any(os.path.getmtime(s) > t for s in src_files)


def _compile(src, obj):
    r = subprocess.run([HIPCC, *FLAGS, "-c", src, "-o", obj], capture_output=True, text=True)
    # the host pass warns that it does not know the packed-fp32 feature: harmless
    err = "\n".join(l for l in r.stderr.splitlines() if "packed-fp32-ops" not in l)
    if r.returncode != 0:
        raise RuntimeError(f"hipcc failed on {src}:\n{err}")
    return err


def build_library(force=False, verbose=False):
    os.makedirs(OBJ, exist_ok=True)
    srcs = sorted(glob.glob(os.path.join(CSRC, "*.hip")))
    hdrs = glob.glob(os.path.join(CSRC, "*.h")) + glob.glob(os.path.join(ROOT, "include", "*.h"))
    jobs = []
    for s in srcs:
        o = os.path.join(OBJ, os.path.basename(s)[:-4] + ".o")
        if force or _newer([s] + hdrs, o):
            jobs.append((s, o))
    with cf.ThreadPoolExecutor(max_workers=min(8, max(1, len(jobs)))) as ex:
        for (s, _), warn in zip(jobs, ex.map(lambda j: _compile(*j), jobs)):
            if verbose and warn.strip():
                print(f"[{os.path.basename(s)}]\n{warn}", file=sys.stderr)
    objs = [os.path.join(OBJ, os.path.basename(s)[:-4] + ".o") for s in srcs]
    if force or jobs or _newer(objs, LIB):
        r = subprocess.run([HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB, *objs],
                           capture_output=True, text=True)
        if r.returncode != 0:
            raise RuntimeError("link failed:\n" + r.stderr)
    return LIB


SHIM_SRC = os.path.join(ROOT, "tests", "cpp", "shim_check.cpp")
SHIM_BIN = os.path.join(ROOT, "tests", "cpp", "shim_check")


def build_shim_check(force=False):
    """The C++ program that drives the library through include/neus2_amd.hpp (host compiler only: the shim and the
    C ABI carry no device code)."""
    deps = [SHIM_SRC, LIB] + glob.glob(os.path.join(ROOT, "include", "*.h*"))
    if not force and not _newer(deps, SHIM_BIN):
        return SHIM_BIN
    cmd = [os.environ.get("CXX", "g++"), "-std=c++17", "-O1", "-Wall", "-D__HIP_PLATFORM_AMD__", "-I", os.path.join(ROOT, "include"),
           "-I", "/opt/rocm/include", SHIM_SRC, "-o", SHIM_BIN, "-L", PKG, "-lneus2_amd", "-L", "/opt/rocm/lib", "-lamdhip64",
           "-Wl,-rpath,$ORIGIN/../../neus2_amd", "-Wl,-rpath,/opt/rocm/lib"]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError("shim_check build failed:\n" + r.stderr)
    return SHIM_BIN


if __name__ == "__main__":
    print(build_library(force="--force" in sys.argv, verbose=True))
    print(build_shim_check(force="--force" in sys.argv))
