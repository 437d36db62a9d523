"""Builds pluto_amd/libpluto_hip.so (the C ABI + gfx950 kernels) and, for the
host-side C++ mirror of the reference API, pluto_amd/libpluto_llm.so.

Usage: python -m pluto_amd.build [--force]
Sources are compiled with hipcc for gfx950 only; objects go to build/ (git
ignored), the shared libraries stay in-tree next to this file.
"""
import concurrent.futures
import glob
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
CSRC = os.path.join(HERE, "csrc")
HOST = os.path.join(HERE, "host")
OBJ = os.path.join(ROOT, "build", "obj")
LIB = os.path.join(HERE, "libpluto_hip.so")
HOST_LIB = os.path.join(HERE, "libpluto_llm.so")

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
# -packed-fp32-ops is switched off on purpose: the compiler must not form
# v_pk_{add,mul,fma}_f32 from scalar float code.
DEVICE_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++20", "-fPIC", "-fno-exceptions",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    # keep matrix-core accumulators in ordinary VGPRs: the softmax works on them
    # directly, and AGPR accumulators cost a copy per element per tile
    "-mllvm", "-amdgpu-mfma-vgpr-form",
    "-Wno-unused-command-line-argument",
    "-I" + os.path.join(ROOT, "include"), "-I" + CSRC,
]


def _newer(target, sources):
    if not os.path.exists(target):
        return False
    t = os.path.getmtime(target)
    return all(os.path.getmtime(s) <= t for s in sources)


def _run(cmd):
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT,
                          text=True)
    noise = "is not a recognized feature for this target"
    out = "\n".join(l for l in proc.stdout.splitlines() if noise not in l)
    if proc.returncode != 0:
        raise RuntimeError("command failed: %s\n%s" % (" ".join(cmd), out))
    return out


def _compile(src, flags):
    obj = os.path.join(OBJ, os.path.basename(src) + ".o")
    _run([HIPCC] + flags + ["-c", src, "-o", obj])
    return obj


def build(force=False, verbose=True):
    os.makedirs(OBJ, exist_ok=True)
    headers = glob.glob(os.path.join(CSRC, "*.h")) + glob.glob(
        os.path.join(ROOT, "include", "*.h"))
    sources = sorted(glob.glob(os.path.join(CSRC, "*.hip")))
    if force or not _newer(LIB, sources + headers):
        with concurrent.futures.ThreadPoolExecutor(max_workers=8) as pool:
            objects = list(pool.map(lambda s: _compile(s, DEVICE_FLAGS), sources))
        _run([HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB] +
             objects)
        if verbose:
            print("built", LIB)
    host_sources = sorted(glob.glob(os.path.join(HOST, "*.cc")))
    host_headers = glob.glob(os.path.join(HOST, "*.h")) + headers
    if host_sources and (force or not _newer(HOST_LIB, host_sources + host_headers + [LIB])):
        flags = ["-O2", "-std=c++20", "-fPIC", "-fno-exceptions", "-x", "hip",
                 "--offload-arch=gfx950",
                 "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
                 "-Wno-unused-command-line-argument",
                 "-I" + os.path.join(ROOT, "include"), "-I" + ROOT]
        with concurrent.futures.ThreadPoolExecutor(max_workers=8) as pool:
            objects = list(pool.map(lambda s: _compile(s, flags), host_sources))
        _run([HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", HOST_LIB] +
             objects + ["-L" + HERE, "-lpluto_hip", "-Wl,-rpath,$ORIGIN"])
        if verbose:
            print("built", HOST_LIB)
    return LIB


if __name__ == "__main__":
    build(force="--force" in sys.argv)
