"""Builds pluto_amd/libpluto_hip.so (the C ABI + gfx950 kernels, hipcc) and
pluto_amd/libpluto_llm.so (the host-side C++ mirror of the reference's layer
API above that C ABI, g++).

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


CXX = os.environ.get("CXX", "g++")
# The host mirror is plain C++ above the C ABI: no HIP headers, no device code.
HOST_FLAGS = ["-O2", "-g", "-std=c++20", "-fPIC", "-fno-exceptions", "-Wall", "-Wextra",
              "-I" + os.path.join(ROOT, "include"), "-I" + ROOT]
HOST_TEST = os.path.join(ROOT, "build", "bin", "host_tests")
HOST_TEST_SOURCES = os.path.join(ROOT, "tests", "cpp")


def build_device(force=False, verbose=True):
    os.makedirs(OBJ, exist_ok=True)
    headers = glob.glob(os.path.join(CSRC, "*.h")) + glob.glob(
        os.path.join(ROOT, "include", "*.h"))
    sources = sorted(glob.glob(os.path.join(CSRC, "*.hip")))
    # the hand-scheduled instruction streams are generated text
    generators = sorted(glob.glob(os.path.join(CSRC, "gen_*.py")))
    for generator in generators:
        _run([sys.executable, generator])
    headers += glob.glob(os.path.join(CSRC, "*.inc")) + generators
    if force or not _newer(LIB, sources + headers):
        with concurrent.futures.ThreadPoolExecutor(max_workers=8) as pool:
            objects = list(pool.map(lambda s: _compile(s, DEVICE_FLAGS), sources))
        _run([HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB] +
             objects)
        if verbose:
            print("built", LIB)
    return LIB


def _compile_host(src):
    obj = os.path.join(OBJ, "host_" + os.path.basename(src) + ".o")
    _run([CXX] + HOST_FLAGS + ["-c", src, "-o", obj])
    return obj


def build_host(force=False, verbose=True):
    """libpluto_llm.so (the reference's layer API over the C ABI) and the C++
    test runner build/bin/host_tests that tests/test_host_cpp.py drives."""
    os.makedirs(OBJ, exist_ok=True)
    os.makedirs(os.path.dirname(HOST_TEST), exist_ok=True)
    headers = glob.glob(os.path.join(HOST, "*.h")) + glob.glob(
        os.path.join(ROOT, "include", "*.h"))
    sources = sorted(glob.glob(os.path.join(HOST, "*.cc")))
    link = ["-L" + HERE, "-lpluto_hip", "-Wl,-rpath,$ORIGIN"]
    if force or not _newer(HOST_LIB, sources + headers + [LIB]):
        with concurrent.futures.ThreadPoolExecutor(max_workers=8) as pool:
            objects = list(pool.map(_compile_host, sources))
        # libpluto_hip.so pulls in the HIP runtime, which is resolved when a
        # process loads it; the link step only needs our own symbols.
        _run([CXX, "-shared", "-fPIC", "-o", HOST_LIB] + objects + link +
             ["-Wl,--allow-shlib-undefined"])
        if verbose:
            print("built", HOST_LIB)
    tests = sorted(glob.glob(os.path.join(HOST_TEST_SOURCES, "*.cc")))
    test_headers = glob.glob(os.path.join(HOST_TEST_SOURCES, "*.h"))
    if tests and (force or not _newer(HOST_TEST, tests + test_headers + headers + [HOST_LIB])):
        # The runner (test infrastructure, unlike the two libraries above) checks
        # results against the CPU oracle and links it: build that first, so a
        # clean checkout needs no particular order of build steps.
        _run(["make", "-C", os.path.join(ROOT, "oracle"), "-s"])
        with concurrent.futures.ThreadPoolExecutor(max_workers=8) as pool:
            objects = list(pool.map(_compile_host, tests))
        _run([CXX, "-o", HOST_TEST] + objects +
             ["-L" + HERE, "-lpluto_llm", "-lpluto_hip", "-Wl,-rpath,$ORIGIN/../../pluto_amd",
              "-L" + os.path.join(ROOT, "oracle"), "-loracle",
              "-Wl,-rpath,$ORIGIN/../../oracle",
              "-Wl,--allow-shlib-undefined", "-Wl,-rpath,/opt/rocm/lib", "-lpthread"])
        if verbose:
            print("built", HOST_TEST)
    return HOST_LIB


def build(force=False, verbose=True):
    build_device(force, verbose)
    build_host(force, verbose)
    return LIB


if __name__ == "__main__":
    build(force="--force" in sys.argv)
