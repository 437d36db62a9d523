"""Drives the C++ tests of the host API (pluto_amd/host: the reference's layer
classes over the C ABI).  The cases live in tests/cpp/*.cc and mirror the
reference's own *_test.cc files; this wrapper runs the compiled runner once for
the CPU-only suites and once, on a GPU, for everything."""
import os
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
RUNNER = os.path.join(ROOT, "build", "bin", "host_tests")


@pytest.fixture(scope="module")
def runner():
    if not os.path.exists(RUNNER):
        from pluto_amd import build
        build.build_host()
    assert os.path.exists(RUNNER), "host test runner was not built"
    return RUNNER


def run(runner, *args, timeout):
    proc = subprocess.run([runner, *args], stdout=subprocess.PIPE, stderr=subprocess.STDOUT,
                          text=True, timeout=timeout)
    print(proc.stdout)
    return proc


def test_cpu_suites(runner):
    proc = run(runner, "--cpu", timeout=60)
    assert proc.returncode == 0, proc.stdout[-4000:]
    assert " 0 failed" in proc.stdout


def test_every_reference_class_has_cases(runner):
    listed = run(runner, "--list", timeout=60).stdout.split()
    suites = {name.split(".")[0] for name in listed}
    assert {"AttentionLayerTest", "AttentionOpsTest", "QwenAttentionTest", "SequenceDeltaNetTest",
            "KeyValueCacheTest", "BufferTest", "ExecutorTest", "PageLockedHostArrayTest",
            "ActivationTypeCpu", "StatusCpu", "LayerHooksTest", "DeltaNetLayerTest",
            "DecoderBranchTest", "DecoderStepTest"} <= suites


@pytest.mark.gpu
def test_all_suites_on_the_gpu(runner):
    proc = run(runner, timeout=600)
    failed = [line for line in proc.stdout.splitlines() if line.startswith("[ FAIL ]")]
    assert proc.returncode == 0 and not failed, "\n".join(failed) + "\n" + proc.stdout[-6000:]
