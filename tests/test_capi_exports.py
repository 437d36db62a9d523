"""CPU-side checks of the drop-in boundary: the shared library is built, loads,
and exports every symbol include/pluto_hip.h declares.  No compute is called."""
import ctypes
import os
import re
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "pluto_hip.h")
LIB = os.path.join(ROOT, "pluto_amd", "libpluto_hip.so")


def declared_symbols():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(pluto_hip_[a-z0-9_]+)\s*\(", text)))


@pytest.fixture(scope="module")
def library():
    if not os.path.exists(LIB):
        from pluto_amd import build
        build.build()
    return LIB


def test_header_is_plain_c():
    # the boundary must compile as C: plain pointers and sizes only
    probe = '#include "pluto_hip.h"\nint main(void) { return PLUTO_HIP_BF16 - 1; }\n'
    out = subprocess.run(["gcc", "-std=c11", "-Wall", "-Werror", "-I", os.path.join(ROOT, "include"),
                          "-x", "c", "-", "-fsyntax-only"], input=probe, text=True,
                         capture_output=True)
    assert out.returncode == 0, out.stderr


def test_library_exports_every_declared_symbol(library):
    symbols = declared_symbols()
    assert len(symbols) >= 30
    out = subprocess.run(["nm", "-D", "--defined-only", library], capture_output=True, text=True,
                         check=True).stdout
    exported = set(line.split()[-1] for line in out.splitlines() if " T " in line)
    missing = [s for s in symbols if s not in exported]
    assert not missing, "declared but not exported: %s" % missing


def test_binding_table_matches_header(library):
    from pluto_amd import capi
    assert sorted(capi.SIGNATURES) == declared_symbols()
    handle = capi.lib()   # loads the library and binds every signature
    assert handle.pluto_hip_abi_version() == 3
    assert handle.pluto_hip_target_arch() == b"gfx950"
    assert handle.pluto_hip_error_name(0) == b"PLUTO_HIP_OK"
    assert handle.pluto_hip_error_name(-1) == b"PLUTO_HIP_EINVAL"
    assert handle.pluto_hip_error_name(-2) == b"PLUTO_HIP_ERANGE"
    assert b"workspace" in handle.pluto_hip_error_string(-4)


def test_sizes_and_validation_need_no_gpu(library):
    from pluto_amd import capi
    handle = capi.lib()
    # workspace size arithmetic and argument validation run on the host only
    assert handle.pluto_hip_mha_backward_workspace_bytes(capi.BF16, 16384, 1024, 12, 768) > 25 * 2 ** 20
    assert handle.pluto_hip_mha_backward_workspace_bytes(capi.F32, 1024, 256, 12, 768) == 1024 * 12 * 4
    assert handle.pluto_hip_mha_backward_workspace_bytes(capi.F32, 1000, 256, 12, 768) == 0
    good = capi.attention_params(24, 4, 128, 32, capacity=8192)
    assert handle.pluto_hip_attention_params_validate(good) == 0
    bad = capi.attention_params(24, 5, 128, 32, capacity=8192)
    assert handle.pluto_hip_attention_params_validate(bad) == capi.EINVAL
    assert handle.pluto_hip_gqa_prefill_workspace_bytes(good, 8192) >= 8192 * 24 * 128 * 2
    positions = (ctypes.c_int * 2)(1023, 32767)
    big = capi.attention_params(24, 4, 128, 32, capacity=32768)
    size = handle.pluto_hip_gqa_decode_workspace_bytes(big, 2, positions, 512)
    assert size >= (2 + 64) * 24 * 128 * 4
    p = capi.delta_params(16, 16, 128, 128)
    assert handle.pluto_hip_gdn_scan_workspace_bytes(p, 2, 16384, 64) == 2 * 16 * 256 * 14336   # 14 KiB a chunk and head
    # every compute entry point rejects bad shapes before touching the device
    assert handle.pluto_hip_mha_forward(None, capi.F32, None, 6, 4, 2, 4, None, None, None) == capi.EINVAL
    assert handle.pluto_hip_mha_forward(None, 7, None, 8, 4, 2, 4, None, None, None) == capi.EUNSUPPORTED
    assert handle.pluto_hip_gdn_scan(None, p, 0, 0, 0, None, None, None, None, None, 0, 1.0,
                                     None, None, None, 0) == capi.EINVAL
