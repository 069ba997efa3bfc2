"""The C-ABI libraries load and export every symbol include/df11.h declares (no GPU calls)."""
import os
import re

from dfloat11_amd import _native, build
from tests.df11_cases import locked_make

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared():
    text = open(os.path.join(ROOT, "include", "df11.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(df11_[a-z0-9_]+)\s*\(", text)))


def test_every_declared_symbol_is_exported():
    names = _declared()
    assert "df11_decode" in names and "df11_encode" in names and len(names) >= 12
    hip = _native.hip_lib()
    codec = _native.codec_lib()
    for name in names:
        assert hasattr(hip, name) or hasattr(codec, name), name


def test_version_and_error_strings():
    hip = _native.hip_lib()
    assert hip.df11_version() == 3
    assert hip.df11_error_string(0) == b"ok"
    assert hip.df11_error_string(-1) == b"invalid argument"
    # header + tables + 17 fused LUT rows + (8 sub-blocks per 4096-byte block + 1) positions, rounded to 16
    fixed = 64 + 2048 * 8 + 2048 + 17 * 512
    assert hip.df11_workspace_bytes(0) == fixed + 16
    assert hip.df11_workspace_bytes(4097) == fixed + ((4 * 17 + 15) // 16) * 16
    # the largest stream whose workspace fits the library's static array, and the next larger one
    assert hip.df11_workspace_bytes(533385216) <= 4194304 < hip.df11_workspace_bytes(533385216 + 4096)


def test_argument_validation_needs_no_gpu():
    hip = _native.hip_lib()
    # null pointers / bad sizes are rejected before any HIP call
    assert hip.df11_prepare(None, None, None, None, 4, 100, 100, None, None, None) == -1
    assert hip.df11_decode(None, None, None, None, None, None, 4, 100, 100, None, 0, None) == -1
    assert hip.df11_decode(None, None, None, None, None, None, 4, -1, 100, None, 0, None) == -1
    # empty streams decode to nothing
    assert hip.df11_decode(None, None, None, None, None, None, 4, 0, 0, None, 0, None) == 0


def test_decode_without_gpu_fails_loudly():
    import pytest
    import torch
    from dfloat11_amd import decode
    if torch.cuda.is_available():
        pytest.skip("GPU present")
    t = torch.zeros(2, 256, dtype=torch.uint8)
    e = torch.zeros(16, dtype=torch.uint8)
    with pytest.raises(_native.DF11Error):
        decode.prepare(t, e, e, e, 4)


def test_libraries_are_in_tree():
    assert os.path.dirname(build.HIP_LIB) == os.path.join(ROOT, "dfloat11_amd")
    assert os.path.exists(build.HIP_LIB) and os.path.exists(build.CODEC_LIB)


def test_plain_c_caller_builds_against_the_header():
    """tests/abi/abi_roundtrip.c is C11 compiled by gcc: the header and both
    libraries are usable without a HIP compiler, Python or torch."""
    import subprocess
    d = os.path.join(ROOT, "tests", "abi")
    locked_make(d)
    out = subprocess.run(["ldd", os.path.join(d, "abi_roundtrip")], capture_output=True, text=True, check=True).stdout
    assert "libdf11_hip.so" in out and "libdf11_codec.so" in out and "not found" not in out


def test_launch_plan_override_is_validated():
    hip = _native.hip_lib()
    assert hip.df11_force_launch_plan(3) == -1 and hip.df11_force_launch_plan(-2) == -1
    for plan in (0, 1, 2, -1):
        assert hip.df11_force_launch_plan(plan) == 0
