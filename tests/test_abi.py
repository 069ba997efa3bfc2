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
    assert hip.df11_version() == 5
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


def test_plan_argument_is_validated_before_anything_else():
    """df11_decode_with_plan rejects a plan number it does not know; the check comes first, so
    no GPU and no valid pointers are needed to see it.  No call changes what a later call does:
    the library keeps no launch state."""
    hip = _native.hip_lib()
    for plan in (4, -2, 100):
        assert hip.df11_decode_with_plan(None, None, None, None, None, None, 2, 16, 16, None, 0, None, plan) == -1
    # an empty stream is a successful no-op under every plan
    for plan in (-1, 0, 1, 2, 3):
        assert hip.df11_decode_with_plan(None, None, None, None, None, None, 2, 0, 0, None, 0, None, plan) == 0


def test_row_decode_arguments_are_validated_without_a_gpu():
    hip = _native.hip_lib()
    rows = hip.df11_decode_rows
    assert rows(None, None, None, None, None, None, 4, 100, 100, None, 0, None, None, 3, 10) == -1     # null pointers
    assert rows(None, None, None, None, None, None, 4, 100, 100, None, 0, None, None, 3, 0) == -1      # no row length
    assert rows(None, None, None, None, None, None, 4, 100, 100, None, 0, None, None, -1, 10) == -1
    assert rows(None, None, None, None, None, None, 4, 100, 100, None, 0, None, None, 0, 10) == 0      # no rows asked for
    assert rows(None, None, None, None, None, None, 4, 0, 0, None, 0, None, None, 3, 10) == 0          # empty stream


def test_launch_plan_follows_stream_size_and_code_lengths():
    """The choice among the compilations of the decode kernel, asked without a GPU for a
    device of 256 CUs: streams of N(0, 0.02) weights (0.324 bitstream bytes per element),
    of one-bit codes (1/8) and of incompressible exponents (1.16)."""
    hip = _native.hip_lib()

    def plan(n_elements, bytes_per_element=0.324, cus=256):
        return hip.df11_launch_plan_name(int(n_elements * bytes_per_element), int(n_elements), cus).decode()

    assert plan(218_103_808) == "deep"                 # a Llama-3-8B decoder block
    assert plan(622_329_856) == "deep"                 # a 151936 x 4096 embedding
    assert plan(4096 * 14336) == "deep/short"          # few sub-blocks per wavefront: priorities by phase
    assert plan(100_000_000) == "deep/short"
    assert plan(120_000_000) == "deep"
    assert plan(4096 * 4096) == "wide"                 # 1.7 rounds of the wide plan, 2.6 of the deep one
    assert plan(8_000_000) == "wide/full"              # within one round of four workgroups per CU
    assert plan(10_000_000) == "wide/full"             # ... also where three per CU would start a second round
    assert plan(12_500_000) == "wide/full"
    assert plan(13_500_000) == "wide"                  # the rest of the wide plan's second round
    assert plan(10_000_000, 0.125) == "wide"           # short codes stay wide
    assert plan(20_000_000) == "deep/small"            # 2.1 rounds of the wide plan
    assert plan(30_000_000) == "deep/small"
    assert plan(100_000) == "deep/small"               # a single round either way
    assert plan(622_329_856, 0.125) == "deepest"       # one-bit codes
    assert plan(4096 * 14336, 0.125) == "deepest/short"
    assert plan(4096 * 4096, 0.125) == "wide"
    for n in (1000, 4096 * 4096, 4096 * 14336, 622_329_856):
        assert plan(n, 1.16) == "wide/dense"           # decode-bound whatever the size
    assert plan(4096 * 14336, cus=64) == "deep"        # the same matrix is 36 rounds on a quarter of the CUs
    assert hip.df11_launch_plan_name(0, 10, 256) == b"" and hip.df11_launch_plan_name(10, 10, 0) == b""
