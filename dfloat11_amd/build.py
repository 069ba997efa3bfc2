"""Compiles the native libraries in-tree.

libdf11_hip.so          HIP kernels + device C-ABI, hipcc --offload-arch=gfx950
libdf11_codec.so        host codec C-ABI, g++
libcalibration_copy.so  a plain copy kernel for the benchmark's counter calibration (no part
                        of the interface; nothing in the package loads it)
"""
import os
import shutil
import subprocess

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
HIP_LIB = os.path.join(HERE, "libdf11_hip.so")
CODEC_LIB = os.path.join(HERE, "libdf11_codec.so")
CALIBRATION_LIB = os.path.join(HERE, "libcalibration_copy.so")

HIPCC_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-shared",
    # keep the compiler from forming packed-FP32 instructions
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
]
# x86-64-v2 rather than native: the library is built on one host and run on another
CXX_FLAGS = ["-O3", "-march=x86-64-v2", "-std=c++17", "-fPIC", "-shared", "-pthread", "-Wall", "-Wextra"]


def _hipcc():
    return shutil.which("hipcc") or "/opt/rocm/bin/hipcc"


def build_hip(verbose=False):
    cmd = [_hipcc(), *HIPCC_FLAGS, "-o", HIP_LIB, os.path.join(CSRC, "df11_decode.hip")]
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError("hipcc failed:\n" + res.stdout + res.stderr)
    if verbose:
        print(" ".join(cmd))
    return HIP_LIB


def build_calibration(verbose=False):
    cmd = [_hipcc(), *HIPCC_FLAGS, "-o", CALIBRATION_LIB, os.path.join(CSRC, "calibration_copy.hip")]
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError("hipcc failed:\n" + res.stdout + res.stderr)
    if verbose:
        print(" ".join(cmd))
    return CALIBRATION_LIB


def build_codec(verbose=False):
    cmd = [shutil.which("g++") or "g++", *CXX_FLAGS, "-o", CODEC_LIB, os.path.join(CSRC, "df11_codec.cpp")]
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError("g++ failed:\n" + res.stdout + res.stderr)
    if verbose:
        print(" ".join(cmd))
    return CODEC_LIB


def build_all(verbose=False):
    return build_hip(verbose), build_codec(verbose), build_calibration(verbose)


if __name__ == "__main__":
    build_all(verbose=True)
