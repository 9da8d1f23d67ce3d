"""Build step for the native library (libhkv.so) and the CPU oracle.

The library is compiled in-tree with hipcc for gfx950 only; the oracle is the
test checker under oracle/ and is built with gcc.  Nothing here runs a GPU.
"""
import os
import subprocess
import sys

PKG_DIR = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(PKG_DIR)
CSRC = os.path.join(PKG_DIR, "csrc")
INCLUDE = os.path.join(ROOT, "include")
LIB_PATH = os.path.join(PKG_DIR, "libhkv.so")
ORACLE_DIR = os.path.join(ROOT, "oracle")
ORACLE_LIB = os.path.join(ORACLE_DIR, "libhkv_oracle.so")

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
HIP_FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-shared",
    "-Wall",
    "-Wno-unused-function",
    # packed fp32 VALU forms are kept out of every kernel in this build
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
]


def build_library(verbose=True):
    cmd = [HIPCC, *HIP_FLAGS, "-I", INCLUDE, "-I", CSRC,
           os.path.join(CSRC, "hkv_table.hip"), "-o", LIB_PATH]
    if verbose:
        print(" ".join(cmd), flush=True)
    subprocess.check_call(cmd)
    return LIB_PATH


def build_ceilings(verbose=True):
    """The access-pattern ceilings of bench.py --ceilings: a measurement tool in a library of its own."""
    out = os.path.join(PKG_DIR, "libhkv_ceilings.so")
    cmd = [HIPCC, *HIP_FLAGS, os.path.join(CSRC, "hkv_ceilings.hip"), "-o", out]
    if verbose:
        print(" ".join(cmd), flush=True)
    subprocess.check_call(cmd)
    return out


def build_cpp_tests(verbose=True):
    """The C++ test of the drop-in header (tests/cpp/api_test.cpp), linked
    against the in-tree library; a GPU test runs the binary."""
    out = None
    # api_test: the reference's test scenarios; bench_matrix: the reference's benchmark table
    for name in ("api_test", "bench_matrix"):
        src = os.path.join(ROOT, "tests", "cpp", name + ".cpp")
        out = os.path.join(ROOT, "tests", "cpp", name)
        cmd = [HIPCC, "--offload-arch=gfx950", "-O2", "-std=c++17",
               "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
               "-I", INCLUDE, src, "-L", PKG_DIR, "-lhkv",
               "-Wl,-rpath,$ORIGIN/../../hierarchicalkv_amd", "-o", out]
        if verbose:
            print(" ".join(cmd), flush=True)
        subprocess.check_call(cmd)
    return out


def build_oracle(verbose=True):
    cmd = ["make", "-C", ORACLE_DIR, "-B", "libhkv_oracle.so"]
    if verbose:
        print(" ".join(cmd), flush=True)
    subprocess.check_call(cmd)
    return ORACLE_LIB


if __name__ == "__main__":
    what = sys.argv[1:] or ["lib", "ceilings", "oracle", "cpp"]
    if "lib" in what:
        build_library()
    if "ceilings" in what:
        build_ceilings()
    if "cpp" in what:
        build_cpp_tests()
    if "oracle" in what:
        build_oracle()
