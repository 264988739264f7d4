"""Builds libbreccia_kv.so (HIP, gfx950) in-tree with hipcc.

Usage: ``python -m breccia_amd.build`` or ``breccia_amd.build.build()``.  The library is
written next to this file so that it travels with the source tree.
"""
from __future__ import annotations

import os
import shutil
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
OBJ = os.path.join(HERE, "build")
LIB = os.path.join(HERE, "libbreccia_kv.so")
BENCH_LIB = os.path.join(HERE, "libbreccia_kv_bench.so")

SOURCES = ["allocator.cpp", "prefix_tree.cpp", "api.hip", "kv_move.hip", "decode_attn.hip", "decode_attn_mfma.hip", "prefill_attn.hip", "select.hip"]
ARCH = "gfx950"
# Packed-FP32 VALU forms are switched off for every kernel in this library.
HIP_FLAGS = ["--offload-arch=" + ARCH, "-O3", "-std=c++17", "-fPIC", "-Wall", "-Wno-unused-function",
             "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]


def _hipcc() -> str:
    exe = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(exe):
        raise RuntimeError("hipcc not found: cannot build libbreccia_kv.so")
    return exe


def _run(cmd: list[str]) -> None:
    proc = subprocess.run(cmd, capture_output=True, text=True)
    noise = "is not a recognized feature for this target"
    err = "\n".join(l for l in proc.stderr.splitlines() if noise not in l)
    if proc.returncode != 0:
        raise RuntimeError("command failed: %s\n%s\n%s" % (" ".join(cmd), proc.stdout, err))
    if err.strip():
        sys.stderr.write(err + "\n")


def build(verbose: bool = False) -> str:
    """Compile every source for gfx950 and link the shared library.  Returns its path."""
    os.makedirs(OBJ, exist_ok=True)
    hipcc = _hipcc()
    objs = []
    for src in SOURCES:
        obj = os.path.join(OBJ, os.path.splitext(src)[0] + ".o")
        cmd = [hipcc] + HIP_FLAGS + ["-I", os.path.join(HERE, "..", "include"), "-c",
                                     os.path.join(CSRC, src), "-o", obj]
        if verbose:
            print(" ".join(cmd))
        _run(cmd)
        objs.append(obj)
    cmd = [hipcc, "-shared", "-fPIC", "--offload-arch=" + ARCH] + objs + ["-o", LIB]
    if verbose:
        print(" ".join(cmd))
    _run(cmd)
    # the tests' and the benchmark's device plumbing and bandwidth probes: a library of its own
    obj = os.path.join(OBJ, "bench_support.o")
    _run([hipcc] + HIP_FLAGS + ["-I", os.path.join(HERE, "..", "include"), "-c",
                                os.path.join(CSRC, "bench_support.hip"), "-o", obj])
    _run([hipcc, "-shared", "-fPIC", "--offload-arch=" + ARCH, obj, "-o", BENCH_LIB])
    return LIB


def build_cpp_mirror_test(verbose: bool = False) -> str:
    """The C++ test program of the host mirror (tests/cpp); links the library and the oracle."""
    root = os.path.abspath(os.path.join(HERE, ".."))
    src = os.path.join(root, "tests", "cpp", "qsa_mirror_test.cpp")
    out = os.path.join(root, "tests", "cpp", "qsa_mirror_test")
    cmd = ["g++", "-std=c++17", "-O2", "-Wall", src, "-o", out,
           "-L" + HERE, "-lbreccia_kv", "-lbreccia_kv_bench", "-L" + os.path.join(root, "oracle"), "-lbkv_oracle",
           "-Wl,-rpath,$ORIGIN/../../breccia_amd", "-Wl,-rpath,$ORIGIN/../../oracle",
           "-Wl,-rpath,/opt/rocm/lib"]
    if verbose:
        print(" ".join(cmd))
    _run(cmd)
    return out


def build_tree_sanitize_test(verbose: bool = False) -> str:
    """The randomised allocator / prefix-tree exercise (tests/cpp), host code only, built with the
    address and undefined-behaviour sanitizers."""
    root = os.path.abspath(os.path.join(HERE, ".."))
    out = os.path.join(root, "tests", "cpp", "tree_sanitize_test")
    cmd = ["g++", "-std=c++17", "-O1", "-g", "-Wall", "-fsanitize=address,undefined", "-fno-omit-frame-pointer",
           os.path.join(root, "tests", "cpp", "tree_sanitize_test.cpp"), os.path.join(CSRC, "allocator.cpp"),
           os.path.join(CSRC, "prefix_tree.cpp"), "-o", out]
    if verbose:
        print(" ".join(cmd))
    _run(cmd)
    return out


def build_quant_arith_test(verbose: bool = False) -> str:
    """The exhaustive CPU check of the int8 append's code arithmetic for binary16 rows (tests/cpp)."""
    root = os.path.abspath(os.path.join(HERE, ".."))
    out = os.path.join(root, "tests", "cpp", "i8h_f16_codes_exhaustive")
    cmd = ["gcc", "-O2", "-fopenmp", "-ffp-contract=off", out + ".c", "-o", out, "-lm"]
    if verbose:
        print(" ".join(cmd))
    _run(cmd)
    return out


if __name__ == "__main__":
    print(build(verbose=True))
