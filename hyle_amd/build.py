"""Builds hyle_amd/libhyle_hip.so: the gfx950 kernels plus the C ABI of include/hyle_hip.h.

hipcc cross-compiles for gfx950 without a GPU.  Objects are compiled in parallel and linked
in-tree so the library travels with the source tree.
"""
from __future__ import annotations

import os
import shutil
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
OBJ = os.path.join(HERE, "build")
LIB = os.path.join(HERE, "libhyle_hip.so")

SOURCES = ["plan.hip", "elementwise.hip", "norm.hip", "norm_exact_rms.hip", "norm_exact_layer.hip", "softmax.hip", "softmax_exact.hip", "reduce.hip", "argmax.hip", "topk.hip", "q8_0.hip", "gguf_k.hip", "gguf_matvec.hip", "gguf_matvec_q8.hip", "cast.hip", "select_fill.hip", "concat.hip", "gather.hip", "sampling.hip", "rope.hip", "file_stream.hip", "backend.hip"]

# -ffp-contract=off: (a + b) * s and x * scale + mask keep two roundings, as the reference does.
# packed-fp32 instructions are switched off for every device function.
FLAGS = [
    "-O3", "--offload-arch=gfx950", "-std=c++17", "-fPIC", "-ffp-contract=off", "-fvisibility=hidden",
    "-Wall", "-Wno-unused-function",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
]


def _hipcc() -> str:
    found = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(found):
        raise RuntimeError("hipcc not found: the gfx950 library cannot be built")
    return found


def _compile(source: str) -> str:
    obj = os.path.join(OBJ, source.replace(".hip", ".o"))
    cmd = [_hipcc(), *FLAGS, "-c", os.path.join(CSRC, source), "-o", obj]
    done = subprocess.run(cmd, capture_output=True, text=True)
    noise = "packed-fp32-ops"
    err = "\n".join(line for line in done.stderr.splitlines() if noise not in line)
    if done.returncode != 0:
        raise RuntimeError(f"hipcc failed on {source}:\n{err}")
    if err.strip():
        sys.stderr.write(err + "\n")
    return obj


def build(verbose: bool = True) -> str:
    os.makedirs(OBJ, exist_ok=True)
    with ThreadPoolExecutor(max_workers=min(8, len(SOURCES))) as pool:
        objects = list(pool.map(_compile, SOURCES))
    link = [_hipcc(), "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB, *objects]
    done = subprocess.run(link, capture_output=True, text=True)
    if done.returncode != 0:
        raise RuntimeError(f"link failed:\n{done.stderr}")
    if verbose:
        print(f"built {LIB} ({os.path.getsize(LIB)} bytes)")
    return LIB


HOST_TEST_SOURCE = os.path.join(os.path.dirname(HERE), "tests", "cpp", "hip_provider_test.cc")
HOST_TEST_BINARY = os.path.join(os.path.dirname(HERE), "tests", "cpp", "hip_provider_test")


def build_host_tests(verbose: bool = True) -> str:
    """Compiles the C++ tests of the host mirror (include/hyle_hip_compute.hpp) with g++ against
    the built library, the HIP runtime and the C oracle (the checker)."""
    root = os.path.dirname(HERE)
    rocm = os.environ.get("ROCM_PATH", "/opt/rocm")
    cmd = [
        "g++", "-std=c++20", "-O1", "-Wall", "-D__HIP_PLATFORM_AMD__",
        "-I" + os.path.join(root, "include"), "-I" + os.path.join(root, "oracle"), "-I" + os.path.join(rocm, "include"),
        HOST_TEST_SOURCE, "-o", HOST_TEST_BINARY,
        "-L" + HERE, "-lhyle_hip", "-L" + os.path.join(root, "oracle"), "-lhyle_oracle",
        "-L" + os.path.join(rocm, "lib"), "-lamdhip64",
        "-Wl,-rpath,$ORIGIN/../../hyle_amd:$ORIGIN/../../oracle:" + os.path.join(rocm, "lib"),
    ]
    done = subprocess.run(cmd, capture_output=True, text=True)
    if done.returncode != 0:
        raise RuntimeError(f"g++ failed on the host tests:\n{done.stderr}")
    if verbose:
        print(f"built {HOST_TEST_BINARY}")
    return HOST_TEST_BINARY


if __name__ == "__main__":
    build()
