"""Builds the HIP library of the sparse MoE block for gfx950 (MI355X), in-tree.

    python -m mummu_amd.build          # compile every kernel file and link lib/libmummu_moe.so

hipcc cross-compiles without a GPU.  Flags that matter:
  -ffp-contract=off     a fused multiply-add happens only where the source writes fmaf, so the
                        bit-exact pieces (dequantizer, router, combine) round as specified
  -packed-fp32-ops off  keep the compiler from forming packed-f32 VALU ops
"""
from __future__ import annotations

import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
OBJ = os.path.join(HERE, "lib", "obj")
LIB = os.path.join(HERE, "lib", "libmummu_moe.so")

SOURCES = ["dequant.hip", "router.hip", "experts.hip", "decode_layer.hip", "dispatch.hip", "gemm.hip", "moe_api.hip", "packed_gemv.hip", "gguf_reader.cpp", "safetensors_loader.cpp"]
HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-ffp-contract=off", "-fvisibility=hidden",
         "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops", "-Wall", "-Wno-unused-function"]


# Per-source additions (none at present).
EXTRA_FLAGS = {}


def _compile(src: str) -> str:
    obj = os.path.join(OBJ, os.path.splitext(src)[0] + ".o")
    cmd = [HIPCC, *FLAGS, *EXTRA_FLAGS.get(src, []), "-c", os.path.join(CSRC, src), "-o", obj]
    r = subprocess.run(cmd, capture_output=True, text=True)
    noise = "is not a recognized feature for this target"
    err = "\n".join(l for l in r.stderr.splitlines() if noise not in l)
    if r.returncode != 0:
        raise RuntimeError(f"hipcc failed on {src}:\n{err}")
    if err.strip():
        sys.stderr.write(err + "\n")
    return obj


def build(verbose: bool = False) -> str:
    os.makedirs(OBJ, exist_ok=True)
    with ThreadPoolExecutor(max_workers=min(8, len(SOURCES))) as ex:
        objs = list(ex.map(_compile, SOURCES))
    cmd = [HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB, *objs, "-Wl,-rpath,/opt/rocm/lib"]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"link failed:\n{r.stderr}")
    if verbose:
        print(f"built {LIB}")
    build_host_mirror_test(verbose)
    return LIB


ROOT = os.path.dirname(HERE)
HOST_TEST_SRC = os.path.join(ROOT, "tests", "cpp", "host_mirror_test.cpp")
HOST_TEST_BIN = os.path.join(ROOT, "tests", "cpp", "host_mirror_test")


def build_host_mirror_test(verbose: bool = False) -> str:
    """The C++ host mirror (include/mummu_moe.hpp) and its test program: plain g++ over the C ABI."""
    cmd = [os.environ.get("CXX", "g++"), "-O1", "-std=c++17", "-Wall", "-I", os.path.join(ROOT, "include"), HOST_TEST_SRC,
           "-o", HOST_TEST_BIN, "-L", os.path.dirname(LIB), "-lmummu_moe", "-Wl,-rpath,$ORIGIN/../../mummu_amd/lib"]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"g++ failed on the host mirror test:\n{r.stderr}")
    if verbose:
        print(f"built {HOST_TEST_BIN}")
    return HOST_TEST_BIN


if __name__ == "__main__":
    build(verbose=True)
