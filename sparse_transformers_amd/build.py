"""Compile the HIP sources under csrc/ into libsparse_mlp_amd.so (gfx950 only).

Usage:  python -m sparse_transformers_amd.build
The library is built in-tree, next to this file, so that it travels with the
source tree; nothing is installed.
"""
from __future__ import annotations

import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB_NAME = "libsparse_mlp_amd.so"
LIB_PATH = os.path.join(HERE, LIB_NAME)
SOURCES = ["capi.hip", "mlp_decode.hip", "mlp_batch.hip", "mlp_prefill.hip", "predictor.hip", "mask_select.hip",
           "mlp_f64.hip", "cache.hip"]

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    # the pass that aggregates uniform atomics per wave reads their result back at once; the cache kernels
    # issue one atomic per block and look at its result much later on purpose
    "-mllvm", "-amdgpu-atomic-optimizer-strategy=None",
    # the first kernel arguments arrive in scalar registers with the wave instead of through a load at its start
    # (one memory round trip less in front of every kernel of a chain of short dependent kernels; structs passed by
    # value end the preloaded part, so the cache kernels take theirs last)
    "-mllvm", "-amdgpu-kernarg-preload-count=16",
    "-Wall",
    "-Wno-unused-command-line-argument",
]


def _compile(src: str, obj: str) -> None:
    subprocess.run([HIPCC, *FLAGS, "-c", src, "-o", obj], check=True)


def build(verbose: bool = True) -> str:
    build_dir = os.path.join(HERE, "build")
    os.makedirs(build_dir, exist_ok=True)
    srcs = [s for s in SOURCES if os.path.exists(os.path.join(CSRC, s))]
    objs = [os.path.join(build_dir, s.replace(".hip", ".o")) for s in srcs]
    if verbose:
        print(f"[build] hipcc gfx950: {', '.join(srcs)}", flush=True)
    with ThreadPoolExecutor(max_workers=min(8, len(srcs))) as ex:
        list(ex.map(lambda so: _compile(os.path.join(CSRC, so[0]), so[1]), zip(srcs, objs)))
    subprocess.run([HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB_PATH, *objs], check=True)
    if verbose:
        print(f"[build] wrote {LIB_PATH}", flush=True)
    return LIB_PATH


def build_capi_client(verbose: bool = True) -> str:
    """tests/capi/capi_client: a C++ client of the C ABI that links nothing but the library and the HIP
    runtime (run by tests/test_gpu_capi_client.py on the GPU box)."""
    root = os.path.dirname(HERE)
    src = os.path.join(root, "tests", "capi", "capi_client.cpp")
    exe = os.path.join(root, "tests", "capi", "capi_client")
    subprocess.run([HIPCC, "--offload-arch=gfx950", "-O2", "-std=c++17", "-o", exe, src, "-L" + HERE,
                    "-lsparse_mlp_amd", "-Wl,-rpath,$ORIGIN/../../sparse_transformers_amd"], check=True)
    if verbose:
        print(f"[build] wrote {exe}", flush=True)
    return exe


if __name__ == "__main__":
    build()
    build_capi_client()
    sys.exit(0)
