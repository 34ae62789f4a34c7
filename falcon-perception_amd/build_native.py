"""Build libfp_paged_kv.so (the gfx950 kernels + C ABI) with hipcc, in-tree.

    python falcon-perception_amd/build_native.py

hipcc cross-compiles for gfx950 without a GPU.  The shared library has no torch
or Python dependency; the host package loads it with ctypes.
"""

from __future__ import annotations

import concurrent.futures
import os
import re
import shutil
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
CSRC = os.path.join(HERE, "csrc")
INCLUDE = os.path.join(ROOT, "include")
OUT_DIR = os.path.join(HERE, "falcon_perception_amd", "_lib")
LIB_PATH = os.path.join(OUT_DIR, "libfp_paged_kv.so")
OBJ_DIR = os.path.join(HERE, "build")

# packed-FP32 VALU forms are switched off for every kernel of this library
FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
    # one remark per kernel with its registers, LDS and scratch: kept beside the object file
    # (build/<source>.resources.txt) and read back by `resource_usage()`
    "-Rpass-analysis=kernel-resource-usage",
    "-I", INCLUDE,
    "-I", CSRC,
]


def _hipcc() -> str:
    exe = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(exe):
        raise RuntimeError("hipcc not found; the ROCm toolchain is required to build libfp_paged_kv.so")
    return exe


def sources() -> list[str]:
    return sorted(os.path.join(CSRC, f) for f in os.listdir(CSRC) if f.endswith(".hip"))


def _compile(src: str) -> str:
    obj = os.path.join(OBJ_DIR, os.path.basename(src)[:-4] + ".o")
    cmd = [_hipcc(), *FLAGS, "-c", src, "-o", obj]
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError(f"hipcc failed for {src}:\n{res.stdout}\n{res.stderr}")
    with open(obj[:-2] + ".resources.txt", "w") as f:
        f.write(res.stderr)
    return obj


def resource_usage() -> dict[str, dict[str, int]]:
    """Per kernel of the last build: {"vgprs", "agprs", "scratch" (bytes per lane), "lds" (bytes per workgroup),
    "occupancy" (wavefronts per SIMD)}, keyed by the mangled kernel name; builds first if nothing has been
    built.  A kernel with scratch > 0 spills registers to memory; the first launch of such a kernel makes the
    runtime set that memory up, which it cannot do while a stream is being captured into a graph."""
    names = [os.path.join(OBJ_DIR, os.path.basename(s)[:-4] + ".resources.txt") for s in sources()]
    if not all(os.path.exists(n) for n in names):
        build_library(verbose=False)
    out: dict[str, dict[str, int]] = {}
    fields = {"vgprs": r"VGPRs: (\d+)", "agprs": r"AGPRs: (\d+)", "scratch": r"ScratchSize \[bytes/lane\]: (\d+)",
              "lds": r"LDS Size \[bytes/block\]: (\d+)", "occupancy": r"Occupancy \[waves/SIMD\]: (\d+)"}
    for n in names:
        with open(n) as f:
            text = f.read()
        for block in re.split(r"remark: [^\n]*Function Name: ", text)[1:]:
            out[block.split()[0]] = {k: int(re.search(v, block).group(1)) for k, v in fields.items()}
    return out


def build_library(verbose: bool = True) -> str:
    """Compile every csrc/*.hip for gfx950 and link libfp_paged_kv.so. Returns its path."""
    os.makedirs(OBJ_DIR, exist_ok=True)
    os.makedirs(OUT_DIR, exist_ok=True)
    srcs = sources()
    with concurrent.futures.ThreadPoolExecutor(max_workers=min(8, len(srcs))) as ex:
        objs = list(ex.map(_compile, srcs))
    tmp = LIB_PATH + ".tmp"
    cmd = [_hipcc(), "--offload-arch=gfx950", "-shared", "-fPIC", *objs, "-o", tmp]
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError(f"link failed:\n{res.stdout}\n{res.stderr}")
    os.replace(tmp, LIB_PATH)
    if verbose:
        print(f"built {LIB_PATH} from {len(srcs)} sources", file=sys.stderr)
    return LIB_PATH


if __name__ == "__main__":
    build_library()
