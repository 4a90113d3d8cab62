"""Builds libkarume_hip.so (gfx950 only) with hipcc, in-tree.

    python -m karume_amd.build            # compile every source, link karume_amd/lib/libkarume_hip.so

The flags are fixed on purpose: one architecture, no fast-math (the int4 dequant multiply and
the accumulation order are part of the numerical contract), and packed-fp32 instructions are
switched off for the device pass.
"""
from __future__ import annotations

import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB_DIR = os.path.join(HERE, "lib")
LIB_PATH = os.path.join(LIB_DIR, "libkarume_hip.so")
OBJ_DIR = os.path.join(HERE, "build")

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
FLAGS = [
    "-O3", "-std=c++17", "-fPIC", "--offload-arch=gfx950",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-fno-fast-math", "-ffp-contract=off", "-Wall", "-Wno-unused-function", "-Wno-unknown-warning-option",
    # the first kernel arguments arrive in scalar registers with the wave (gfx950 preloads them)
    # instead of through a load every kernel would wait for before its first address is known
    "-mllvm", "-amdgpu-kernarg-preload-count=16",
]


def sources() -> list[str]:
    return sorted(os.path.join(CSRC, f) for f in os.listdir(CSRC) if f.endswith(".hip"))


def _compile(src: str) -> str:
    obj = os.path.join(OBJ_DIR, os.path.basename(src)[:-4] + ".o")
    cmd = [HIPCC, *FLAGS, "-c", src, "-o", obj]
    proc = subprocess.run(cmd, capture_output=True, text=True)
    noise = "is not a recognized feature for this target"
    err = "\n".join(l for l in proc.stderr.splitlines() if noise not in l)
    if proc.returncode != 0:
        raise RuntimeError(f"hipcc failed on {src}:\n{err}")
    if err.strip():
        sys.stderr.write(err + "\n")
    return obj


def build(verbose: bool = True) -> str:
    os.makedirs(LIB_DIR, exist_ok=True)
    os.makedirs(OBJ_DIR, exist_ok=True)
    srcs = sources()
    with ThreadPoolExecutor(max_workers=min(8, len(srcs))) as pool:
        objs = list(pool.map(_compile, srcs))
    cmd = [HIPCC, "-shared", "-fPIC", "--offload-arch=gfx950", "-Wl,--no-undefined", "-o", LIB_PATH,
           *objs]
    proc = subprocess.run(cmd, capture_output=True, text=True)
    if proc.returncode != 0:
        raise RuntimeError(f"link failed:\n{proc.stderr}")
    if verbose:
        print(f"built {LIB_PATH} from {len(srcs)} sources")
    return LIB_PATH


if __name__ == "__main__":
    build()
