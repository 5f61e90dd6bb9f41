"""Build libpikv_hip.so (gfx950 HIP kernels + C ABI) in-tree with hipcc.

    python -m pikv_amd.build

No fast-math: the integer codes depend on IEEE float32 division and
round-half-even.  Packed-FP32 code generation is switched off.
"""
from __future__ import annotations

import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
OBJ = os.path.join(HERE, "build")
LIB = os.path.join(HERE, "libpikv_hip.so")

SOURCES = ["status.hip", "quant_scatter.hip", "router.hip", "read_path.hip", "attend.hip", "decode_fused.hip",
           "evict.hip", "fakequant.hip", "minshift.hip"]

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
FLAGS = [
    "--offload-arch=gfx950", "-O3", "-fPIC", "-std=c++17",
    "-fno-fast-math", "-ffp-contract=off",
    "-fhip-fp32-correctly-rounded-divide-sqrt",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall", "-Wno-unused-function", "-Wno-unknown-attributes",
    # the SLP vectoriser turns the per-word nibble expansions into short vector AND / OR
    # pairs, which then no longer match the three-operand and-or instruction
    "-fno-slp-vectorize",
]


def _compile(src: str) -> str:
    obj = os.path.join(OBJ, os.path.splitext(src)[0] + ".o")
    cmd = [HIPCC, *FLAGS, "-c", os.path.join(CSRC, src), "-o", obj]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"hipcc failed for {src}:\n{r.stdout}\n{r.stderr}")
    return obj


def build(verbose: bool = True) -> str:
    os.makedirs(OBJ, exist_ok=True)
    srcs = [s for s in SOURCES if os.path.exists(os.path.join(CSRC, s))]
    missing = sorted(set(SOURCES) - set(srcs))
    if missing:
        raise RuntimeError(f"missing kernel sources: {missing}")
    with ThreadPoolExecutor(max_workers=min(8, len(srcs))) as ex:
        objs = list(ex.map(_compile, srcs))
    cmd = [HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", *objs, "-o", LIB]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"link failed:\n{r.stdout}\n{r.stderr}")
    if verbose:
        print(f"built {LIB}")
    return LIB


if __name__ == "__main__":
    build()
    sys.exit(0)
