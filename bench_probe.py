"""Build and load libbench_probe.so, the streaming probes of bench.py / bench_profile.py
(bench_probe.hip): measurement aids, kept out of libpikv_hip.so and its header.

    python3 bench_probe.py        # build (hipcc cross-compiles gfx950 without a GPU)
"""
from __future__ import annotations

import ctypes as C
import os
import subprocess

HERE = os.path.dirname(os.path.abspath(__file__))
SRC = os.path.join(HERE, "bench_probe.hip")
LIB = os.path.join(HERE, "libbench_probe.so")
_handle = None


def build() -> str:
    cmd = [os.environ.get("HIPCC", "/opt/rocm/bin/hipcc"), "--offload-arch=gfx950", "-O3", "-fPIC", "-std=c++17",
           "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops", "-shared", SRC, "-o", LIB]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"hipcc failed for bench_probe.hip:\n{r.stdout}\n{r.stderr}")
    return LIB


def lib():
    """The loaded probe library; built first when the file is not there."""
    global _handle
    if _handle is None:
        if not os.path.exists(LIB):
            build()
        _handle = C.CDLL(LIB)
        _handle.bench_stream_probe.restype = C.c_int
        _handle.bench_stream_probe.argtypes = [C.c_int, C.c_void_p, C.c_void_p, C.c_int64, C.c_int, C.c_void_p, C.c_void_p]
    return _handle


def stream_probe(mode: int, src_ptr, dst_ptr, nbytes: int, streaming_stores: int, sink_ptr, stream) -> None:
    """mode 0: read nbytes of src; 1: write nbytes of dst; 2: copy.  Pointers are device addresses (ints)."""
    rc = lib().bench_stream_probe(mode, src_ptr, dst_ptr, nbytes, streaming_stores, sink_ptr, stream)
    if rc != 0:
        raise RuntimeError(f"bench_stream_probe failed with status {rc}")


if __name__ == "__main__":
    print("built", build())
