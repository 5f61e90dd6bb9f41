"""GPU: a host program written against include/pikv_hip.h alone (C++, hipMalloc'ed
buffers, no Python or torch in the process) drives router tail -> slots -> quantise +
scatter -> advance -> gather + dequantise -> eviction -> compaction and compares every
result bit for bit with the scalar C restatement it links."""
import os
import subprocess

import pytest

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
BINARY = os.path.join(ROOT, "tests", "abi_host", "abi_parity")


def test_native_host_program(dev):
    assert os.path.exists(BINARY), "build with `make -C tests/abi_host` (after the two libraries)"
    r = subprocess.run([BINARY], capture_output=True, text=True, timeout=100)
    print(r.stdout)
    print(r.stderr)
    assert r.returncode == 0, r.stdout[-2000:] + r.stderr[-2000:]
    assert r.stdout.strip().endswith("abi_parity: ALL OK")
    assert "MISMATCH" not in r.stdout
