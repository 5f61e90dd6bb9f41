"""CPU checks of the boundary: the shared library loads, exports every function
include/pikv_hip.h declares with the declared number of arguments, and the
host-side validation rejects bad calls before anything reaches a GPU."""
import ctypes
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "pikv_hip.h")


def _declared():
    src = open(HEADER).read()
    src = re.sub(r"/\*.*?\*/", "", src, flags=re.S)
    out = {}
    for m in re.finditer(r"\b(pikv_\w+)\s*\(([^;{]*?)\)\s*;", src, flags=re.S):
        name, args = m.group(1), m.group(2).strip()
        n = 0 if args in ("", "void") else len([a for a in args.split(",") if a.strip()])
        out[name] = n
    return out


def test_header_declares_expected_surface():
    d = _declared()
    for need in ["pikv_router_fused", "pikv_router_tail", "pikv_capacity_slots", "pikv_quant_scatter",
                 "pikv_cache_advance", "pikv_quantize_rows", "pikv_gather_dequant",
                 "pikv_gather_dequant_scores", "pikv_h2o_accumulate", "pikv_evict_select",
                 "pikv_h2o_budget", "pikv_compact_rows", "pikv_fakequant_colblocks", "pikv_fakequant_preset",
                 "pikv_router_workspace_bytes", "pikv_fakequant_workspace_bytes",
                 "pikv_router_fused_workspace_bytes", "pikv_quant_gather", "pikv_attend_values",
                 "pikv_attend_workspace_bytes", "pikv_evict_workspace_bytes",
                 "pikv_decode_attend", "pikv_decode_attend_workspace_bytes", "pikv_quant8_minshift",
                 "pikv_capacity_slots_static", "pikv_capacity_slots_static_max",
                 "pikv_status_string", "pikv_abi_version"]:
        assert need in d


def test_library_exports_every_declared_symbol():
    from pikv_amd import _native as N
    assert os.path.exists(N.LIB_PATH), "build with `python -m pikv_amd.build`"
    lib = ctypes.CDLL(N.LIB_PATH)
    d = _declared()
    for name, nargs in d.items():
        assert hasattr(lib, name), f"{name} declared but not exported"
        assert name in N.SIGNATURES, f"{name} has no ctypes signature"
        assert len(N.SIGNATURES[name][1]) == nargs, f"{name}: binding has wrong arity"
    assert set(N.SIGNATURES) == set(d)


def test_pure_host_entry_points():
    """Entry points that never touch the device can run here."""
    from pikv_amd import _native as N
    lib = N.lib()
    assert lib.pikv_abi_version() >= 1000
    assert N.status_string(0) == "ok"
    assert "NULL" in N.status_string(-1)
    assert lib.pikv_router_workspace_bytes(32768, 8, 2) >= (65536 // 512) * 8 * 4
    assert lib.pikv_router_workspace_bytes(0, 8, 2) == 0
    assert lib.pikv_fakequant_workspace_bytes(1000, 256, 128) >= 2 * 4 * 16
    # argument validation happens before any launch: NULL pointers and bad
    # shapes come back as status codes
    assert lib.pikv_quant_scatter(None, None, 0, 1, 1, 128, 128, 0, None, None, None, None, None, 1,
                                  None, None, None, None, None, None, None, None, 0.0, None) == -1
    assert lib.pikv_capacity_slots(1, 10, 100, 5, 1, None, None, 0, None) == -2
    assert lib.pikv_router_fused(1, 1, 0, None, None, None, 1.0, 0.0, 0, 4, 63, 4, 2, 0,
                                 None, None, 1, 1, None, None, None, 0, None) == -3
    assert lib.pikv_router_fused(1, 1, 7, None, None, None, 1.0, 0.0, 0, 4, 64, 4, 2, 0,
                                 None, None, 1, 1, None, None, None, 0, None) == -3
    assert lib.pikv_router_fused(1, 1, 0, None, None, None, 1.0, 0.0, 5, 4, 64, 4, 2, 0,
                                 None, None, 1, 1, None, None, None, 0, None) == -3   # unknown arithmetic
    assert lib.pikv_evict_select(9, 1, 1, 1, 1, 1, 1, 1, 64, 1, 1, 1, None, 0, None) == -3
    assert lib.pikv_evict_workspace_bytes(2, 4097) == 2 * (3 * 2 * 2048 + 2 * 2 * 1024 + 2) * 4
    assert lib.pikv_evict_select(0, 1, 1, 1, 1, 1, 1, 2, 10000, 1, 1, 1, 1, 100, None) == -4
    # bf16 router needs its workspace (re-laid gate weights): too small -> workspace status
    need = lib.pikv_router_fused_workspace_bytes(64, 128, 8, 2)
    assert need >= 128 * 16 * 2
    assert lib.pikv_router_fused(1, 1, 1, None, None, None, 1.0, 0.0, 0, 64, 128, 8, 2, 0,
                                 None, None, 1, 1, None, None, 1, 128 * 16 * 2 - 1, None) == -4
    # pyramid gather: NULL index list; attention output: heads must divide, workspace must fit
    assert lib.pikv_quant_gather(1, None, 1, 128, 128, 0, 1, None, 1, 4, None, 1, 1, 1, 1,
                                 1, None, 1, None, None, None, None, None, 0.0, None) == -1
    assert lib.pikv_attend_values(1, None, 64, 1, 1, None, 0, 128, 3, 4, 128, 1, 1, 1, 64, 1.0, 0.0, None, None,
                                  1, 1, 1 << 20, None) == -2
    # partial outputs, one per block of cached tokens: a small batch is cut into 256-token pieces so that
    # more compute units take part, a batch that fills the chip walks 4096 tokens per block
    ws = lib.pikv_attend_workspace_bytes(2, 4, 128, 5000)
    assert ws == 20 * 2 * 4 * 128 * 4
    assert lib.pikv_attend_workspace_bytes(64, 32, 128, 32768) == 8 * 64 * 32 * 128 * 4
    assert lib.pikv_attend_values(1, None, 5000, 1, 1, None, 0, 128, 4, 4, 128, 1, 1, 2, 5000, 1.0, 0.0, None, None,
                                  1, 1, ws - 1, None) == -4


def test_integration_stub_matches_header():
    """The ctypes stub shown to maintainers binds the declared number of arguments."""
    doc = open(os.path.join(ROOT, "INTEGRATION.md")).read()
    d = _declared()
    found = re.findall(r"_lib\.(pikv_\w+)\.argtypes\s*=\s*\[(.*?)\]", doc, flags=re.S)
    assert found
    for name, args in found:
        assert len([a for a in args.split(",") if a.strip()]) == d[name], name


def test_header_is_plain_c(tmp_path):
    """include/pikv_hip.h compiles as C99 and as C++ with nothing but <stdint.h>."""
    import subprocess
    src = tmp_path / "use.c"
    src.write_text('#include "pikv_hip.h"\nint main(void) { return pikv_abi_version() > 0 ? 0 : 1; }\n')
    inc = os.path.join(ROOT, "include")
    subprocess.run(["gcc", "-std=c99", "-Wall", "-Wextra", "-pedantic", "-Werror", "-I", inc, "-fsyntax-only", str(src)],
                   check=True)
    subprocess.run(["g++", "-std=c++11", "-Wall", "-Werror", "-I", inc, "-fsyntax-only", "-x", "c++", str(src)],
                   check=True)


def test_ops_reject_cpu_tensors():
    """The product path has no CPU fallback."""
    import torch
    from pikv_amd import ops
    with pytest.raises(ValueError):
        ops.router_fused(torch.zeros(4, 64), torch.zeros(4, 64))
    with pytest.raises(ValueError):
        ops.quantize_rows(torch.zeros(4, 128), 128, 0)
    with pytest.raises(ValueError):
        ops.CachePool([4], 1, 64, 64, 0, "cpu")


def test_missing_library_fails_loudly(monkeypatch, tmp_path):
    from pikv_amd import _native as N
    monkeypatch.setattr(N, "_lib", None)
    monkeypatch.setattr(N, "LIB_PATH", str(tmp_path / "nope.so"))
    with pytest.raises(N.PiKVNativeError):
        N.lib()
