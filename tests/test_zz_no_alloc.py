"""The allocation-free capacity-slot entry point (pikv_capacity_slots_static) against the
workspace form (pikv_capacity_slots) and the sequential rule of the oracle
(core/single/module/pikv_routing.py:93-104), through the C ABI.  Two calls in a row share
the library's device array; the second is smaller, so stale counters of the first would show."""
import numpy as np
import pytest
import torch

import pikv_oracle as O
from pikv_amd import _native as N

pytestmark = pytest.mark.gpu


def _both(idx_np, E, cap, dev):
    lib = N.lib()
    A = idx_np.size
    idx = torch.from_numpy(idx_np).to(dev)
    st = torch.cuda.current_stream().cuda_stream
    out = []
    for static in (False, True):
        slot = torch.full((max(A, 1),), -7, dtype=torch.int32, device=dev)
        count = torch.full((E,), -7, dtype=torch.int32, device=dev)
        if static:
            rc = lib.pikv_capacity_slots_static(idx.data_ptr(), A, E, cap, slot.data_ptr(), count.data_ptr(), st)
        else:
            nb = int(lib.pikv_router_workspace_bytes(A, E, 1))
            ws = torch.empty(max(nb, 256), dtype=torch.uint8, device=dev)
            rc = lib.pikv_capacity_slots(idx.data_ptr(), A, E, cap, slot.data_ptr(), count.data_ptr(),
                                         ws.data_ptr(), nb, st)
        assert rc == 0, N.status_string(rc)
        torch.cuda.synchronize()
        out.append((slot[:A].cpu().numpy(), count.cpu().numpy()))
    return out


def test_static_slots_match_workspace_form_twice(dev):
    r = np.random.default_rng(11)
    # first a long skewed stream over 64 experts, then a short one over 8: the second call
    # reads fewer, differently strided counters of the same array
    for A, E, cap in ((300_001, 64, 4000), (1_531, 8, 150), (0, 4, 3)):
        p = 1.0 / np.arange(1, E + 1) ** 1.2
        idx = r.choice(E, size=A, p=p / p.sum()).astype(np.int32)
        (s_ws, c_ws), (s_st, c_st) = _both(idx, E, cap, dev)
        assert np.array_equal(s_st, s_ws)
        assert np.array_equal(c_st, c_ws)
        s_ref, c_ref = O.capacity_slots(idx.reshape(-1, 1), E, cap)
        assert np.array_equal(s_st, s_ref.reshape(-1))
        assert np.array_equal(c_st, c_ref)


def test_static_slots_reject_oversize(dev):
    lib = N.lib()
    limit = int(lib.pikv_capacity_slots_static_max())
    assert limit == 1 << 20
    one = torch.zeros(1, dtype=torch.int32, device=dev)
    assert lib.pikv_capacity_slots_static(one.data_ptr(), limit + 1, 8, 4, one.data_ptr(), None, None) == -4
    assert lib.pikv_capacity_slots_static(one.data_ptr(), 1, 65, 4, one.data_ptr(), None, None) == -2
    assert lib.pikv_capacity_slots_static(None, 1, 8, 4, one.data_ptr(), None, None) == -1
    # at the limit itself the call is served
    r = np.random.default_rng(5)
    idx = r.integers(0, 64, size=limit).astype(np.int32)
    (s_ws, c_ws), (s_st, c_st) = _both(idx, 64, 1 << 14, dev)
    assert np.array_equal(s_st, s_ws) and np.array_equal(c_st, c_ws)


def test_static_slots_allocate_nothing_and_replay_from_a_graph(dev):
    """After the set-up call (pikv_capacity_slots_static_max on this device) the entry point leaves the
    device's free memory untouched, and it can be captured into a HIP graph: every replay, with slot and
    count scribbled over in between and eager work of the program around it, gives the eager result."""
    lib = N.lib()
    assert int(lib.pikv_capacity_slots_static_max()) == 1 << 20       # set-up: address looked up outside any capture
    r = np.random.default_rng(23)
    A, E, cap = 70_001, 24, 2500
    idx_np = r.integers(0, E, size=A).astype(np.int32)
    idx = torch.from_numpy(idx_np).to(dev)
    slot = torch.empty(A, dtype=torch.int32, device=dev)
    count = torch.empty(E, dtype=torch.int32, device=dev)
    torch.cuda.synchronize()
    free0, _ = torch.cuda.mem_get_info(dev)
    st = torch.cuda.current_stream().cuda_stream
    for _ in range(3):
        assert lib.pikv_capacity_slots_static(idx.data_ptr(), A, E, cap, slot.data_ptr(), count.data_ptr(), st) == 0
    torch.cuda.synchronize()
    free1, _ = torch.cuda.mem_get_info(dev)
    assert free1 == free0
    s_ref, c_ref = O.capacity_slots(idx_np.reshape(-1, 1), E, cap)
    assert np.array_equal(slot.cpu().numpy(), s_ref.reshape(-1)) and np.array_equal(count.cpu().numpy(), c_ref)
    side = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            rc = lib.pikv_capacity_slots_static(idx.data_ptr(), A, E, cap, slot.data_ptr(), count.data_ptr(),
                                                torch.cuda.current_stream().cuda_stream)
    assert rc == 0
    for rep in range(3):
        slot.fill_(-9 - rep)
        count.fill_(-9 - rep)
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert np.array_equal(slot.cpu().numpy(), s_ref.reshape(-1)), rep
        assert np.array_equal(count.cpu().numpy(), c_ref), rep
        (idx.float().sum() + 1).item()                                    # eager work between the replays
