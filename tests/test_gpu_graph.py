"""GPU: the entry points allocate nothing, clear nothing with memsets and never
synchronise, so a caller may capture them into a HIP graph.  A captured prefill step
(router -> quantise + scatter -> advance -> scores -> H2O accumulate) and a captured
decode read (scores -> statistics -> attention output with H2O accumulate) are
replayed several times, with eager work and synchronisations in between, and every
replay must leave exactly what the eager run leaves."""
import pytest

pytestmark = pytest.mark.gpu


def _prefill(ops, torch, pool, hidden, gate_w, k_src, v_src, q, top_k, cap, heads, now):
    pool.fill.zero_()
    pool.acc.zero_()
    r = ops.router_fused(hidden, gate_w, top_k=top_k, capacity=cap)
    pool.quant_scatter(k_src, v_src, r.topk_idx, r.slot, top_k, now=now)
    pool.advance(r.count, cap)
    scores, tmax, tsum = pool.scores(q, heads)
    pool.h2o_accumulate(scores, tmax, tsum, now=now)
    return r.topk_idx, r.slot, r.count


def _state(pool):
    return [t.clone() for t in (pool.k_codes, pool.k_scale, pool.v_codes, pool.v_scale, pool.acc, pool.ts, pool.fill)]


def test_prefill_step_replays(dev):
    import torch
    from pikv_amd import ops
    g = torch.Generator(device=dev).manual_seed(3)
    T, H, E, top_k, heads, dh = 2048, 512, 8, 2, 4, 128
    D = heads * dh
    hidden = torch.randn(T, H, generator=g, device=dev).to(torch.bfloat16)
    gate_w = (0.05 * torch.randn(E, H, generator=g, device=dev)).to(torch.bfloat16)
    k_src = torch.randn(T, D, generator=g, device=dev).to(torch.bfloat16)
    v_src = torch.randn(T, D, generator=g, device=dev).to(torch.bfloat16)
    q = torch.randn(E, heads, dh, generator=g, device=dev).to(torch.bfloat16)
    cap = int(T * 1.25 * top_k / E)
    args = (hidden, gate_w, k_src, v_src, q, top_k, cap, heads)

    eager_pool = ops.CachePool([cap] * E, heads, dh, dh, ops.Q_I8_SYM, dev)
    want_route = [t.clone() for t in _prefill(ops, torch, eager_pool, *args, now=4.0)]
    want = _state(eager_pool)

    pool = ops.CachePool([cap] * E, heads, dh, dh, ops.Q_I8_SYM, dev)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for _ in range(2):
            _prefill(ops, torch, pool, *args, now=4.0)
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        route = _prefill(ops, torch, pool, *args, now=4.0)
    for rep in range(4):
        # eager work between the replays: scribble over what the graph must rebuild
        pool.k_codes.fill_(3)
        pool.acc.fill_(-1.0)
        pool.fill.fill_(1)
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        for got, ref in zip(route, want_route):
            assert torch.equal(got, ref), rep
        assert torch.equal(pool.fill, eager_pool.fill), rep
        # rows past a cache's fill are not written: they keep the scribble
        valid = (torch.arange(cap, device=dev).unsqueeze(0) < pool.fill.unsqueeze(1)).reshape(-1)
        for got, ref in zip(_state(pool)[:-1], want[:-1]):
            assert torch.equal(got[valid], ref[valid]), rep


def test_decode_read_replays(dev):
    import torch
    from pikv_amd import ops
    g = torch.Generator(device=dev).manual_seed(5)
    B, N, hkv, hq, dh = 3, 4500, 8, 32, 128
    D = hkv * dh
    lens = torch.tensor([4500, 2049, 64], dtype=torch.int32, device=dev)

    def filled():
        pool = ops.CachePool([N] * B, hkv, dh, 32, ops.Q_I4_ASYM, dev, with_v=True)
        gg = torch.Generator(device=dev).manual_seed(6)
        ks = torch.randn(B * N, D, generator=gg, device=dev).to(torch.bfloat16)
        vs = torch.randn(B * N, D, generator=gg, device=dev).to(torch.bfloat16)
        cid = torch.arange(B, device=dev, dtype=torch.int32).repeat_interleave(N)
        slot = torch.arange(N, device=dev, dtype=torch.int32).repeat(B)
        pool.quant_scatter(ks, vs, cid, slot, 1, now=0.0)
        pool.fill.copy_(lens)
        return pool

    q = torch.randn(B, hq, dh, generator=g, device=dev).to(torch.bfloat16)

    def read(pool):
        pool.acc.zero_()
        s, m, z = pool.scores(q, hq)
        pool.h2o_accumulate(s, m, z, now=2.0, stats_only=True)
        return pool.attend_values(s, pool.head_stats, accumulate=True, now=2.0)

    eager_pool = filled()
    want_out = read(eager_pool).clone()
    want_acc, want_ts = eager_pool.acc.clone(), eager_pool.ts.clone()

    pool = filled()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for _ in range(2):
            read(pool)
    torch.cuda.current_stream().wait_stream(side)
    ts0 = pool.ts.clone()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        out = read(pool)
    for rep in range(4):
        pool.acc.fill_(7.0)
        pool.ts.fill_(-1.0)
        out.fill_(123.0)
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out, want_out), rep
        assert torch.equal(pool.acc, want_acc), rep
        # timestamps of the valid rows are set; rows past a cache's fill keep the scribble
        valid = (torch.arange(N, device=dev).unsqueeze(0) < lens.unsqueeze(1)).reshape(-1)
        assert torch.equal(pool.ts[valid], want_ts[valid]), rep
        assert bool((pool.ts[~valid] == -1.0).all()), rep


@pytest.mark.parametrize("hkv,hq,dh,eight", [
    (8, 32, 128, False),     # the decode shape: one pass over K and V
    (2, 24, 128, False),     # 12 q heads per kv head: two launches of each kernel, pairs of neighbouring rows as one
    (1, 4, 128, False),      # one kv head: four neighbouring rows as one
    (2, 14, 64, False),      # heads of 64, 14 q heads on the one slab
    (8, 64, 128, True),      # 8-bit codes, 8 q heads per kv head: the one-pass form, two blocks per token range
    (3, 12, 128, True),      # ... 3 kv heads x 4: records of 32 lanes
    (8, 64, 128, False),     # 4-bit, 8 q heads per kv head: the one-pass form with two operand sets
])
def test_decode_attend_replays(dev, hkv, hq, dh, eight):
    """The one-call decode read under capture: its workspace is allocated before the capture, and every
    replay must rebuild the attention output and the H2O accumulators from scribbled memory."""
    import torch
    from pikv_amd import ops
    g = torch.Generator(device=dev).manual_seed(9)
    B, N = 3, 4500
    D = hkv * dh
    lens = torch.tensor([4500, 2049, 64], dtype=torch.int32, device=dev)

    def filled():
        pool = (ops.CachePool([N] * B, hkv, dh, dh, ops.Q_I8_ASYM, dev, with_v=True) if eight else
                ops.CachePool([N] * B, hkv, dh, 32, ops.Q_I4_ASYM, dev, with_v=True))
        gg = torch.Generator(device=dev).manual_seed(10)
        ks = torch.randn(B * N, D, generator=gg, device=dev).to(torch.bfloat16)
        vs = torch.randn(B * N, D, generator=gg, device=dev).to(torch.bfloat16)
        cid = torch.arange(B, device=dev, dtype=torch.int32).repeat_interleave(N)
        slot = torch.arange(N, device=dev, dtype=torch.int32).repeat(B)
        pool.quant_scatter(ks, vs, cid, slot, 1, now=0.0)
        pool.fill.copy_(lens)
        return pool

    q = torch.randn(B, hq, dh, generator=g, device=dev).to(torch.bfloat16)

    def read(pool):
        pool.acc.zero_()
        return pool.decode_attend(q, hq, now=2.0)

    eager_pool = filled()
    want_out = read(eager_pool).clone()
    want_acc, want_ts = eager_pool.acc.clone(), eager_pool.ts.clone()

    pool = filled()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for _ in range(2):
            read(pool)
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        out = read(pool)
    valid = (torch.arange(N, device=dev).unsqueeze(0) < lens.unsqueeze(1)).reshape(-1)
    for rep in range(4):
        pool.acc.fill_(7.0)
        pool.ts.fill_(-1.0)
        out.fill_(123.0)
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out, want_out), rep
        assert torch.equal(pool.acc, want_acc), rep
        assert torch.equal(pool.ts[valid], want_ts[valid]), rep
        assert bool((pool.ts[~valid] == -1.0).all()), rep
