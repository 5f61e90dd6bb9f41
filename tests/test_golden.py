"""Golden digests (tests/golden/path_digests.json) of the seeded cases in
tests/golden/cases.py.  CPU: the numpy restatement still produces them, and so does its
C twin.  GPU: the kernels produce them through the C ABI - here nothing of the
restatement is consulted, only the stored digests."""
import json
import os
import sys

import numpy as np
import pytest

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.join(HERE, "golden"))

import cases as G  # noqa: E402

WANT = json.load(open(os.path.join(HERE, "golden", "path_digests.json")))


def test_restatement_reproduces_golden():
    import make_golden
    got = make_golden.compute()
    assert got.keys() == WANT.keys()
    for key in WANT:
        assert got[key] == WANT[key], key


def test_c_twin_reproduces_golden():
    import c_oracle as C
    c = G.router_case()
    E = c["E"]
    _, _, idx, _ = C.router(c["logits"], np.eye(E, dtype=np.float32), None, c["k"])
    slot, count = C.capacity_slots(idx, E, c["capacity"])
    assert G.digest(idx, np.int32) == WANT["router"]["idx"]
    assert G.digest(slot, np.int32) == WANT["router"]["slot"]
    assert G.digest(count, np.int32) == WANT["router"]["count"]
    c = G.evict_case()
    pool = C.CPool(c["caps"], 32, 32, 0, with_v=False)
    pool.fill[:] = c["lens"]
    pool.acc[:], pool.ts[:] = c["acc"], c["ts"]
    flag, kidx, new_len = pool.evict(0, c["n_heavy"], c["n_recent"], compact=False)
    keep = np.concatenate([flag[b:b + L] for b, L in zip(pool.base, c["lens"])])
    surv = np.concatenate([kidx[b:b + m] for b, m in zip(pool.base, new_len)])
    assert G.digest(keep, np.uint8) == WANT["evict"]["h2o_keep"]
    assert G.digest(surv, np.int32) == WANT["evict"]["h2o_survivors"]
    assert G.digest(new_len, np.int32) == WANT["evict"]["h2o_counts"]
    flag, _, new_len = pool.evict(1, c["n_evict"], None, compact=False)
    keep = np.concatenate([flag[b:b + L] for b, L in zip(pool.base, c["lens"])])
    assert G.digest(keep, np.uint8) == WANT["evict"]["lru_keep"]
    assert G.digest(new_len, np.int32) == WANT["evict"]["lru_counts"]


@pytest.mark.gpu
def test_kernels_reproduce_golden(dev):
    import torch
    from pikv_amd import ops
    from util import codes_np, np_of, to_dev

    c = G.router_case()
    out = ops.router_tail(to_dev(c["logits"], dev), top_k=c["k"], capacity=c["capacity"])
    assert G.digest(np_of(out.topk_idx), np.int32) == WANT["router"]["idx"]
    assert G.digest(np_of(out.slot), np.int32) == WANT["router"]["slot"]
    assert G.digest(np_of(out.count), np.int32) == WANT["router"]["count"]

    c = G.quant_case()
    for name, scheme in G.SCHEMES.items():
        for group in (32, 64, 256):
            for dtype in ("f32", "bf16"):      # the values are bf16-representable: same result either way
                codes, scale, zero = ops.quantize_rows(to_dev(c["x"], dev, dtype), group, scheme)
                want = WANT[f"quant/{name}/g{group}"]
                assert G.digest(codes_np(codes, scheme), np.int16) == want["codes"], (name, group, dtype)
                assert G.digest(np_of(scale), np.float32) == want["scale"], (name, group, dtype)
                z = np.zeros_like(np_of(scale)) if zero is None else np_of(zero)
                assert G.digest(z, np.float32) == want["zero"], (name, group, dtype)

    c = G.scatter_case()
    for name, scheme, group in (("i8_sym", 0, 64), ("i4_asym", 2, 32)):
        pool = ops.CachePool(c["caps"], c["heads"], c["dh"], group, scheme, dev, with_v=True)
        for n, st in enumerate(c["steps"]):
            slot, count = ops.capacity_slots(to_dev(st["idx"].reshape(-1), dev), c["E"], st["capacity"])
            pool.quant_scatter(to_dev(st["k_src"], dev, "bf16"), to_dev(st["v_src"], dev, "bf16"),
                               to_dev(st["idx"], dev), slot, c["k"], now=float(n + 1))
            pool.advance(count, st["capacity"])
        fill = np_of(pool.fill)
        base = np_of(pool.row_base)
        valid = np.concatenate([np.arange(b, b + f) for b, f in zip(base, fill)])
        want = WANT[f"scatter/{name}"]
        assert G.digest(fill, np.int32) == want["fill"]
        assert G.digest(codes_np(pool.k_codes, scheme)[valid], np.int16) == want["k_codes"]
        assert G.digest(codes_np(pool.v_codes, scheme)[valid], np.int16) == want["v_codes"]
        assert G.digest(np_of(pool.k_scale)[valid], np.float32) == want["k_scale"]
        vz = np.zeros_like(np_of(pool.v_scale)) if pool.v_zero is None else np_of(pool.v_zero)
        assert G.digest(vz[valid], np.float32) == want["v_zero"]
        assert G.digest(np_of(pool.ts)[valid], np.float32) == want["ts"]

    c = G.evict_case()
    pool = ops.CachePool(c["caps"], 1, 32, 32, 0, dev)
    pool.fill.copy_(to_dev(np.array(c["lens"], dtype=np.int32), dev))
    pool.acc.copy_(to_dev(c["acc"], dev))
    pool.ts.copy_(to_dev(c["ts"], dev))
    base = np_of(pool.row_base)
    for multi_block in (False, True):
        pool.evict_select(ops.EVICT_H2O, n_heavy=to_dev(c["n_heavy"], dev), n_recent=to_dev(c["n_recent"], dev),
                          multi_block=multi_block)
        flag, kidx, new_len = np_of(pool.keep_flag), np_of(pool.keep_index), np_of(pool.new_len)
        keep = np.concatenate([flag[b:b + L] for b, L in zip(base, c["lens"])])
        surv = np.concatenate([kidx[b:b + m] for b, m in zip(base, new_len)])
        assert G.digest(keep, np.uint8) == WANT["evict"]["h2o_keep"]
        assert G.digest(surv, np.int32) == WANT["evict"]["h2o_survivors"]
        assert G.digest(new_len, np.int32) == WANT["evict"]["h2o_counts"]
        pool.evict_select(ops.EVICT_LRU, n_evict=to_dev(c["n_evict"], dev), multi_block=multi_block)
        flag, new_len = np_of(pool.keep_flag), np_of(pool.new_len)
        keep = np.concatenate([flag[b:b + L] for b, L in zip(base, c["lens"])])
        assert G.digest(keep, np.uint8) == WANT["evict"]["lru_keep"]
        assert G.digest(new_len, np.int32) == WANT["evict"]["lru_counts"]
