"""Writes tests/golden/path_digests.json: SHA-256 digests of what the path must produce
for the seeded cases of cases.py - expert indices, capacity slots, counts, quantisation
codes / scales / zero points for every scheme, the cache planes after two routed
appends, eviction keep sets and survivor lists.

The expected values come from the numpy restatement (oracle/pikv_oracle.py) AFTER its
functions were pinned by the known-answer, closed-form and brute-force checks of
tests/test_oracle.py and tests/test_oracle_properties.py; the reference itself holds no
vectors for this path and was not run.  The file freezes those semantics: the C twin,
the GPU kernels and any later edit of the restatement are compared against it.

    python tests/golden/make_golden.py
"""
import json
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, HERE)
sys.path.insert(0, os.path.join(HERE, "..", "..", "oracle"))

import cases as G          # noqa: E402
import pikv_oracle as O    # noqa: E402


def compute():
    out = {}
    c = G.router_case()
    probs, idx, w, _ = O.router_tail(c["logits"], c["k"])
    slot, count = O.capacity_slots(idx, c["E"], c["capacity"])
    out["router"] = dict(idx=G.digest(idx, np.int32), slot=G.digest(slot, np.int32), count=G.digest(count, np.int32))

    c = G.quant_case()
    for name, scheme in G.SCHEMES.items():
        for group in (32, 64, 256):
            if scheme in (0, 1) or group >= 32:
                q, s, z = O.quantize_groups(c["x"], group, scheme)
                out[f"quant/{name}/g{group}"] = dict(codes=G.digest(q, np.int16), scale=G.digest(s, np.float32),
                                                     zero=G.digest(z, np.float32))

    c = G.scatter_case()
    for name, scheme, group in (("i8_sym", 0, 64), ("i4_asym", 2, 32)):
        pool = O.CachePool(c["caps"], c["heads"] * c["dh"], group, scheme)
        for n, st in enumerate(c["steps"]):
            slot, count = O.capacity_slots(st["idx"], c["E"], st["capacity"])
            pool.quant_scatter(st["k_src"], st["v_src"], st["idx"], slot, c["k"], now=float(n + 1))
            pool.advance(count, st["capacity"])
        valid = np.concatenate([pool.valid_rows(e) for e in range(c["E"])])
        out[f"scatter/{name}"] = dict(fill=G.digest(pool.fill, np.int32),
                                      k_codes=G.digest(pool.k_codes[valid], np.int16),
                                      v_codes=G.digest(pool.v_codes[valid], np.int16),
                                      k_scale=G.digest(pool.k_scale[valid], np.float32),
                                      v_zero=G.digest(pool.v_zero[valid], np.float32),
                                      ts=G.digest(pool.ts[valid], np.float32))

    c = G.evict_case()
    base = np.concatenate([[0], np.cumsum(c["caps"])[:-1]]).astype(np.int64)
    h2o, lru, h2o_list = [], [], []
    for i, L in enumerate(c["lens"]):
        a, t = c["acc"][base[i]:base[i] + L], c["ts"][base[i]:base[i] + L]
        k1 = O.h2o_keep(a, t, int(c["n_heavy"][i]), int(c["n_recent"][i]))
        k2 = O.lru_keep(t, int(c["n_evict"][i]))
        h2o.append(k1)
        lru.append(k2)
        h2o_list.append(np.nonzero(k1)[0])
    out["evict"] = dict(h2o_keep=G.digest(np.concatenate(h2o), np.uint8), lru_keep=G.digest(np.concatenate(lru), np.uint8),
                        h2o_survivors=G.digest(np.concatenate(h2o_list), np.int32),
                        h2o_counts=G.digest([k.sum() for k in h2o], np.int32),
                        lru_counts=G.digest([k.sum() for k in lru], np.int32))
    return out


if __name__ == "__main__":
    path = os.path.join(HERE, "path_digests.json")
    with open(path, "w") as f:
        json.dump(compute(), f, indent=1, sort_keys=True)
    print("wrote", path)
