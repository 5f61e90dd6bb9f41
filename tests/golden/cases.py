"""Seeded inputs of the golden cases (shared by the generator and by the tests that
replay them).  Pure numpy: the same seeds give the same bytes on any machine with this
numpy version, so only the expected outputs need to be stored."""
from __future__ import annotations

import hashlib

import numpy as np

F32 = np.float32
SCHEMES = {"i8_sym": 0, "i8_asym": 1, "i4_asym": 2, "i4_sym": 3}


def digest(a, dtype) -> str:
    """SHA-256 of the array's bytes after a cast to a fixed dtype (layout independent)."""
    return hashlib.sha256(np.ascontiguousarray(np.asarray(a), dtype=dtype).tobytes()).hexdigest()


def bf16_round(x):
    u = np.ascontiguousarray(x, dtype=F32).view(np.uint32)
    r = (u + 0x7FFF + ((u >> 16) & 1)) & 0xFFFF0000
    return r.astype(np.uint32).view(F32)


def router_case():
    r = np.random.default_rng(101)
    T, E, k, cap = 700, 8, 2, 160
    lg = r.standard_normal((T, E)).astype(F32)
    lg[::3] = np.round(lg[::3] * 2) / 2          # exact ties
    lg[::5, 1] = lg[::5, 0]
    return dict(logits=lg, k=k, E=E, capacity=cap)


def quant_case():
    r = np.random.default_rng(102)
    x = r.standard_normal((96, 256)).astype(F32)
    x[:, 17] *= 20                                # an outlier channel
    x = bf16_round(x)                             # every value exact in bf16 and in float32
    x[3] = 0.0
    x[4] = 1.0                                    # constant rows
    x[5, :32] = np.arange(32) % 16 * 0.5         # rounding ties
    return dict(x=x)


def scatter_case():
    r = np.random.default_rng(103)
    E, k, heads, dh = 4, 2, 4, 64
    caps = [40, 128, 7, 64]
    steps = []
    for T in (96, 50):
        idx = np.stack([r.permutation(E)[:k] for _ in range(T)]).astype(np.int32)
        capacity = int(1 * T * 1.5 * k / E)
        ks = bf16_round(r.standard_normal((T, heads * dh)).astype(F32))
        vs = bf16_round(3 * r.standard_normal((T, heads * dh)).astype(F32))
        steps.append(dict(idx=idx, capacity=capacity, k_src=ks, v_src=vs))
    return dict(E=E, k=k, heads=heads, dh=dh, caps=caps, steps=steps)


def evict_case():
    r = np.random.default_rng(104)
    lens = [2999, 1024, 33, 1, 0, 9000]
    caps = [3000, 1024, 40, 5, 16, 9000]
    rows = int(sum(caps))
    acc = (np.round(r.random(rows) * 8) / 8).astype(F32)
    acc[::7] = 0.0
    acc[3::11] = -0.0
    ts = r.integers(0, 50, rows).astype(F32)
    n_heavy = np.array([187, 64, 2, 1, 1, 562], dtype=np.int32)
    n_recent = np.array([89, 30, 1, 1, 1, 70], dtype=np.int32)
    n_evict = np.array([1000, 0, 33, 5, 0, 8999], dtype=np.int32)
    return dict(lens=lens, caps=caps, acc=acc, ts=ts, n_heavy=n_heavy, n_recent=n_recent, n_evict=n_evict)
