"""ctypes access to libpikv_oracle.so (the scalar C restatement,
oracle/pikv_oracle.c).  TEST INFRASTRUCTURE ONLY - used by tests/ as a second,
independently written checker and by bench.py as the timed CPU baseline.
Arrays are numpy; bfloat16 inputs are passed as uint16 bit patterns."""
from __future__ import annotations

import ctypes as C
import os
import subprocess

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
LIB = os.path.join(HERE, "libpikv_oracle.so")

F32, BF16 = 0, 1
_lib = None


def build():
    subprocess.run(["make", "-C", HERE, "-s"], check=True)
    return LIB


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(LIB):
            build()
        _lib = C.CDLL(LIB)
        _lib.pko_threads.restype = C.c_int
        _lib.pko_half_to_f32.restype = C.c_float
        _lib.pko_half_to_f32.argtypes = [C.c_uint16]
        _lib.pko_f32_to_half.restype = C.c_uint16
        _lib.pko_f32_to_half.argtypes = [C.c_float]
    return _lib


def threads() -> int:
    return int(lib().pko_threads())


def _p(a):
    return None if a is None else a.ctypes.data_as(C.c_void_p)


def _src(x):
    """numpy float32 or uint16(bf16 bits) -> (contiguous array, dtype code)."""
    x = np.ascontiguousarray(x)
    if x.dtype == np.uint16:
        return x, BF16
    return np.ascontiguousarray(x, dtype=np.float32), F32


def router(x, w, bias, k, temperature=1.0, expert_scale=None, expert_mask=None, renorm_eps=0.0):
    x, dt = _src(x)
    w, dtw = _src(w)
    assert dt == dtw
    T, H = x.shape
    E = w.shape[0]
    probs = np.empty((T, E), np.float32)
    logits = np.empty((T, E), np.float32)
    idx = np.empty((T, k), np.int32)
    wts = np.empty((T, k), np.float32)
    f = lambda v: None if v is None else np.ascontiguousarray(v, dtype=np.float32)
    bias, expert_scale, expert_mask = f(bias), f(expert_scale), f(expert_mask)
    lib().pko_router(_p(x), _p(w), C.c_int(dt), _p(bias), _p(expert_scale), _p(expert_mask),
                     C.c_float(temperature), C.c_float(renorm_eps), C.c_int64(T), C.c_int(H),
                     C.c_int(E), C.c_int(k), _p(probs), _p(logits), _p(idx), _p(wts))
    return probs, logits, idx, wts


def capacity_slots(idx, E, capacity):
    flat = np.ascontiguousarray(idx, dtype=np.int32).reshape(-1)
    slot = np.empty_like(flat)
    count = np.empty(E, np.int32)
    lib().pko_capacity_slots(_p(flat), C.c_int64(flat.size), C.c_int(E), C.c_int64(capacity),
                             _p(slot), _p(count))
    return slot.reshape(np.asarray(idx).shape), count


class CPool:
    """numpy planes in the device layout (packed int4, half metadata as uint16)."""

    def __init__(self, caps, D, group, scheme, with_v=True):
        self.cap = np.asarray(caps, np.int32)
        self.base = np.concatenate([[0], np.cumsum(self.cap.astype(np.int64))[:-1]]).astype(np.int64)
        self.rows = int(self.cap.astype(np.int64).sum())
        self.fill = np.zeros(len(self.cap), np.int32)
        self.D, self.group, self.scheme = D, group, scheme
        self.bits = 8 if scheme in (0, 1) else 4
        self.asym = scheme in (1, 2)
        ng = D // group
        cw = D if self.bits == 8 else D // 2
        md = np.float32 if self.bits == 8 else np.uint16
        mk = lambda: (np.zeros((self.rows, cw), np.int8 if scheme == 0 else np.uint8),
                      np.zeros((self.rows, ng), md), np.zeros((self.rows, ng), md))
        self.k_codes, self.k_scale, self.k_zero = mk()
        self.with_v = with_v
        self.v_codes, self.v_scale, self.v_zero = mk() if with_v else (None, None, None)
        self.acc = np.zeros(self.rows, np.float32)
        self.ts = np.zeros(self.rows, np.float32)

    def quant_scatter(self, k_src, v_src, cache_id, slot, fanout, now=0.0):
        k_src, dt = _src(k_src)
        k2 = k_src.reshape(-1, self.D)
        v2 = None
        if self.with_v:
            v_src, _ = _src(v_src)
            v2 = v_src.reshape(-1, self.D)
        cid = np.ascontiguousarray(cache_id, np.int32).reshape(-1)
        sl = np.ascontiguousarray(slot, np.int32).reshape(-1)
        lib().pko_quant_scatter(_p(k2), _p(v2), C.c_int(dt), C.c_int64(k2.shape[0]), C.c_int(fanout),
                                C.c_int(self.D), C.c_int(self.group), C.c_int(self.scheme),
                                _p(cid), _p(sl), _p(self.base), _p(self.fill), _p(self.cap),
                                C.c_int64(0), _p(self.k_codes), _p(self.v_codes), _p(self.k_scale),
                                _p(self.v_scale), _p(self.k_zero), _p(self.v_zero), _p(self.acc),
                                _p(self.ts), C.c_float(now))

    def advance(self, count, limit=-1):
        add = np.asarray(count, np.int64)
        if limit >= 0:
            add = np.minimum(add, limit)
        self.fill = np.minimum(self.fill.astype(np.int64) + add, self.cap).astype(np.int32)

    def gather_dequant(self, which="k", row0=0, n=None):
        codes, scale, zero = ((self.k_codes, self.k_scale, self.k_zero) if which == "k"
                              else (self.v_codes, self.v_scale, self.v_zero))
        n = self.rows - row0 if n is None else n
        out = np.empty((n, self.D), np.float32)
        lib().pko_gather_dequant(_p(codes), _p(scale), _p(zero), C.c_int(self.D), C.c_int(self.group),
                                 C.c_int(self.scheme), None, C.c_int64(row0), C.c_int64(n), _p(out))
        return out

    def scores_h2o(self, q, n_kv, n_q, dh, scale_qk, now, decay=1.0, want_scores=True):
        q, qdt = _src(q)
        stride = int(self.cap.max())
        scores = np.zeros((len(self.cap), n_q, stride), np.float32) if want_scores else None
        imp = np.zeros((len(self.cap), stride), np.float32)
        lib().pko_scores_h2o(_p(self.k_codes), _p(self.k_scale), _p(self.k_zero), C.c_int(self.scheme),
                             C.c_int(self.group), C.c_int(n_kv), C.c_int(n_q), C.c_int(dh), _p(q),
                             C.c_int(qdt), C.c_float(scale_qk), _p(self.base), _p(self.fill),
                             C.c_int(len(self.cap)), C.c_int64(stride), C.c_float(decay),
                             C.c_float(now), _p(scores), _p(self.acc), _p(self.ts), _p(imp))
        return scores, imp

    def evict(self, policy, n_heavy, n_recent=None, compact=True):
        nh = np.ascontiguousarray(n_heavy, np.int32)
        nr = None if n_recent is None else np.ascontiguousarray(n_recent, np.int32)
        flag = np.zeros(self.rows, np.uint8)
        kidx = np.zeros(self.rows, np.int32)
        new_len = np.zeros(len(self.cap), np.int32)
        lib().pko_evict_select(C.c_int(policy), _p(self.acc), _p(self.ts), _p(self.base),
                               _p(self.fill), _p(nh), _p(nr), C.c_int(len(self.cap)), _p(flag),
                               _p(kidx), _p(new_len))
        if compact:
            for pl in (self.k_codes, self.k_scale, self.k_zero, self.v_codes, self.v_scale,
                       self.v_zero, self.acc, self.ts):
                if pl is None:
                    continue
                rb = pl.strides[0]
                lib().pko_compact_plane(_p(pl), C.c_int64(rb), _p(self.base), _p(kidx), _p(new_len),
                                        C.c_int(len(self.cap)))
            self.fill = new_len.copy()
        return flag, kidx, new_len
