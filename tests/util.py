"""Shared helpers for the parity tests: seeded synthetic inputs in numpy and
their transfer to the GPU as float32 or bfloat16 tensors."""
from __future__ import annotations

import numpy as np

import pikv_oracle as O


def rng(seed):
    return np.random.default_rng(seed)


def kv_like(r, n, D, outlier_frac=0.01, outlier_scale=20.0, dtype="bf16"):
    """N(0,1) rows with a seeded subset of channels scaled up (the outlier
    channels of the prefill workload).  Returned as float32 values that are
    exactly representable in `dtype`."""
    x = r.standard_normal((n, D)).astype(np.float32)
    n_out = max(1, int(D * outlier_frac))
    ch = r.permutation(D)[:n_out]
    x[:, ch] *= outlier_scale
    if dtype == "bf16":
        x = O.bf16_round(x)
    return x


def to_dev(x: np.ndarray, dev, dtype="f32"):
    import torch
    t = torch.from_numpy(np.ascontiguousarray(x))
    if dtype == "bf16":
        # values are already bf16-representable: the cast is exact
        return t.to(dev).to(torch.bfloat16).contiguous()
    return t.to(dev).contiguous()


def np_of(t):
    import torch
    if t.dtype == torch.bfloat16:
        t = t.float()
    if t.dtype == torch.float16:
        t = t.float()
    return t.detach().cpu().numpy()


def codes_np(pool_or_codes, scheme, D=None):
    """Device code plane -> int16 numpy codes [rows, D]."""
    c = np_of(pool_or_codes)
    if scheme in (O.Q_I4_ASYM, O.Q_I4_SYM):
        return O.unpack_int4(c.astype(np.uint8), signed=(scheme == O.Q_I4_SYM))
    return c.astype(np.int16)


def assert_topk_of_probs(idx, probs, k, idx_ref=None, probs_ref=None, ulps=4):
    """The routing contract: the selection is the stable top-k (value descending, lower
    expert first among equal float32 values, NaN last) of the probabilities the same side
    returned - on EVERY row.  Against a second implementation (idx_ref, probs_ref) rows may
    differ only where exp() of the two sides can round differently: the reference's own
    probabilities of the two choices are then within `ulps` units in the last place at every
    rank, and such rows are rare."""
    idx = np.asarray(idx)
    probs = np.asarray(probs, dtype=np.float32)
    own = O.topk_desc(probs, k)
    assert np.array_equal(idx, own), f"{int((idx != own).any(axis=1).sum())} rows are not the top-k of their own probabilities"
    if idx_ref is None:
        return 0
    idx_ref = np.asarray(idx_ref)
    diff = (idx != idx_ref).any(axis=1)
    n = int(diff.sum())
    if n:
        pr = np.asarray(probs_ref, dtype=np.float32)[diff]
        a = np.take_along_axis(pr, idx[diff].astype(np.int64), 1)
        b = np.take_along_axis(pr, idx_ref[diff].astype(np.int64), 1)
        assert (np.abs(a - b) <= ulps * np.spacing(np.maximum(a, b))).all(), "selections differ beyond a rounding of exp()"
        assert n <= max(2, len(idx) // 500), f"{n} near-tie rows of {len(idx)}"
    return n
