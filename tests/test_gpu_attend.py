"""GPU parity: attention output over the compressed V cache (probabilities times
dequantised V rows) through the C ABI against a float64 evaluation on the numpy
restatement's dequantised rows.  Tolerance 1e-3 of the output's root-mean-square
(float32 path).  Both input forms are covered: raw scores + per-head softmax
statistics, and ready probabilities."""
import numpy as np
import pytest

import pikv_oracle as O
from util import np_of, rng, to_dev
from test_gpu_read_evict import _fill_pool

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("scheme,group,heads,hq,dh", [
    (O.Q_I4_ASYM, 32, 8, 32, 128),     # decode shape: matrix-core form, 4 q heads per kv head
    (O.Q_I4_SYM, 32, 2, 4, 128),       # matrix-core form, symmetric codes
    (O.Q_I4_ASYM, 32, 1, 8, 128),      # matrix-core form, all 16 operand rows in use
    (O.Q_I4_ASYM, 32, 4, 4, 128),      # matrix-core form, one row pair per kv head
    (O.Q_I4_ASYM, 32, 16, 16, 128),    # more kv heads than the matrix-core form takes: vector form
    (O.Q_I8_SYM, 128, 4, 4, 128),      # int8 per token per head
    (O.Q_I8_SYM, 256, 4, 8, 64),       # one scale per token
    (O.Q_I8_ASYM, 64, 2, 16, 64),      # 8 q heads per kv head: two passes of 4
    (O.Q_I4_SYM, 64, 4, 4, 64),
])
@pytest.mark.parametrize("form", ["stats", "probs"])
def test_attend_values(dev, scheme, group, heads, hq, dh, form):
    import torch
    r = rng(scheme * 11 + heads + hq)
    caps = [4200, 64, 130, 10]
    lens = [4100, 64, 1, 0]           # spans three token ranges, full tile, single row, empty
    pool, ref = _fill_pool(dev, r, caps, lens, heads, dh, group, scheme)
    q = O.bf16_round(r.standard_normal((len(caps), hq, dh)).astype(np.float32) * 3)
    scores, tmax, tsum = pool.scores(to_dev(q, dev, "bf16"), hq)
    pool.h2o_accumulate(scores, tmax, tsum, now=1.0, write_probs=(form == "probs"))
    out = pool.attend_values(scores, None if form == "probs" else pool.head_stats)
    got = np_of(out)
    assert got.shape == (len(caps), hq, dh)
    sc = np_of(scores)
    for c, L in enumerate(lens):
        if L == 0:
            assert not got[c].any()
            continue
        rows = ref.valid_rows(c)
        v_hat = O.dequantize_groups(ref.v_codes[rows], ref.v_scale[rows], ref.v_zero[rows], group)
        if form == "probs":
            p = sc[c, :, :L]
        else:
            p, _ = O.h2o_importance(sc[c, :, :L])
        want = O.attend_values(p, v_hat, heads)
        rms = np.sqrt((want.astype(np.float64) ** 2).mean()) + 1e-12
        err = np.abs(got[c] - want).max()
        assert err <= 1e-3 * rms, (c, err, rms)


def test_attend_peaked_distribution(dev):
    """One token carries almost all the weight: the output must equal that row of V to
    float32 accuracy, which a bf16-only weight operand would miss by 2^-9."""
    import torch
    r = rng(5)
    heads, hq, dh, L = 8, 32, 128, 300
    pool, ref = _fill_pool(dev, r, [320], [L], heads, dh, 32, O.Q_I4_ASYM)
    probs = np.full((1, hq, 320), 1e-7, dtype=np.float32)
    hot = r.integers(0, L, hq)
    probs[0, np.arange(hq), hot] = 0.77777
    out = np_of(pool.attend_values(to_dev(probs, dev)))
    rows = ref.valid_rows(0)
    v_hat = O.dequantize_groups(ref.v_codes[rows], ref.v_scale[rows], ref.v_zero[rows], 32)
    want = O.attend_values(probs[0, :, :L], v_hat, heads)
    assert np.abs(out[0] - want).max() <= 2e-5 * np.abs(want).max()
