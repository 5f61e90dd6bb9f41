"""GPU parity of the PiKVAttention mirror: a decode step attends over the whole
quantised cache natively; checked against a float64 evaluation on the numpy
restatement's quantise -> dequantise of the same K/V rows (tolerance 1e-3 of the
output's root-mean-square).  Also: past_key_values round trip and overflow handling."""
import math

import numpy as np
import pytest

import pikv_oracle as O
from util import np_of

pytestmark = pytest.mark.gpu

_SCHEME = {"int4": O.Q_I4_ASYM, "int8": O.Q_I8_SYM}


def _f64(t):
    return t.detach().double().cpu().numpy()


@pytest.mark.parametrize("quant,group,heads,kv_heads,dh", [("int4", 32, 8, 2, 128), ("int8", 64, 4, 4, 64),
                                                         ("int4", 32, 12, 12, 64),    # the head geometry of GPT-2 small
                                                         ("int8", 64, 12, 12, 64)])
def test_decode_step_over_quantised_cache(dev, quant, group, heads, kv_heads, dh):
    import torch
    from pikv_amd.attention import PiKVAttention
    torch.manual_seed(3)
    H, B, S0 = 256, 2, 70
    att = PiKVAttention(H, heads, head_dim=dh, dropout=0.0, cache_size=300, num_kv_heads=kv_heads,
                        kv_quant=quant, kv_group=group).to(dev).eval()
    with torch.no_grad():
        for m in (att.q_proj, att.k_proj, att.v_proj):
            m.weight.normal_(0.0, 0.2)
    x0 = torch.randn(B, S0, H, device=dev)
    x1 = torch.randn(B, 1, H, device=dev)
    with torch.no_grad():
        out0, (k0, v0) = att(x0, use_cache=True)
        out1, (k1, v1) = att(x1, use_cache=True)
    assert out0.shape == (B, S0, H) and out1.shape == (B, 1, H)
    assert att.cache_ptr.tolist() == [S0 + 1] * B
    D = kv_heads * dh
    scheme = _SCHEME[quant]
    rep = heads // kv_heads
    with torch.no_grad():
        q1 = att.q_proj(x1).view(B, heads, dh)
    for b in range(B):
        k_rows = np.concatenate([np_of(k0[b]).reshape(S0, D), np_of(k1[b]).reshape(1, D)])
        v_rows = np.concatenate([np_of(v0[b]).reshape(S0, D), np_of(v1[b]).reshape(1, D)])
        kq, ks, kz = O.quantize_groups(k_rows, group, scheme)
        vq, vs, vz = O.quantize_groups(v_rows, group, scheme)
        # the cache holds exactly these codes
        base = int(att.pool.row_base[b])
        from util import codes_np
        assert np.array_equal(codes_np(att.pool.k_codes, scheme)[base:base + S0 + 1], kq)
        k_hat = O.dequantize_groups(kq, ks, kz, group).astype(np.float64).reshape(S0 + 1, kv_heads, dh)
        v_hat = O.dequantize_groups(vq, vs, vz, group).astype(np.float64).reshape(S0 + 1, kv_heads, dh)
        ctx = np.zeros((heads, dh))
        for h in range(heads):
            s = k_hat[:, h // rep, :] @ _f64(q1[b, h]) / math.sqrt(dh)
            p = np.exp(s - s.max())
            p /= p.sum()
            ctx[h] = p @ v_hat[:, h // rep, :]
        want = ctx.reshape(-1) @ _f64(att.o_proj.weight).T + _f64(att.o_proj.bias)
        got = _f64(out1[b, 0])
        assert np.abs(got - want).max() <= 1e-3 * np.sqrt((want ** 2).mean())
    # the prefill call attends causally over its own tokens, in float, like the reference
    with torch.no_grad():
        q0 = att.q_proj(x0).view(B, S0, heads, dh)
    s = torch.einsum("bshd,bthd->bhst", q0, k0.repeat_interleave(rep, dim=2)) / math.sqrt(dh)
    s = s.masked_fill(torch.triu(torch.ones(S0, S0, device=dev), 1).bool(), float("-inf"))
    ctx0 = torch.einsum("bhst,bthd->bshd", torch.softmax(s, -1), v0.repeat_interleave(rep, dim=2))
    want0 = att.o_proj(ctx0.reshape(B, S0, heads * dh))
    assert torch.allclose(out0, want0, rtol=1e-4, atol=1e-5)


def test_past_key_values_round_trip_and_overflow(dev):
    import torch
    from pikv_amd.attention import PiKVAttention
    torch.manual_seed(4)
    att = PiKVAttention(128, 4, head_dim=32, dropout=0.0, cache_size=64, num_kv_heads=2, kv_quant="int8",
                        kv_group=32).to(dev).eval()
    B, L = 3, 40
    pk = torch.randn(B, 2, L, 32, device=dev)
    pv = torch.randn(B, 2, L, 32, device=dev)
    att.load_past_key_values((pk, pv))
    k, v = att.past_key_values()
    assert k.shape == (B, 2, L, 32)
    for b in range(B):
        rows = np_of(pk[b].transpose(0, 1)).reshape(L, 64)
        q, s, z = O.quantize_groups(rows, 32, O.Q_I8_SYM)
        want = O.dequantize_groups(q, s, z, 32).reshape(L, 2, 32).transpose(1, 0, 2)
        assert np.array_equal(np_of(k[b]), want)
    # decode steps until the caches overflow: H2O keeps heavy + recent rows and appends
    x = torch.randn(B, 1, 128, device=dev)
    with torch.no_grad():
        for step in range(30):
            out, _ = att(x)
            assert torch.isfinite(out).all()
            fill = att.cache_ptr
            assert int(fill.max()) <= 64 and int(fill.min()) >= 1
    assert int(att.cache_ptr.max()) < 64 + 1
    # wipe-on-overflow variant of the reference
    att2 = PiKVAttention(128, 4, head_dim=32, dropout=0.0, cache_size=16, num_kv_heads=2, kv_quant="int8",
                         kv_group=32, on_overflow="reset").to(dev).eval()
    with torch.no_grad():
        att2(torch.randn(1, 12, 128, device=dev))
        assert att2.cache_ptr.tolist() == [12]
        att2(torch.randn(1, 12, 128, device=dev))
        assert att2.cache_ptr.tolist() == [12]       # 12 + 12 > 16: wiped, then the new rows


def _dense_reference(att, x, past_k_rows, past_v_rows, key_mask=None, own_quant=None):
    """float64 attention of the module's projections over [past rows ; own rows], causal
    inside the call.  past_*_rows: [B, L, kv_heads, dh] float64 (already dequantised)."""
    import torch
    B, S, _ = x.shape
    heads, kvh, dh = att.num_heads, att.num_kv_heads, att.head_dim
    rep = heads // kvh
    with torch.no_grad():
        q = _f64(att.q_proj(x)).reshape(B, S, heads, dh)
        k = _f64(att.k_proj(x)).reshape(B, S, kvh, dh)
        v = _f64(att.v_proj(x)).reshape(B, S, kvh, dh)
    if own_quant is not None:                     # the native read path sees its own row quantised too
        group, scheme = own_quant
        k, v = [O.dequantize_groups(*O.quantize_groups(t.astype(np.float32).reshape(B * S, kvh * dh), group, scheme),
                                    group).astype(np.float64).reshape(B, S, kvh, dh) for t in (k, v)]
    L = past_k_rows.shape[1]
    out = np.zeros((B, S, heads * dh))
    for b in range(B):
        kk = np.concatenate([past_k_rows[b], k[b]])
        vv = np.concatenate([past_v_rows[b], v[b]])
        for h in range(heads):
            s = q[b, :, h] @ kk[:, h // rep].T / math.sqrt(dh)             # [S, L+S]
            for i in range(S):
                s[i, L + i + 1:] = -np.inf
            if key_mask is not None:
                s[:, ~key_mask[b]] = -np.inf
            p = np.exp(s - s.max(axis=1, keepdims=True))
            p /= p.sum(axis=1, keepdims=True)
            out[b, :, h * dh:(h + 1) * dh] = p @ vv[:, h // rep]
    return out @ _f64(att.o_proj.weight).T + _f64(att.o_proj.bias)


@pytest.mark.parametrize("layout", ["hf", "reference"])
def test_forward_attends_over_past_and_current(dev, layout):
    """core/single/pikv_attention.py:240-254: past and current K/V are concatenated along the
    sequence and attended over together - for multi-token calls and calls with a mask too."""
    import torch
    from pikv_amd.attention import PiKVAttention
    torch.manual_seed(11)
    H, heads, kvh, dh, B, L, S = 128, 4, 2, 32, 2, 23, 5
    att = PiKVAttention(H, heads, head_dim=dh, dropout=0.0, cache_size=64, num_kv_heads=kvh, kv_quant="int8",
                        kv_group=32).to(dev).eval()
    with torch.no_grad():
        for m in (att.q_proj, att.k_proj, att.v_proj):
            m.weight.normal_(0.0, 0.3)
    pk = torch.randn(B, L, kvh, dh, device=dev)           # reference layout
    pv = torch.randn(B, L, kvh, dh, device=dev)
    past = (pk, pv) if layout == "reference" else (pk.transpose(1, 2).contiguous(), pv.transpose(1, 2).contiguous())
    dq = []
    for t in (pk, pv):
        rows = np_of(t).reshape(B * L, kvh * dh)
        q, s, z = O.quantize_groups(rows, 32, O.Q_I8_SYM)
        dq.append(O.dequantize_groups(q, s, z, 32).astype(np.float64).reshape(B, L, kvh, dh))
    x = torch.randn(B, S, H, device=dev)
    with torch.no_grad():
        out, _ = att(x, past_key_values=past)
    want = _dense_reference(att, x, dq[0], dq[1])
    assert np.abs(_f64(out) - want).max() <= 1e-4 * np.sqrt((want ** 2).mean()) + 1e-6
    assert att.cache_ptr.tolist() == [L + S] * B
    # the same with a key mask over past + current (one hidden past row, one hidden own row)
    mask = torch.ones(B, L + S, device=dev)
    mask[0, 3] = 0
    mask[1, L + 1] = 0
    with torch.no_grad():
        out_m, _ = att(x, attention_mask=mask, past_key_values=past)
    want_m = _dense_reference(att, x, dq[0], dq[1], key_mask=np_of(mask) != 0)
    assert np.abs(_f64(out_m) - want_m).max() <= 1e-4 * np.sqrt((want_m ** 2).mean()) + 1e-6
    assert np.abs(want_m - want).max() > 1e-3              # the mask mattered
    # a masked single-token call also sees the past (through the dequantised rows)
    x1 = torch.randn(B, 1, H, device=dev)
    m1 = torch.ones(B, L + 1, device=dev)
    with torch.no_grad():
        out_1, _ = att(x1, attention_mask=m1, past_key_values=past)
        out_n, _ = att(x1, past_key_values=past)           # native read path, same context
    want_1 = _dense_reference(att, x1, dq[0], dq[1])
    assert np.abs(_f64(out_1) - want_1).max() <= 1e-4 * np.sqrt((want_1 ** 2).mean()) + 1e-6
    want_n = _dense_reference(att, x1, dq[0], dq[1], own_quant=(32, O.Q_I8_SYM))
    assert np.abs(_f64(out_n) - want_n).max() <= 1e-3 * np.sqrt((want_n ** 2).mean())


def test_past_key_values_shape_is_checked(dev):
    import torch
    from pikv_amd.attention import PiKVAttention
    att = PiKVAttention(128, 4, head_dim=32, dropout=0.0, cache_size=64, num_kv_heads=2, kv_quant="int8",
                        kv_group=32).to(dev).eval()
    good = torch.randn(2, 2, 10, 32, device=dev)
    with pytest.raises(ValueError):
        att.load_past_key_values((torch.randn(2, 4, 10, 32, device=dev),) * 2)       # 4 query heads, not 2 kv heads
    with pytest.raises(ValueError):
        att.load_past_key_values((torch.randn(2, 2, 10, 16, device=dev),) * 2)       # wrong head_dim
    with pytest.raises(ValueError):
        att.load_past_key_values((good, good[:, :, :5]))                             # k and v differ
    with pytest.raises(ValueError):
        att.load_past_key_values((good, good), layout="reference")                   # [B,S,heads,dh] expected
    with pytest.raises(ValueError):
        att.load_past_key_values((torch.randn(2, 2, 65, 32, device=dev),) * 2)       # longer than the cache
    with pytest.raises(ValueError):
        att.load_past_key_values(good)                                               # not a pair
    att.load_past_key_values((good, good))
    assert att.cache_ptr.tolist() == [10, 10]
    with pytest.raises(ValueError):
        att(torch.randn(3, 2, 128, device=dev))                                      # 3 sequences, 2 caches in use
    with pytest.raises(ValueError):
        att(torch.randn(2, 2, 128, device=dev), attention_mask=torch.ones(2, 7, device=dev))
    # S == kv_heads: the shape cannot tell the layouts apart, past_layout decides (with a warning)
    sq = torch.randn(1, 2, 2, 32, device=dev)
    att.load_past_key_values((sq, sq), layout="hf")
    k_hf, _ = att.past_key_values()
    att.load_past_key_values((sq, sq), layout="reference")
    k_ref, _ = att.past_key_values()
    assert torch.equal(k_hf.transpose(1, 2), k_ref)
    with pytest.warns(UserWarning, match="fits both layouts"):
        att.load_past_key_values((sq, sq))
    k_auto, _ = att.past_key_values()
    assert att.past_layout == "reference" and torch.equal(k_auto, k_ref)
    # the module reads its own `present` back correctly in either layout, also when S == kv_heads
    for lay in ("reference", "hf"):
        a2 = PiKVAttention(128, 4, head_dim=32, dropout=0.0, cache_size=64, num_kv_heads=2, kv_quant="int8",
                           kv_group=32, past_layout=lay).to(dev).eval()
        x = torch.randn(1, 2, 128, device=dev)                                       # S = 2 = kv heads
        with torch.no_grad():
            _, present = a2(x, use_cache=True)
        assert tuple(present[0].shape) == (1, 2, 2, 32)
        want_k, _ = a2.past_key_values()
        a2.reset_cache()
        with pytest.warns(UserWarning):
            a2.load_past_key_values(present)
        got_k, _ = a2.past_key_values()
        assert torch.equal(got_k, want_k), lay


def test_hf_dynamic_cache_drives_the_adapter(dev):
    """A randomly initialised GPT-2 (nothing is fetched) prefills 16 tokens; the per-layer K/V of
    the cache object the installed transformers returns go into PiKVAttention, one native
    decode step runs over them, and the result is compared with float64 attention over the
    dequantised cache.  The legacy tuple-of-tuples form that
    downstream_tasks/llm/next_tok_pred/s_transformers.py:85-98 loops over is accepted too."""
    import torch
    transformers = pytest.importorskip("transformers")
    from transformers import GPT2Config, GPT2LMHeadModel
    from pikv_amd.attention import PiKVAttention
    torch.manual_seed(5)
    cfg = GPT2Config(n_layer=2, n_head=4, n_embd=256, vocab_size=512, bos_token_id=0, eos_token_id=0)
    model = GPT2LMHeadModel(cfg).to(dev).eval()
    B, L = 2, 16
    ids = torch.randint(0, 512, (B, L), device=dev)
    with torch.no_grad():
        pkv = model(ids, use_cache=True).past_key_values
    if hasattr(pkv, "layers"):
        per_layer = [(l.keys, l.values) for l in pkv.layers]
    else:
        per_layer = [(kv[0], kv[1]) for kv in pkv]
    assert per_layer[0][0].shape == (B, 4, L, 64)
    for layer_idx in range(2):
        att = PiKVAttention(256, 4, head_dim=64, dropout=0.0, cache_size=64, kv_quant="int8", kv_group=64,
                            layer_idx=layer_idx).to(dev).eval()
        with torch.no_grad():
            for m in (att.q_proj, att.k_proj, att.v_proj):
                m.weight.normal_(0.0, 0.2)
        hk, hv = per_layer[layer_idx]
        dq = []
        for t in (hk, hv):
            rows = np_of(t.transpose(1, 2)).reshape(B * L, 256)
            q, s, z = O.quantize_groups(rows, 64, O.Q_I8_SYM)
            dq.append(O.dequantize_groups(q, s, z, 64).reshape(B, L, 4, 64))
        x = torch.randn(B, 1, 256, device=dev)
        with torch.no_grad():
            out_obj, _ = att(x, past_key_values=pkv)                     # the cache object itself
            k_back, v_back = att.past_key_values()
            out_tup, _ = att(x, past_key_values=tuple(per_layer))        # legacy per-layer tuples
        assert torch.equal(out_obj, out_tup)
        # round trip: the cache returns the dequantised rows in the Hugging Face layout
        assert k_back.shape == (B, 4, L + 1, 64)
        assert np.array_equal(np_of(k_back[:, :, :L]), dq[0].transpose(0, 2, 1, 3))
        assert np.array_equal(np_of(v_back[:, :, :L]), dq[1].transpose(0, 2, 1, 3))
        # the decode step: float64 attention over [dequantised past ; dequantised own row]
        with torch.no_grad():
            own = [np_of(p(x)).reshape(B, 256) for p in (att.k_proj, att.v_proj)]
        full = []
        for past, rows in zip(dq, own):
            q, s, z = O.quantize_groups(rows, 64, O.Q_I8_SYM)
            own_dq = O.dequantize_groups(q, s, z, 64).reshape(B, 1, 4, 64)
            full.append(np.concatenate([past, own_dq], axis=1).astype(np.float64))
        with torch.no_grad():
            qv = _f64(att.q_proj(x)).reshape(B, 4, 64)
        ctx = np.zeros((B, 256))
        for b in range(B):
            for h in range(4):
                s = full[0][b, :, h] @ qv[b, h] / 8.0
                p = np.exp(s - s.max())
                p /= p.sum()
                ctx[b, h * 64:(h + 1) * 64] = p @ full[1][b, :, h]
        want = ctx @ _f64(att.o_proj.weight).T + _f64(att.o_proj.bias)
        assert np.abs(_f64(out_obj[:, 0]) - want).max() <= 1e-3 * np.sqrt((want ** 2).mean())
