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


@pytest.mark.parametrize("quant,group,heads,kv_heads,dh", [("int4", 32, 8, 2, 128), ("int8", 64, 4, 4, 64)])
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
