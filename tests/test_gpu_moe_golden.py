"""PiKVMoE against the REFERENCE's own module (core/single/pikv_moe.py:139-336,
core/single/routing_strategy.py:100-150): tests/golden/ref_moe_forward.npz holds what the
reference's PiKVMoE computed, in the build container, on the seeded case of
tests/golden/moe_case.py (tests/golden/make_ref_moe_golden.py wrote it).  The mirror is given
the same explicit weights by parameter NAME - every parameter of the reference's first forward
outside kv_caches.* exists here under the same name and shape - and must reproduce

  * the router: blended routing weights, importance, load-balancing loss to 1e-6, the top-k
    expert indices exactly, the renormalised top-k weights to 1e-6;
  * the logits of the first forward to 1e-3 of their root-mean-square, for the part of the graph
    the two share: embedding / experts / dense combine / vocabulary projection.  The reference adds
    to every expert output the value its learned pyramid compressor and value LoRA produce for the
    still all-zero cache (kv_cache_compression.py; outside the data path, not mirrored); the
    fixture records those four vectors, and the term they contribute - a linear one - is taken off
    the reference's logits before the comparison.

Deliberately different and therefore not compared: what the caches hold afterwards (the reference
stores one mean vector per forward, this package the routed tokens' quantised rows) and with it
every later forward."""
import json
import os
import sys

import numpy as np
import pytest

from util import np_of

pytestmark = pytest.mark.gpu

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.join(HERE, "golden"))


@pytest.fixture()
def golden_config():
    import moe_case as MC
    from pikv_amd.config import config
    saved = dict(config)
    config.update(MC.CONFIG)
    config.update(kv_heads=4, kv_quant='int8', kv_group=None, capacity_factor=1.5)
    yield MC
    config.clear()
    config.update(saved)


def test_pikvmoe_matches_reference_module(dev, golden_config):
    import torch
    from pikv_amd import moe
    MC = golden_config
    gold = np.load(os.path.join(HERE, "golden", "ref_moe_forward.npz"))
    shared = json.loads(str(gold["shared_keys"]))
    model = moe.PiKVMoE(rank=4, alpha=1.0).to(dev).eval()
    sd = model.state_dict()
    # every parameter on the path of the reference's first forward is here, same name, same shape
    for key, shape in shared.items():
        assert key in sd and list(sd[key].shape) == shape, key
    ref_only = [k for k in json.loads(str(gold["all_keys"])) if k not in sd]
    assert all(k.startswith("kv_caches.") for k in ref_only), ref_only
    with torch.no_grad():
        for key, shape in shared.items():
            sd[key].copy_(torch.from_numpy(MC.weight_for(key, shape)))
    model.load_state_dict(sd)
    x = torch.from_numpy(MC.input_embeddings()).to(dev)
    with torch.no_grad():
        rw, idx, tkw, lb, imp = model.router(x)
        logits = model(x)
    assert np.array_equal(np_of(idx).astype(np.int32), gold["expert_indices"])
    assert np.abs(np_of(rw) - gold["routing_weights"]).max() <= 1e-6
    assert np.abs(np_of(tkw) - gold["top_k_weights"]).max() <= 1e-6
    assert np.abs(np_of(imp) - gold["importance"]).max() <= 1e-6
    assert abs(float(lb) - float(gold["lb_loss"])) <= 1e-6
    # logits: the reference's minus the (linear) term of its zero-cache constants
    W = MC.weight_for("vocab_proj.weight", shared["vocab_proj.weight"]).astype(np.float64)
    extra = np.einsum("bse,eh->bsh", gold["routing_weights"].astype(np.float64), gold["cached_values"].astype(np.float64))
    want = gold["logits"].astype(np.float64) - extra @ W.T
    got = np_of(logits).astype(np.float64)
    rms = np.sqrt((want ** 2).mean())
    assert np.abs(got - want).max() <= 1e-3 * rms, (np.abs(got - want).max(), rms)
    assert np.abs(extra @ W.T).max() > 1e-3 * rms      # the term taken off is not a no-op
    # the same input again: the caches now hold rows, the logits move (the mirror's cached means)
    with torch.no_grad():
        again = model(x)
    assert not torch.equal(again, logits)


def test_routing_strategy_classes_and_gradients(dev, golden_config):
    """ExpertRouter / LoadBalancingRouter / ImportanceAwareRouter (core/single/routing_strategy.py:
    6-98) against torch on the same weights: values within 1e-6, selection = stable top-k of the
    returned probabilities, additive expert mask, and gradients that reach the gate."""
    import torch
    from pikv_amd import routing_strategy as RS
    torch.manual_seed(5)
    H, E = 64, 6
    x = torch.randn(3, 17, H, device=dev)
    mask = torch.tensor([0.0, -1e9, 0.0, 0.0, -1e9, 0.0], device=dev)
    for cls in (RS.ExpertRouter, RS.LoadBalancingRouter, RS.ImportanceAwareRouter):
        r = cls(H, E, top_k=3, temperature=0.7).to(dev)
        out = r(x, expert_mask=mask)
        lg = r.router(x) / 0.7 + mask
        p = torch.softmax(lg, dim=-1)
        if cls is RS.ImportanceAwareRouter:
            impv = r.importance_predictor(x)
            assert torch.allclose(out[3], impv)
            pw = p * impv
            p_out = pw / pw.sum(-1, keepdim=True)
        else:
            p_out = p
        assert torch.allclose(out[0], p_out, atol=1e-6)
        order = torch.sort(p, dim=-1, descending=True, stable=True).indices[..., :3]
        assert torch.equal(out[1], order) or torch.allclose(p.gather(-1, out[1]), p.gather(-1, order), atol=1e-7)
        assert not torch.isin(out[1], torch.tensor([1, 4], device=dev)).any()
        sel = p.gather(-1, out[1])
        assert torch.allclose(out[2], sel / sel.sum(-1, keepdim=True), atol=1e-6)
        if cls is RS.LoadBalancingRouter:
            u = p.mean(0).mean(0)
            assert torch.allclose(out[3], 0.01 * u.std() / u.mean(), atol=1e-7)
        loss = (out[0] ** 2).sum() + out[2].sum()
        loss.backward()
        assert r.router[0].weight.grad is not None and float(r.router[0].weight.grad.abs().sum()) > 0
    ad = RS.AdaptiveRouter(H, E, top_k=2).to(dev)
    rw, idx, tkw, lb, imp = ad(x)
    assert rw.shape == (3, 17, E) and idx.shape == (3, 17, 2) and imp.shape == (3, 17, 1)
    assert torch.equal(idx, torch.sort(rw, dim=-1, descending=True, stable=True).indices[..., :2])
    (rw.sum() + tkw.sum() + lb).backward()
    assert ad.router_selector[0].weight.grad is not None
    with pytest.raises(ValueError):
        RS.ExpertRouter(H, E)(x.cpu())
