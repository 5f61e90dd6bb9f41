#!/usr/bin/env python3
"""Writes tests/golden/ref_moe_forward.npz: what the REFERENCE's PiKVMoE (core/single/pikv_moe.py)
computes on the seeded case of moe_case.py - the one item of the data path's callers that nothing
but the reference's own module graph can pin (router -> experts -> vocabulary projection, forward 1).

Run in the build container only (the reference tree is read from /root/reference and never
travels):  python3 tests/golden/make_ref_moe_golden.py
The GPU test reads the .npz; it does not import this script or the reference."""
from __future__ import annotations

import json
import os
import sys

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, HERE)
import moe_case as MC  # noqa: E402

REF = "/root/reference"


def main():
    sys.path.insert(0, REF)
    # core/single/distillation.py:9 imports a name from itself, so `import core.single.pikv_moe` raises
    # ImportError as the tree stands.  PiKVMoE touches that module's three names only with
    # use_distillation=True (pikv_moe.py:189-213, 318-334); an empty stand-in registered under its name
    # lets the import of pikv_moe.py - unmodified - go through.  Nothing on the path run below is replaced.
    import types
    stub = types.ModuleType("core.single.distillation")
    for name in ("PiKVDistillation", "create_teacher_model", "distillation_training_step"):
        setattr(stub, name, None)
    sys.modules["core.single.distillation"] = stub
    from core.single.config import config as ref_config
    ref_config.update(MC.CONFIG)
    ref_config['device'] = torch.device("cpu")
    from core.single import pikv_moe as ref_moe

    torch.manual_seed(0)
    model = ref_moe.PiKVMoE(rank=4, alpha=1.0)
    model.eval()
    sd = model.state_dict()
    shared = {k: tuple(v.shape) for k, v in sd.items() if MC.is_shared(k)}
    with torch.no_grad():
        for k in shared:
            sd[k].copy_(torch.from_numpy(MC.weight_for(k, shared[k])))
    model.load_state_dict(sd)
    x = torch.from_numpy(MC.input_embeddings())
    with torch.no_grad():
        routing_weights, expert_indices, top_k_weights, lb_loss, importance = model.router(x)
        # what forward() adds to every expert's output on the first call (caches still zero):
        # the learned pyramid compressor and value LoRA applied to an all-zero cache
        cached = torch.stack([model.kv_caches[i].get_all() for i in range(MC.CONFIG['num_experts'])])
        logits = model(x)
    out = {
        "routing_weights": routing_weights.numpy().astype(np.float32),
        "expert_indices": expert_indices.numpy().astype(np.int32),
        "top_k_weights": top_k_weights.numpy().astype(np.float32),
        "lb_loss": np.float32(float(lb_loss)),
        "importance": importance.numpy().astype(np.float32),
        "cached_values": cached.numpy().astype(np.float32),
        "logits": logits.numpy().astype(np.float32),
        "shared_keys": np.array(json.dumps({k: list(v) for k, v in sorted(shared.items())})),
        "all_keys": np.array(json.dumps(sorted(sd.keys()))),
        "torch_version": np.array(torch.__version__),
    }
    path = os.path.join(HERE, "ref_moe_forward.npz")
    np.savez_compressed(path, **out)
    print("wrote", path, os.path.getsize(path), "bytes;", len(shared), "shared parameters of", len(sd))


if __name__ == "__main__":
    main()
