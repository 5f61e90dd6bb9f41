"""The seeded PiKVMoE case shared by make_ref_moe_golden.py (which runs the reference's module
on it, in the build container) and tests/test_gpu_moe_golden.py (which runs this package's
mirror on it): dimensions, explicit weights for every parameter the two module graphs have in
common, and the input.  Nothing here imports the reference."""
from __future__ import annotations

import zlib

import numpy as np

CONFIG = {'num_experts': 4, 'hidden_size': 256, 'num_heads': 8, 'kv_cache_size': 128,
          'cache_decrement': 0, 'num_layers': 5, 'vocab_size': 128}
BATCH, SEQ = 2, 64

# parameters of the reference's PiKVMoE that lie on the path of its first forward and that the
# mirror holds under the same names; everything under kv_caches.* (the learned pyramid compressor,
# the value LoRA, the mean-vector buffers) is outside it
SHARED_PREFIXES = ("embedding.", "experts.", "router.", "query_proj.", "key_proj.", "query_lora.",
                   "key_lora.", "vocab_proj.")


def is_shared(key: str) -> bool:
    return key.startswith(SHARED_PREFIXES)


def weight_for(key: str, shape) -> np.ndarray:
    """Deterministic float32 values for parameter `key`: N(0, s) with s chosen per kind so that
    router logits spread over a few units (top-k decided by clear margins) and activations stay
    of order one."""
    r = np.random.default_rng(zlib.crc32(key.encode()))
    shape = tuple(int(s) for s in shape)
    if key.endswith("expert_capacity"):
        return np.ones(shape, np.float32)
    if key.endswith(".bias"):
        s = 0.05
    elif "lora_B" in key:
        s = 0.05                      # the reference initialises lora_B to zero; a non-zero B exercises the LoRA path
    elif key.startswith("router."):
        s = 0.12
    elif key.startswith("embedding."):
        s = 1.0
    else:
        s = 0.06
    return (r.standard_normal(shape) * s).astype(np.float32)


def input_embeddings() -> np.ndarray:
    return np.random.default_rng(20240917).standard_normal((BATCH, SEQ, CONFIG['hidden_size'])).astype(np.float32)
