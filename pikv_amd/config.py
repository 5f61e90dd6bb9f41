"""Model configuration with the reference's keys and defaults
(core/single/config.py:4-17).  `device` is always the GPU: this package has no
CPU path."""
import torch

config = {
    'num_experts': 4,
    'hidden_size': 256,
    'num_heads': 8,
    'kv_cache_size': 128,
    'epochs': 10,
    'batch_size': 32,
    'learning_rate': 1e-3,
    'device': torch.device("cuda"),
    'pyramidal_cache': True,
    'cache_decrement': 10,
    'num_layers': 5,
    'vocab_size': 50257,
    # additions of this build (absent keys fall back to these values)
    'kv_heads': 4,            # heads of the cached K/V rows; head_dim = hidden_size / kv_heads
    'kv_quant': 'int8',       # 'int8' | 'int8_asym' | 'int4' | 'int4_sym'
    'kv_group': None,         # elements per scale; None = one scale per token
    'top_k': 2,
    'capacity_factor': 1.5,
}
