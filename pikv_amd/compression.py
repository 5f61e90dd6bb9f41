"""QuantizedCompressor with the reference's interface, backed by the HIP kernels.

Mirrors core/single/pikv_compression.py:368-516 (constructor, forward,
_quantize, get_compression_stats) and the symmetric option of
core/single/module/pikv_compression.py:919-1060.  forward() reproduces the
reference's behaviour - fake quantisation with min/max taken over ALL rows of
each block of `group_size` columns, float output; with dynamic_quantization=False
the first block the module ever sees fixes one (scale, zero_point) for everything after.  quantize()/dequantize() are
the additions of this build: they keep the integer codes, at per-token,
per-token-per-head or per-group granularity (the formula is the same one).

All tensors must live on the GPU; there is no CPU path.
"""
from __future__ import annotations

from typing import Dict, Optional, Tuple

import torch
import torch.nn as nn

from . import ops


class BaseCompressor(nn.Module):
    """core/single/pikv_compression.py:7-47."""

    def __init__(self, hidden_size: int, compression_ratio: float = 0.5):
        super().__init__()
        self.hidden_size = hidden_size
        self.compression_ratio = compression_ratio

    def forward(self, keys, values, importance=None):
        return keys, values

    def get_compression_stats(self) -> Dict[str, float]:
        return {"compression_ratio": self.compression_ratio,
                "memory_reduction": 1.0 - self.compression_ratio}


class QuantizedCompressor(BaseCompressor):
    def __init__(self, hidden_size: int, bits: int = 8, group_size: int = 128,
                 dynamic_quantization: bool = True, symmetric: bool = False,
                 dynamic: Optional[bool] = None):
        super().__init__(hidden_size, bits / 32)
        if bits not in (4, 8):
            raise ValueError(f"bits must be 4 or 8, got {bits}")
        self.bits = bits
        self.group_size = min(group_size, hidden_size)
        # the module/ copy of the reference names the flag `dynamic`
        self.dynamic_quantization = dynamic_quantization if dynamic is None else dynamic
        self.symmetric = symmetric
        self.register_buffer("scale", torch.ones(1))
        self.register_buffer("zero_point", torch.zeros(1))
        self.calibrated = False
        self.register_buffer("quantization_error", torch.zeros(1))
        self.register_buffer("sample_count", torch.tensor(0.0))

    # ---- reference behaviour -------------------------------------------------
    def _fake(self, x2d: torch.Tensor, group: int):
        dq, stats, mse = ops.fakequant_colblocks(x2d, group, self.bits, self.symmetric)
        # quantization_error holds the value of the last block processed
        self.quantization_error = mse[-1:].clone()
        self.sample_count += mse.numel()
        return dq, stats

    # ---- pre-calibrated mode (core/single/pikv_compression.py:430-472) ------------------
    def _calibrate(self, x2d: torch.Tensor):
        """The first tensor the module quantises fixes scale and zero_point for good."""
        stats = ops.fakequant_colblocks(x2d, x2d.shape[1], self.bits, self.symmetric)[1]
        self.scale = stats[0, 2:3].clone()
        self.zero_point = stats[0, 3:4].clone()
        self.calibrated = True

    def _fake_static(self, x2d: torch.Tensor, group: int):
        if not self.calibrated:
            self._calibrate(x2d[:, :group].contiguous())
        # (min, max, scale, zero) row as the kernel takes it; only scale and zero are read
        preset = torch.cat([self.scale.new_zeros(2), self.scale.reshape(1).float(),
                            self.zero_point.reshape(1).float()])
        dq, mse = ops.fakequant_preset(x2d, preset, group, self.bits, self.symmetric)
        self.quantization_error = mse[-1:].clone()
        self.sample_count += mse.numel()
        return dq

    def _quantize(self, x: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
        """One reduction domain = the whole tensor x (as the reference's
        _quantize: x.min()/x.max()).  Returns (q_x, dq_x, scale); q_x holds the
        integer codes as floats, like the reference."""
        x2 = x.reshape(-1, x.shape[-1]).float().contiguous()
        if not self.dynamic_quantization:
            dq = self._fake_static(x2, x2.shape[1]).reshape(x.shape)
            return torch.round(dq / self.scale + self.zero_point), dq, self.scale
        # one column block as wide as the tensor: min/max over every element
        dq, stats = self._fake(x2, x2.shape[1])
        scale, zero = stats[0, 2], stats[0, 3]
        dq = dq.reshape(x.shape)
        # dq = (q - zero) * scale, so the codes are recovered exactly by rounding
        q = torch.round(dq / scale + zero)
        return q, dq, scale

    def forward(self, keys: torch.Tensor, values: torch.Tensor,
                importance: Optional[torch.Tensor] = None):
        """core/single/pikv_compression.py:474-506."""
        shape = keys.shape
        k2 = keys.reshape(-1, shape[-1]).float().contiguous()
        v2 = values.reshape(-1, shape[-1]).float().contiguous()
        if not self.dynamic_quantization:
            # the first column block of the first keys calibrates; everything else reuses it
            dqk = self._fake_static(k2, self.group_size)
            dqv = self._fake_static(v2, self.group_size)
            return dqk.reshape(shape).to(keys.dtype), dqv.reshape(shape).to(values.dtype)
        dqk, _ = self._fake(k2, self.group_size)
        dqv, _ = self._fake(v2, self.group_size)
        return dqk.reshape(shape).to(keys.dtype), dqv.reshape(shape).to(values.dtype)

    def get_compression_stats(self) -> Dict[str, float]:
        stats = super().get_compression_stats()
        stats.update({"bits": self.bits, "quantization_error": float(self.quantization_error.item()),
                      "group_size": self.group_size, "num_samples": float(self.sample_count.item())})
        return stats

    # ---- integer-code interface (this build) ---------------------------------
    def scheme(self) -> int:
        if self.bits == 8:
            return ops.Q_I8_SYM if self.symmetric else ops.Q_I8_ASYM
        return ops.Q_I4_SYM if self.symmetric else ops.Q_I4_ASYM

    def domain(self, granularity: str, head_dim: Optional[int] = None) -> int:
        """Number of contiguous elements that share one scale."""
        if granularity == "token":
            return self.hidden_size
        if granularity == "token_head":
            if not head_dim:
                raise ValueError("granularity='token_head' needs head_dim")
            return head_dim
        if granularity == "group":
            return self.group_size
        raise ValueError("granularity must be 'token', 'token_head' or 'group' "
                         "(the reference's all-rows domain is what forward() uses)")

    def quantize(self, x: torch.Tensor, granularity: str = "group", head_dim: Optional[int] = None):
        """(codes, scale, zero|None) with integer codes kept (4-bit codes packed
        two per byte, low nibble = even element)."""
        x2 = x.reshape(-1, x.shape[-1]).contiguous()
        return ops.quantize_rows(x2, self.domain(granularity, head_dim), self.scheme())

    def dequantize(self, codes, scale, zero, granularity: str = "group",
                   head_dim: Optional[int] = None, out_dtype=torch.float32):
        return ops.dequantize_rows(codes, scale, zero, self.domain(granularity, head_dim),
                                   self.scheme(), out_dtype)
