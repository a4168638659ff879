"""RMSNorm fused with the residual sum.

``x * rsqrt(mean(x^2) + eps) * w`` with the statistics in float32; the reference places it before the mixer,
before the feed-forward and after the last block (models/src/llama.rs:401-408, 416-421, 474, 487).
"""
from __future__ import annotations

from typing import Dict, Optional

import torch

from ..kernels import ops
from .base import Norm, WeightSpec, register_norm


class RMSNorm(Norm):
    def __init__(self, width: int, eps: float):
        self.width, self.eps = int(width), float(eps)
        self.weight: Optional[torch.Tensor] = None
        self.act_dtype = torch.float32

    def graph_safe(self) -> bool:
        return True

    def weight_specs(self) -> Dict[str, WeightSpec]:
        return {"weight": WeightSpec((self.width,), "norm")}

    def load(self, get, device, act_dtype) -> None:
        self.weight = get("weight").to(device).contiguous()
        self.act_dtype = act_dtype

    def device_bytes(self) -> int:
        return self.weight.numel() * self.weight.element_size()

    def add_norm(self, resid, delta, rows=None):
        return ops.add_rmsnorm(resid, delta, self.weight, self.eps, self.act_dtype, rows)


register_norm("rmsnorm", RMSNorm)
