"""RMSNorm fused with the residual sum.

``x * rsqrt(mean(x^2) + eps) * w`` with the statistics in float32; the reference places it before the mixer,
before the feed-forward and after the last block (models/src/llama.rs:401-408, 416-421, 474, 487).
"""
from __future__ import annotations

from typing import Dict, Optional

import torch

from ..kernels import ops
from .base import Begun, Norm, WeightSpec, register_norm


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

    # the norm begun by its neighbours (bfloat16 steps of at most 16 rows): see kernels/gemm_bf16.py; with many rows
    # the library adds its product to the residual rows itself, and the norm reads them once
    def add_product(self, resid, x, w, tiled=None):
        if self.act_dtype is not torch.bfloat16 or w.dtype is not torch.bfloat16:
            return None
        from ..kernels import gemm_bf16
        from .linear import Normed, as_tensor
        y = gemm_bf16.try_linear_resid(x, w, resid, self.weight, self.eps, tiled)
        if y is not None:
            y.norm = self
            return y
        if gemm_bf16.try_addmm_resid(as_tensor(x), w, resid):
            return Normed(self.add_norm(resid, None), self)
        return None

    def embed(self, table, tokens):
        if self.act_dtype is not torch.bfloat16 or tokens.numel() > 16 or table.shape[1] != self.width:
            return None
        resid, u, ss = ops.embed_begin_norm(tokens, table, self.weight)
        return resid, Begun(u, ss, self.eps, self.width, self)


register_norm("rmsnorm", RMSNorm)
