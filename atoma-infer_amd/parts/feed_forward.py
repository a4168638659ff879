"""Dense SwiGLU feed-forward: ``down(silu(gate(x)) * up(x))``, no biases (models/src/llama.rs:362-366, 372-374).

gate and up are fused into one [2 I, width] matrix at load time, so one product feeds the SiLU-multiply kernel.
"""
from __future__ import annotations

from typing import Dict, Optional

import torch

from ..kernels import ops
from .base import FeedForward, WeightSpec, register_feed_forward
from .linear import linear, linear_delta


class SwiGLU(FeedForward):
    def __init__(self, width: int, intermediate: int):
        self.width, self.inter = int(width), int(intermediate)
        self.w_gate_up: Optional[torch.Tensor] = None
        self.w_down: Optional[torch.Tensor] = None

    def weight_specs(self) -> Dict[str, WeightSpec]:
        return {"gate_proj.weight": WeightSpec((self.inter, self.width)),
                "up_proj.weight": WeightSpec((self.inter, self.width)),
                "down_proj.weight": WeightSpec((self.width, self.inter))}

    def load(self, get, device, act_dtype) -> None:
        g, u = get("gate_proj.weight"), get("up_proj.weight")
        dt = g.dtype if g.dtype is u.dtype else torch.float32
        self.w_gate_up = torch.cat([g.to(device=device, dtype=dt), u.to(device=device, dtype=dt)], dim=0).contiguous()
        self.w_down = get("down_proj.weight").to(device).contiguous()

    def device_bytes(self) -> int:
        return sum(w.numel() * w.element_size() for w in (self.w_gate_up, self.w_down))

    def forward(self, x: torch.Tensor, ctx) -> torch.Tensor:
        return linear_delta(ops.swiglu(linear(x, self.w_gate_up)), self.w_down)


register_feed_forward("swiglu", SwiGLU)
