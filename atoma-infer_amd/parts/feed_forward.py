"""Dense SwiGLU feed-forward: ``down(silu(gate(x)) * up(x))``, no biases (models/src/llama.rs:362-366, 372-374).

gate and up are fused into one [2 I, width] matrix at load time, so one product feeds the SiLU-multiply kernel.
When I is a multiple of 16 the rows are interleaved in blocks of 16 (16 gate rows, then the 16 up rows of the
same outputs): a lane of the weight-streaming MFMA product then holds a gate value and its up value, and the
activation runs in that product's epilogue for few rows of x.
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
        self.block = 0
        self.w_gate_up: Optional[torch.Tensor] = None
        self.w_gate_up_tiled = self.w_down_tiled = None
        self.w_down: Optional[torch.Tensor] = None

    def graph_safe(self) -> bool:
        return True

    def weight_specs(self) -> Dict[str, WeightSpec]:
        return {"gate_proj.weight": WeightSpec((self.inter, self.width)),
                "up_proj.weight": WeightSpec((self.inter, self.width)),
                "down_proj.weight": WeightSpec((self.width, self.inter))}

    def load(self, get, device, act_dtype) -> None:
        g, u = get("gate_proj.weight"), get("up_proj.weight")
        dt = g.dtype if g.dtype is u.dtype else torch.float32
        g, u = g.to(device=device, dtype=dt), u.to(device=device, dtype=dt)
        self.block = 16 if self.inter % 16 == 0 else 0
        if self.block:
            gu = torch.stack([g.view(self.inter // 16, 16, self.width), u.view(self.inter // 16, 16, self.width)], dim=1)
            self.w_gate_up = gu.reshape(2 * self.inter, self.width).contiguous()
        else:
            self.w_gate_up = torch.cat([g, u], dim=0).contiguous()
        self.w_down = get("down_proj.weight").to(device).contiguous()
        # second copies of the matrices in the order the streaming kernels' waves read them, for steps of few rows
        self.w_gate_up_tiled = self.w_down_tiled = None
        if act_dtype is torch.bfloat16 and self.w_gate_up.dtype is torch.bfloat16 and self.w_down.dtype is torch.bfloat16:
            from ..kernels import gemm_bf16
            plan = gemm_bf16.tiled_plan(2 * self.inter, self.width, swiglu=True) if self.block else None
            if plan is not None:
                self.w_gate_up_tiled = gemm_bf16.tile_weight(self.w_gate_up, *plan)
            self.w_down_tiled = gemm_bf16.tile_copies_resid(self.w_down)

    def device_bytes(self) -> int:
        return sum(w.numel() * w.element_size() for w in (self.w_gate_up, self.w_down))

    accepts_begun = True
    takes_sink = True

    def forward(self, x, ctx, sink=None):
        h = None
        if self.block and x.dtype is torch.bfloat16 and self.w_gate_up.dtype is torch.bfloat16:
            from ..kernels import gemm_bf16
            h = gemm_bf16.try_linear_swiglu(x, self.w_gate_up, self.w_gate_up_tiled)
        if h is None:
            h = ops.swiglu(linear(x, self.w_gate_up), block=self.block)
        return linear_delta(h, self.w_down, sink, self.w_down_tiled)


register_feed_forward("swiglu", SwiGLU)
