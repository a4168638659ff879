"""Token embedding and output head.

Embedding gather into the float32 residual stream (models/src/llama.rs:470, 481).  The head is a bias-free product
with the embedding matrix when tied, else with its own [vocab, width] matrix (models/src/llama.rs:476-477,
482-486); logits leave in float32 straight from the float32 accumulators.
"""
from __future__ import annotations

from typing import Dict, Optional

import torch

from ..kernels import ops
from .base import Part, WeightSpec
from .linear import linear


class TokenEmbedding(Part):
    def __init__(self, vocab_size: int, width: int):
        self.vocab_size, self.width = int(vocab_size), int(width)
        self.weight: Optional[torch.Tensor] = None

    def graph_safe(self) -> bool:
        return True

    def weight_specs(self) -> Dict[str, WeightSpec]:
        return {"weight": WeightSpec((self.vocab_size, self.width), "embedding")}

    def load(self, get, device, act_dtype) -> None:
        self.weight = get("weight").to(device).contiguous()

    def device_bytes(self) -> int:
        return 0  # a step reads only the rows of its tokens

    def forward(self, tokens: torch.Tensor, norm=None):
        """The float32 residual rows of ``tokens``; with ``norm`` (the norm that reads them first) a pair (rows,
        that norm begun or None)."""
        if norm is None:
            return ops.embed(tokens, self.weight)
        got = norm.embed(self.weight, tokens)
        return got if got is not None else (ops.embed(tokens, self.weight), None)


class OutputHead(Part):
    def __init__(self, width: int, vocab_size: int, tied_to: Optional[TokenEmbedding] = None):
        self.width, self.vocab_size, self.tied_to = int(width), int(vocab_size), tied_to
        self.weight: Optional[torch.Tensor] = None
        self.tiled = None

    def graph_safe(self) -> bool:
        return True

    def weight_specs(self) -> Dict[str, WeightSpec]:
        return {} if self.tied_to is not None else {"weight": WeightSpec((self.vocab_size, self.width))}

    def load(self, get, device, act_dtype) -> None:
        self.weight = self.tied_to.weight if self.tied_to is not None else get("weight").to(device).contiguous()
        # a second copy in the order the streaming kernel's waves read it, for steps of few rows (the row-major one
        # serves the embedding's gather and the products of many rows)
        self.tiled = None
        if act_dtype is torch.bfloat16 and self.weight.dtype is torch.bfloat16 and self.weight.is_cuda:
            from ..kernels import gemm_bf16
            plan = gemm_bf16.tiled_plan(self.vocab_size, self.width, swiglu=False)
            if plan is not None:
                self.tiled = gemm_bf16.tile_weight(self.weight, *plan)

    def device_bytes(self) -> int:
        return self.weight.numel() * self.weight.element_size()

    def forward(self, x) -> torch.Tensor:
        return linear(x, self.weight, torch.float32, tiled=self.tiled)
