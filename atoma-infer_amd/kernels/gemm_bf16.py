"""bfloat16 x bfloat16 products on the matrix cores."""
from __future__ import annotations

from typing import Optional

import torch


def try_linear(x: torch.Tensor, w: torch.Tensor, out_dtype: torch.dtype, out: Optional[torch.Tensor] = None,
               ) -> Optional[torch.Tensor]:
    """x [M, K] @ w [N, K]^T if a fast kernel takes the shape, else None (the caller falls back to float32 FMAs)."""
    return None
