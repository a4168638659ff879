"""Matrix products ``x @ W^T`` with weights [out, in] as checkpoints store them.

Which kernel runs is decided by the operands, never by the model:

* any float32 operand -> the true float32 kernel (plain FMAs, no matrix-core mode);
* bfloat16 x bfloat16 -> the hand-written MFMA kernels where their shape conditions hold (skinny products that
  stream the weight once, and float32-output products for logits), the library product (hipBLASLt through
  ``torch.matmul``, as the reference uses cuBLAS through candle for its linears: models/src/llama.rs:269-271,
  311, 364-365) for large bfloat16-output products, and the float32 kernel for whatever is left.
"""
from __future__ import annotations

import dataclasses
from typing import Optional

import torch

from ..kernels import ops
from .base import Begun


@dataclasses.dataclass
class ResidualSink:
    """Where a part's last product may add itself: the float32 residual rows and the norm that reads them next."""
    resid: torch.Tensor
    norm: object


@dataclasses.dataclass
class Normed:
    """What a product handed to a ``ResidualSink`` may return instead of a delta: the residual rows have the product
    added already, and ``data`` is ``norm`` of the new rows, finished."""
    data: torch.Tensor
    norm: object


def as_tensor(x) -> torch.Tensor:
    """``x`` as a tensor: a begun norm is finished."""
    return x.tensor() if isinstance(x, Begun) else x


def linear(x, w: torch.Tensor, out_dtype: Optional[torch.dtype] = None,
           out: Optional[torch.Tensor] = None, tiled=None) -> torch.Tensor:
    """x [M, K] (row stride free) times w [N, K] transposed -> [M, N] in ``out_dtype`` (default: x's dtype).
    x may be a ``Begun`` norm.  ``tiled``: a copy of ``w`` in the order the streaming kernel reads it
    (``kernels.gemm_bf16.tile_weight``), which steps of few rows read in its place."""
    out_dtype = out_dtype or x.dtype
    if x.dtype is torch.bfloat16 and w.dtype is torch.bfloat16:
        from ..kernels import gemm_bf16
        y = gemm_bf16.try_linear(x, w, out_dtype, out, tiled=tiled)
        if y is not None:
            return y
    return ops.gemm_generic(as_tensor(x), w, out_dtype, out)


def linear_delta(x, w: torch.Tensor, sink: Optional[ResidualSink] = None, tiled=None):
    """A product whose result is only ever added to the residual stream.

    With a ``sink`` whose norm can, the product adds itself to the residual rows and begins that norm (few rows) or
    the norm follows at once (many rows): the result is then a ``Begun`` norm or a ``Normed`` one, not a delta, and
    the caller hands it on as it is.  Otherwise the delta comes back for
    ``Norm.add_norm``: for few rows as float32 planes [slices, M, N] of a K-split product, which ``add_norm`` sums
    (the split keeps the whole GPU busy on a small product and costs no extra kernel).  ``tiled``: the copies of
    ``w`` in the order the few-row kernels read it (``kernels.gemm_bf16.tile_copies_resid``), if the part keeps any.
    """
    if sink is not None:
        # (a copy of w in the order its kernel reads it goes along only where the part has made one)
        y = sink.norm.add_product(sink.resid, x, w) if tiled is None or tiled.few is None else \
            sink.norm.add_product(sink.resid, x, w, tiled=tiled.few)
        if y is not None:
            return y
    x = as_tensor(x)
    if x.dtype is torch.bfloat16 and w.dtype is torch.bfloat16:
        from ..kernels import gemm_bf16
        y = gemm_bf16.linear_planes(x, w, tiled.many if tiled is not None else None)
        if y is not None:
            return y
        # many rows: the library's product, its float32 sums handed to the residual stream unrounded, as the
        # planes of the few-row kernel are
        y = gemm_bf16.try_linear(x, w, torch.float32, library_only=True)
        if y is not None:
            return y
    return linear(x, w)
