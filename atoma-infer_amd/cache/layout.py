"""The order of elements inside a (page, KV head) tile of the cache, as index tensors.

The kernels own the layout (csrc/kernels/cache_layout.h); this module states the same two formulas for code that
has to look into a cache from Python: tests, tools, and anything that moves logical [token, column] data in or out.
"""
from __future__ import annotations

import torch


def key_index(page_size: int, head_size: int) -> torch.Tensor:
    """int64 [page_size, head_size]: offset of (token t, column d) inside a key tile."""
    t = torch.arange(page_size)[:, None]
    d = torch.arange(head_size)[None, :]
    return (((d // 16) * 2 + (d % 16) // 8) * page_size + t) * 8 + d % 8


def value_index(page_size: int, head_size: int) -> torch.Tensor:
    """int64 [head_size, page_size]: offset of (column d, token t) inside a value tile."""
    d = torch.arange(head_size)[:, None]
    t = torch.arange(page_size)[None, :]
    if page_size % 16:
        return d * page_size + t
    # runs of 16 tokens, each laid out as a page of 16 tokens
    run, t = (t // 16) * 16 * head_size, t % 16
    tile, c = d // 32, d % 32
    rows = torch.clamp(head_size - tile * 32, max=32)
    return run + tile * 512 + (((t % 8) // 4) * rows + c) * 8 + (t // 8) * 4 + t % 4


def pack_keys(k: torch.Tensor) -> torch.Tensor:
    """Logical keys [..., page_size, head_size] -> tiles [..., page_size * head_size]."""
    p, h = k.shape[-2:]
    out = torch.empty(k.shape[:-2] + (p * h,), dtype=k.dtype, device=k.device)
    out[..., key_index(p, h).reshape(-1).to(k.device)] = k.reshape(k.shape[:-2] + (p * h,))
    return out


def unpack_keys(tile: torch.Tensor, page_size: int, head_size: int) -> torch.Tensor:
    return tile[..., key_index(page_size, head_size).to(tile.device)]


def pack_values(v: torch.Tensor) -> torch.Tensor:
    """Logical values [..., head_size, page_size] -> tiles [..., head_size * page_size]."""
    h, p = v.shape[-2:]
    out = torch.empty(v.shape[:-2] + (p * h,), dtype=v.dtype, device=v.device)
    out[..., value_index(p, h).reshape(-1).to(v.device)] = v.reshape(v.shape[:-2] + (p * h,))
    return out


def unpack_values(tile: torch.Tensor, page_size: int, head_size: int) -> torch.Tensor:
    return tile[..., value_index(page_size, head_size).to(tile.device)]
