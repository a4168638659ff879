"""Position encodings.

``RotaryEncoding``: rotation of half-split pairs (i, i + hd/2) by angle position x inv_freq_i.  Inverse
frequencies are ``theta^(-2i/hd)`` (models/src/llama.rs:146-152), optionally rescaled by the llama3 rule
(models/src/llama.rs:163-186).  The table of cos and sin is built once, in float32, for every position below
``max_positions`` (models/src/llama.rs:189-199) and stays float32 whatever the activation dtype is; all layers
with equal parameters share it.  ``NoPosition`` encodes nothing.
"""
from __future__ import annotations

import math
from typing import Dict, Optional, Tuple

import torch

from ..kernels import ops
from .base import PositionEncoding, register_position

_TABLES: Dict[tuple, Tuple[torch.Tensor, torch.Tensor]] = {}


def rotary_inv_freq(head_size: int, theta: float, scaling: Optional[dict]) -> torch.Tensor:
    """float32 inverse frequencies [head_size / 2]; ``scaling`` holds the llama3 constants or is None."""
    f32 = torch.float32
    exps = torch.arange(0, head_size, 2, dtype=f32) / torch.tensor(float(head_size), dtype=f32)
    freq = 1.0 / torch.pow(torch.tensor(float(theta), dtype=f32), exps)
    if scaling is None:
        return freq
    orig = torch.tensor(float(scaling["original_max_position_embeddings"]), dtype=f32)
    factor = torch.tensor(float(scaling["factor"]), dtype=f32)
    low = torch.tensor(float(scaling["low_freq_factor"]), dtype=f32)
    high = torch.tensor(float(scaling["high_freq_factor"]), dtype=f32)
    wavelen = torch.tensor(2.0, dtype=f32) * torch.tensor(math.pi, dtype=f32) / freq
    smooth = (orig / wavelen - low) / (high - low)
    mid = (1.0 - smooth) * freq / factor + smooth * freq
    return torch.where(wavelen < orig / high, freq, torch.where(wavelen > orig / low, freq / factor, mid))


class RotaryEncoding(PositionEncoding):
    def __init__(self, head_size: int, theta: float, max_positions: int, scaling: Optional[dict] = None,
                 rotary_dim: Optional[int] = None):
        self.head_size, self.theta, self.max_positions = int(head_size), float(theta), int(max_positions)
        self.scaling = dict(scaling) if scaling else None
        self.rotary_dim = int(rotary_dim) if rotary_dim is not None else self.head_size
        if self.rotary_dim % 2 or not 0 < self.rotary_dim <= self.head_size:
            raise ValueError(f"rotary_dim {self.rotary_dim} must be even and at most the head size {self.head_size}")
        self.cos = self.sin = None

    def _key(self, device):
        sc = tuple(sorted(self.scaling.items())) if self.scaling else None
        return (self.rotary_dim, self.theta, self.max_positions, sc, str(device))

    def graph_safe(self) -> bool:
        return True

    def prepare(self, device) -> None:
        key = self._key(device)
        if key not in _TABLES:
            inv = rotary_inv_freq(self.rotary_dim, self.theta, self.scaling)
            ang = torch.arange(self.max_positions, dtype=torch.float32)[:, None] * inv[None, :]
            _TABLES[key] = (torch.cos(ang).to(device).contiguous(), torch.sin(ang).to(device).contiguous())
        self.cos, self.sin = _TABLES[key]

    def load(self, get, device, act_dtype) -> None:
        self.prepare(device)

    def rotary_tables(self):
        return self.cos, self.sin, self.rotary_dim

    def apply(self, q, k, positions) -> None:
        # q and k are rotated with the same kernel that mixers fuse with the cache write, without a cache
        t, nh, hd = q.shape
        nkv = k.shape[1]
        for x, heads in ((q, nh), (k, nkv)):
            ops.rope_cache_write(x.view(t, heads * hd), positions, self.cos, self.sin, self.rotary_dim, None, None,
                                 None, 1, heads, 0, hd)


class NoPosition(PositionEncoding):
    def __init__(self, **_):
        pass

    def graph_safe(self) -> bool:
        return True

    def apply(self, q, k, positions) -> None:
        return None


def clear_tables() -> None:
    _TABLES.clear()


register_position("rotary", RotaryEncoding)
register_position("none", NoPosition)
