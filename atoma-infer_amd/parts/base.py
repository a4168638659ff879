"""Interfaces of the parts a layer is put together from.

A part is built from its own sizes and constants only; it never sees the model
configuration and does not know which model it is in.  Every part

* declares the checkpoint tensors it binds, by name relative to its prefix
  (``weight_specs``), which serves the loader's checks and the random-weights
  writer alike;
* takes them in ``load`` (where it may fuse or re-lay them for its kernels);
* runs on device tensors with the step's ``StepContext``.

Kinds of parts are registered by name (``register_mixer`` and friends) so that a
model builder, or a test, can choose them layer by layer.
"""
from __future__ import annotations

import dataclasses
from typing import Callable, Dict, Optional, Tuple

import torch


@dataclasses.dataclass(frozen=True)
class WeightSpec:
    """One checkpoint tensor: its shape, and how the random-weights writer fills it.

    ``init``: "linear" and "embedding" draw N(0, 0.02); "norm" is 1 (plus N(0, norm_jitter) on request);
    "int_table" draws integers in [0, high).  Integer tables are kept as int32 on the device.
    """
    shape: Tuple[int, ...]
    init: str = "linear"
    high: int = 0

    @property
    def is_int(self) -> bool:
        return self.init == "int_table"


@dataclasses.dataclass(frozen=True)
class CacheSpec:
    """What a mixer keeps per token: keys and values of ``kv_heads`` heads of ``head_size``.

    ``window``: None keeps every token; w keeps the last w.  Layers whose specs are equal share one
    group of pages and one block table per request.

    ``value_size``: elements per head and token of the second tensor, when it is not as wide as the first: None
    means ``head_size``; 0 means that the mixer keeps one tensor only (a latent vector per token, say) and its
    ``LayerCache.v`` is None.  How a mixer orders the ``page_size * size`` elements of a (page, head) tile is its own
    affair; the pool only hands out the tiles.
    """
    kv_heads: int
    head_size: int
    window: Optional[int] = None
    value_size: Optional[int] = None

    def __post_init__(self):
        if self.kv_heads <= 0 or self.head_size <= 0 or (self.value_size is not None and self.value_size < 0):
            raise ValueError(f"invalid cache spec: {self}")

    @property
    def value_elements(self) -> int:
        return self.head_size if self.value_size is None else self.value_size


@dataclasses.dataclass(frozen=True)
class StateSpec:
    """Per-request state of fixed size that a mixer keeps: ``shape`` numbers per request, float32 unless ``dtype``
    ("float32", "bfloat16", "int32") says otherwise; zero at admission."""
    shape: Tuple[int, ...]
    dtype: str = "float32"

    def __post_init__(self):
        if self.dtype not in ("float32", "bfloat16", "int32"):
            raise ValueError(f"state dtype must be float32, bfloat16 or int32, not {self.dtype!r}")


WeightGetter = Callable[[str], torch.Tensor]


class Part:
    """Base of all parts."""

    def weight_specs(self) -> Dict[str, WeightSpec]:
        return {}

    def load(self, get: WeightGetter, device: torch.device, act_dtype: torch.dtype) -> None:
        """Take the tensors named in ``weight_specs`` (``get(name)`` returns the CPU tensor as stored)."""

    def device_bytes(self) -> int:
        """Bytes of weights this part reads once per step (for the roofline)."""
        return 0

    def graph_safe(self) -> bool:
        """Whether a step through this part may be recorded once into a HIP graph and replayed.

        True only if ``forward`` launches the same kernels with the same arguments for every step of the same shape
        and takes whatever differs between such steps (positions, block tables, state slots, plans) from the
        context's device tensors.  A part that branches on the context's host copies, loops over requests on the
        host or waits for the device says False, the default; a model that holds such a part runs every step
        directly."""
        return False


@dataclasses.dataclass
class Begun:
    """Activations whose norm is begun (a norm's optional short cut, see ``Norm.add_product``): ``data`` [T <= 16, W]
    bfloat16 is the residual rows times the norm's weight, ``shares`` [parts, 16] float32 the rows' sums of squares in
    parts; the finished row is ``data[t] / sqrt(shares[:, t].sum() / width + eps)``.  A product that is linear in its
    rows may finish it in its epilogue (those of ``kernels.gemm_bf16`` do); ``tensor()`` finishes it into a tensor
    for any other reader."""
    data: torch.Tensor
    shares: torch.Tensor
    eps: float
    width: int
    norm: object = None      # the part whose norm this is, so that no other takes it for its own

    @property
    def shape(self):
        return self.data.shape

    @property
    def dtype(self):
        return self.data.dtype

    def tensor(self) -> torch.Tensor:
        from ..kernels import ops
        return ops.finish_norm(self.data, self.shares, self.eps, self.width)


class Norm(Part):
    def add_norm(self, resid: torch.Tensor, delta: Optional[torch.Tensor], rows: Optional[torch.Tensor] = None,
                 ) -> torch.Tensor:
        """``resid += delta`` (float32, in place; skipped when delta is None), return norm(resid) in the activation dtype.

        With ``rows`` the sum and norm are taken at those rows only, ``resid`` stays unchanged and the result
        has one row per entry of ``rows``.
        """
        raise NotImplementedError

    # Optional: a norm may be *begun* by the kernel that makes its input rows and finished by the product that reads
    # them (``Begun``), which saves the norm's own launch where launches are what a step costs.
    # A norm that cannot says None, and the caller runs ``add_norm``.
    def add_product(self, resid: torch.Tensor, x, w: torch.Tensor, tiled=None):
        """``resid += x @ w^T`` in place with this norm of the new rows begun (``Begun``) or
        finished (``parts.linear.Normed``); or None, nothing done.  ``tiled`` is passed only by a part that keeps
        a second copy of ``w`` in the order a few-row kernel reads it (``kernels.gemm_bf16.tile_weight_resid``)."""
        return None

    def embed(self, table: torch.Tensor, tokens: torch.Tensor):
        """(resid, Begun) for the rows ``table[tokens]`` with this norm begun; or None."""
        return None


class PositionEncoding(Part):
    """Encodes positions into queries and keys."""

    def prepare(self, device: torch.device) -> None:
        """Build device tables."""

    def rotary_tables(self):
        """(cos, sin, rotary_dim) float32 tables [positions, rotary_dim/2] if this encoding is a rotation of
        half-split pairs, else None.  Mixers with a fused rotate-and-store kernel use them."""
        return None

    def apply(self, q: torch.Tensor, k: torch.Tensor, positions: torch.Tensor) -> None:
        """Encode in place: q [T, heads, hd], k [T, kv_heads, hd], positions [T] int32."""
        raise NotImplementedError

    def score_slopes(self, num_heads: int) -> Optional[torch.Tensor]:
        """float32 [num_heads] on the device, or None: an encoding that biases the attention scores by the distance,
        head h's score of the key at j for the query at p gaining ``slopes[h] * (j - p)``.  Attention with such a
        bias runs the general kernel (the matrix-core kernel has no bias)."""
        return None


class Mixer(Part):
    """Mixes information between the tokens of a request (attention here).

    Two class attributes widen the contract for parts that know how (both default to False, and a part that leaves
    them so sees tensors only): ``accepts_begun``: ``x`` may be a ``Begun`` norm, to be handed to ``linear`` and its
    fused relatives; ``takes_sink``: ``forward`` has a keyword ``sink`` (a ``ResidualSink`` or None) and may hand its
    last product to ``linear_delta(x, w, sink)``, whose result it returns as it is."""
    accepts_begun = False
    takes_sink = False

    def cache_spec(self) -> Optional[CacheSpec]:
        return None

    def state_spec(self) -> Optional[StateSpec]:
        return None

    def forward(self, x: torch.Tensor, ctx, cache) -> torch.Tensor:
        """x [T, width] in the activation dtype -> [T, width].  ``cache`` is this layer call's ``LayerCache``."""
        raise NotImplementedError


class FeedForward(Part):
    accepts_begun = False      # as for mixers
    takes_sink = False

    def forward(self, x: torch.Tensor, ctx) -> torch.Tensor:
        raise NotImplementedError


class Block(Part):
    """An arrangement of norms, a mixer and a feed-forward around the residual stream."""

    mixer: Mixer
    #: True if ``forward`` has a keyword ``next_norm``: the norm that will read this block's output (the next
    #: block's ``entry_norm()``, or the final norm), so that the block's last product may begin it
    fuses_next_norm = False

    def forward(self, resid: torch.Tensor, delta: Optional[torch.Tensor], ctx, cache) -> torch.Tensor:
        """Consume the pending ``delta`` into ``resid`` (float32 [T, width], in place) and return the new pending delta."""
        raise NotImplementedError

    def entry_norm(self) -> Optional[Norm]:
        """The norm that consumes the pending delta, if the block before may begin it; None otherwise."""
        return None


_KINDS: Dict[str, Dict[str, Callable]] = {"mixer": {}, "feed_forward": {}, "norm": {}, "position": {}, "block": {}}


def _register(family: str, name: str, factory: Callable, replace: bool):
    table = _KINDS[family]
    if name in table and not replace:
        raise ValueError(f"{family} kind '{name}' is already registered")
    table[name] = factory


def register_mixer(name, factory, *, replace=False): _register("mixer", name, factory, replace)
def register_feed_forward(name, factory, *, replace=False): _register("feed_forward", name, factory, replace)
def register_norm(name, factory, *, replace=False): _register("norm", name, factory, replace)
def register_position(name, factory, *, replace=False): _register("position", name, factory, replace)
def register_block(name, factory, *, replace=False): _register("block", name, factory, replace)


def make_part(family: str, kind: str, **params):
    """Build a part of ``family`` ("mixer", "feed_forward", "norm", "position", "block") by its registered kind."""
    table = _KINDS[family]
    if kind not in table:
        raise KeyError(f"unknown {family} kind '{kind}'; registered: {', '.join(sorted(table)) or 'none'}")
    return table[kind](**params)


def registered_kinds(family: str) -> Tuple[str, ...]:
    return tuple(sorted(_KINDS[family]))
