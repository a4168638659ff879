"""What an architecture's builder returns: parts, their checkpoint prefixes, and the order of layer calls.

The run order is data.  ``LayerCall(layer=i)`` runs layer ``i`` with a cache entry of its own; naming a layer twice
runs its weights twice, each call with its own entry; ``kv_from=j`` makes a call read the entry that call ``j``
(an earlier position of the run order) writes, and write nothing itself.
"""
from __future__ import annotations

import dataclasses
from typing import List, Optional, Tuple

from ..parts.base import Block, Norm, Part


@dataclasses.dataclass(frozen=True)
class LayerCall:
    layer: int
    kv_from: Optional[int] = None


@dataclasses.dataclass
class ModelSpec:
    width: int
    vocab_size: int
    max_positions: int
    embedding: Tuple[str, Part]
    layers: List[Tuple[str, Block]]
    final_norm: Tuple[str, Norm]
    head: Tuple[str, Part]
    run_order: List[LayerCall] = dataclasses.field(default_factory=list)
    eos_token_ids: Tuple[int, ...] = ()
    #: regular expressions of checkpoint tensors that are neither bound nor an error
    ignorable: Tuple[str, ...] = ()
    #: where the scheduler may cut a prompt: a portion that does not end the request's tokens ends at a multiple of
    #: this (1: anywhere; a mixer that scans its tokens in blocks asks for the block length)
    chunk_alignment: int = 1

    def __post_init__(self):
        if self.chunk_alignment < 1:
            raise ValueError("chunk_alignment must be at least 1")
        if not self.run_order:
            self.run_order = [LayerCall(i) for i in range(len(self.layers))]
        for pos, call in enumerate(self.run_order):
            if not 0 <= call.layer < len(self.layers):
                raise ValueError(f"run order entry {pos} names layer {call.layer}, but there are {len(self.layers)}")
            if call.kv_from is not None:
                if not 0 <= call.kv_from < pos:
                    raise ValueError(f"run order entry {pos}: kv_from must name an earlier entry")
                src = self.run_order[call.kv_from]
                if src.kv_from is not None:
                    raise ValueError(f"run order entry {pos}: kv_from names entry {call.kv_from}, which owns no cache")
                a = self.layers[call.layer][1].mixer.cache_spec()
                b = self.layers[src.layer][1].mixer.cache_spec()
                if a != b:
                    raise ValueError(f"run order entry {pos}: its cache needs {a} differ from entry "
                                     f"{call.kv_from}'s {b}")

    def graph_safe(self) -> bool:
        """Whether every part allows its steps to be recorded into HIP graphs (``Part.graph_safe``)."""
        return all(part.graph_safe() for _, part in self.parts())

    def parts(self) -> List[Tuple[str, Part]]:
        """Every (prefix, part) that binds tensors, in checkpoint order."""
        return [self.embedding] + list(self.layers) + [self.final_norm, self.head]
