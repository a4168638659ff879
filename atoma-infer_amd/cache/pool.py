"""Device memory of the cache, laid out from a model's run order.

Every layer call that owns a cache entry is put into the group of its ``CacheSpec`` (KV heads, head size,
window); a group has one pool of pages, and a page holds ``page_size`` tokens of every entry of its group, so
one page number serves all those layers (the reference does the same for its single group:
backends/vllm/src/worker.rs:570-598).  Keys and values of an entry are [pages, kv_heads, page_size * head]:
a (page, head) tile is contiguous, and the order of its elements is the one in which the MFMA attention kernel's
lanes read them (``cache/layout.py`` and csrc/kernels/cache_layout.h state it).

Mixers that declare a ``StateSpec`` get a tensor [slots, *shape] (float32 unless the spec says otherwise) per layer
call, indexed by the request's state slot.  A ``CacheSpec`` may ask for values of another width than the keys, or for
no second tensor at all.
"""
from __future__ import annotations

import dataclasses
from typing import Dict, List, Optional, Tuple

import torch

from ..parts.base import CacheSpec
from .manager import CacheManager, GroupGeometry


@dataclasses.dataclass
class GroupPlan:
    spec: CacheSpec
    calls: List[int]          # run-order positions that own an entry of this group

    def bytes_per_token(self, elem: int) -> int:
        return len(self.calls) * self.spec.kv_heads * (self.spec.head_size + self.spec.value_elements) * elem


@dataclasses.dataclass
class CachePlan:
    groups: List[GroupPlan]
    #: run-order position -> (group, entry within group, writable); absent for calls whose mixer keeps no cache
    where: Dict[int, Tuple[int, int, bool]]
    #: run-order position -> (state shape, dtype name)
    states: Dict[int, Tuple[Tuple[int, ...], str]]

    def bytes_per_token(self, elem: int) -> int:
        return sum(g.bytes_per_token(elem) for g in self.groups)


def plan_cache(spec) -> CachePlan:
    groups: List[GroupPlan] = []
    index: Dict[CacheSpec, int] = {}
    where: Dict[int, Tuple[int, int, bool]] = {}
    states: Dict[int, Tuple[Tuple[int, ...], str]] = {}
    for pos, call in enumerate(spec.run_order):
        mixer = spec.layers[call.layer][1].mixer
        st = mixer.state_spec()
        if st is not None:
            states[pos] = (tuple(st.shape), st.dtype)
        cs = mixer.cache_spec()
        if cs is None:
            continue
        if call.kv_from is not None:
            g, e, _ = where[call.kv_from]
            where[pos] = (g, e, False)
            continue
        if cs not in index:
            index[cs] = len(groups)
            groups.append(GroupPlan(cs, []))
        g = index[cs]
        where[pos] = (g, len(groups[g].calls), True)
        groups[g].calls.append(pos)
    return CachePlan(groups, where, states)


@dataclasses.dataclass
class LayerCache:
    """What one layer call sees of the cache in one step."""
    k: Optional[torch.Tensor] = None
    v: Optional[torch.Tensor] = None
    page_size: int = 1
    writable: bool = True
    group: int = -1
    slot_mapping: Optional[torch.Tensor] = None     # [T] int32: page * page_size + offset of each token
    block_tables: Optional[torch.Tensor] = None     # [S, blocks] int32
    state: Optional[torch.Tensor] = None            # [slots, *shape], float32 unless the StateSpec says otherwise


class CachePool:
    """Pages and state tensors on the device, with the manager that hands them out."""

    def __init__(self, plan: CachePlan, page_size: int, num_pages: List[int], num_state_slots: int,
                 dtype: torch.dtype, device: torch.device):
        if len(num_pages) != len(plan.groups):
            raise ValueError("one page count per group is needed")
        self.plan, self.page_size, self.dtype, self.device = plan, int(page_size), dtype, device
        self.num_state_slots = int(num_state_slots)
        self.k: List[torch.Tensor] = []
        self.v: List[Optional[torch.Tensor]] = []       # None for a group whose mixers keep one tensor only
        geometry = []
        for g, n in zip(plan.groups, num_pages):
            cs = g.spec
            # zero-filled, so that pages never written hold finite numbers
            self.k.append(torch.zeros((len(g.calls), n, cs.kv_heads, page_size * cs.head_size), dtype=dtype,
                                      device=device))
            self.v.append(torch.zeros((len(g.calls), n, cs.kv_heads, page_size * cs.value_elements), dtype=dtype,
                                      device=device) if cs.value_elements else None)
            geometry.append(GroupGeometry(page_size, n, cs.window))
        self.states = {pos: torch.zeros((num_state_slots, *shape), dtype=getattr(torch, dt), device=device)
                       for pos, (shape, dt) in plan.states.items()}
        self.manager = CacheManager(geometry, num_state_slots)

    def layer_cache(self, pos: int, slot_mappings, block_tables) -> LayerCache:
        lc = LayerCache(state=self.states.get(pos))
        if pos in self.plan.where:
            g, e, writable = self.plan.where[pos]
            lc.k, lc.page_size, lc.writable, lc.group = self.k[g][e], self.page_size, writable, g
            lc.v = self.v[g][e] if self.v[g] is not None else None
            lc.slot_mapping, lc.block_tables = slot_mappings[g], block_tables[g]
        return lc

    def bytes(self) -> int:
        return sum(t.numel() * t.element_size() for t in self.k + self.v if t is not None)


def pages_for_tokens(plan: CachePlan, page_size: int, max_tokens: int, max_requests: int) -> List[int]:
    """Pages per group that hold ``max_tokens`` tokens of at most ``max_requests`` live requests, where the caller
    has rounded each request's count up to a multiple of 64.  Page sizes that divide 64 then need no more than
    ``max_tokens / page_size`` pages; any other size rounds each request up further, by less than a page each."""
    per_group = -(-max_tokens // page_size)
    if 64 % page_size:
        per_group += max_requests
    return [max(per_group, 1) for _ in plan.groups]


def pages_for_memory(plan: CachePlan, page_size: int, elem: int, budget_bytes: int) -> List[int]:
    """Pages per group from a byte budget, the same number in each group
    (the reference: floor(free x utilization / bytes per page), backends/vllm/src/config.rs:195-208, 708-718)."""
    per_page = plan.bytes_per_token(elem) * page_size
    if per_page == 0:
        return []
    n = max(int(budget_bytes // per_page), 1)
    return [n for _ in plan.groups]
