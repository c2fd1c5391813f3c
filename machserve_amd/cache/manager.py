"""The cache manager: pages of keys and values, a block table per request, and slots for
per-request state of fixed size.

Layers are sorted into *groups* by what they need: all keys ("full"), or a window of the
most recent ``W`` keys ("window{W}").  Each group has a page pool and block tables of its
own, shared by the layers of the group (one page id addresses the same page in each of
their K and V pools, as in ``crates/mach-model/src/paged_kv.rs:3-5``).  Pages are taken when
a step needs them, one logical page at a time, and given back when the request ends or,
in a window group, when every later row's window has passed the page; freed pages are
handed out again.  A request also holds one *state slot*: an index into arrays
``[slots, ...]`` that mixers with state of fixed size own, zeroed on admission
(the reference indexes its recurrent state by slot the same way,
``crates/mach-model/src/batched.rs:410-415, 2644-2683``).

Layout of a page: keys ``[kv_heads, page_size, head_dim]``, values transposed
``[kv_heads, head_dim, page_size]``.

This module is host logic only; device tensors are made by ``allocate_device``.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Dict, List, Optional, Tuple

from .pool import BlockPool, CacheError, OutOfPages, SlotPool


def group_name(window: Optional[int]) -> str:
    return "full" if window is None else f"window{window}"


@dataclass
class GroupSpec:
    name: str
    window: Optional[int]
    kv_heads: int
    head_dim: int
    layers: List[int] = field(default_factory=list)


@dataclass
class KVBinding:
    """What an attention layer gets: the group whose tables address its pools, and the pools."""
    group: str
    kpool: object = None
    vpool: object = None


@dataclass
class StateBinding:
    """What a mixer with state gets: ``tensors[name]`` is ``[slots, *shape]``."""
    tensors: Dict[str, object]


class _Group:
    def __init__(self, spec: GroupSpec, page_size: int, num_pages: int):
        self.spec = spec
        self.page_size = page_size
        self.pool = BlockPool(num_pages)
        self.tables: Dict[int, List[int]] = {}
        self.first_live: Dict[int, int] = {}  # first logical page not yet given back


class CacheManager:
    def __init__(self, layer_requests, page_size: int, num_pages: int, max_requests: int):
        """``layer_requests[p]`` is the cache request of the p-th layer run of a step (see
        ``parts.base`` and ``DecoderModel.cache_requests``); "layer" below means such a run."""
        from ..parts.base import PagedKVRequest, SharedKVRequest, StateRequest
        if page_size < 16 or page_size % 16:
            raise CacheError(f"page size {page_size} must be a positive multiple of 16")
        if max_requests < 1:
            raise CacheError("at least one request slot is needed")
        self.page_size = page_size
        self.max_requests = max_requests
        self.slots = SlotPool(max_requests)
        self.lengths: Dict[int, int] = {}
        self.groups: Dict[str, _Group] = {}
        self.layer_group: Dict[int, str] = {}
        self.layer_source: Dict[int, int] = {}
        self.state_requests: Dict[int, StateRequest] = {}
        specs: Dict[str, GroupSpec] = {}
        for i, req in enumerate(layer_requests):
            if isinstance(req, PagedKVRequest):
                name = group_name(req.window)
                if name not in specs:
                    specs[name] = GroupSpec(name, req.window, req.kv_heads, req.head_dim)
                g = specs[name]
                if (g.kv_heads, g.head_dim) != (req.kv_heads, req.head_dim):
                    # same need, other geometry: a group of its own
                    name = f"{name}/kv{req.kv_heads}x{req.head_dim}"
                    g = specs.setdefault(name, GroupSpec(name, req.window, req.kv_heads, req.head_dim))
                g.layers.append(i)
                self.layer_group[i] = name
            elif isinstance(req, SharedKVRequest):
                self.layer_source[i] = req.source_layer
            elif isinstance(req, StateRequest):
                self.state_requests[i] = req
            elif req is not None:
                raise CacheError(f"layer {i}: unknown cache request {req!r}")
        for i, src in self.layer_source.items():
            if src not in self.layer_group:
                raise CacheError(f"layer {i} reads the cache of layer {src}, which keeps none")
            self.layer_group[i] = self.layer_group[src]
        for name, spec in specs.items():
            self.groups[name] = _Group(spec, page_size, num_pages)
        self.device = None  # filled by allocate_device

    # ------------------------------------------------------------------ requests
    def admit(self) -> int:
        """A state slot for a new request; its block tables start empty and its state zero."""
        slot = self.slots.alloc()
        if slot is None:
            raise CacheError(f"all {self.max_requests} request slots are in use")
        self.lengths[slot] = 0
        for g in self.groups.values():
            g.tables[slot] = []
            g.first_live[slot] = 0
        if self.device is not None:
            self.device.zero_state(slot)
        return slot

    def length(self, slot: int) -> int:
        return self.lengths[slot]

    def pages_needed(self, slot: int, n_new: int) -> Dict[str, int]:
        """Pages each group must add before ``n_new`` more tokens of ``slot`` can be written."""
        end = self.lengths[slot] + n_new
        need = {}
        for name, g in self.groups.items():
            have = len(g.tables[slot])
            need[name] = max(0, -(-end // self.page_size) - have)
        return need

    def can_extend(self, slot: int, n_new: int, reserved: Optional[Dict[str, int]] = None) -> bool:
        need = self.pages_needed(slot, n_new)
        return all(self.groups[n].pool.available() - (reserved or {}).get(n, 0) >= k for n, k in need.items())

    def extend(self, slot: int, n_new: int) -> None:
        """Take the pages for the next ``n_new`` tokens of ``slot`` in every group, or none at all."""
        if not self.slots.is_live(slot):
            raise CacheError(f"slot {slot} is not in use")
        need = self.pages_needed(slot, n_new)
        for name, k in need.items():
            if self.groups[name].pool.available() < k:
                raise OutOfPages(f"group {name}: {k} pages needed for {n_new} tokens of slot {slot}, "
                                 f"{self.groups[name].pool.available()} free")
        for name, k in need.items():
            g = self.groups[name]
            for _ in range(k):
                g.tables[slot].append(g.pool.alloc())

    def commit(self, slot: int, n_new: int) -> None:
        """The step wrote ``n_new`` tokens: advance the length and give back the pages that no
        later row's window reaches."""
        self.lengths[slot] += n_new
        L = self.lengths[slot]
        for g in self.groups.values():
            W = g.spec.window
            if W is None:
                continue
            # the next row is at position L and sees keys > L - W
            dead = max(0, L - W + 1) // self.page_size
            table = g.tables[slot]
            for p in range(g.first_live[slot], min(dead, len(table))):
                if table[p] >= 0:
                    g.pool.free(table[p])
                    table[p] = -1
            g.first_live[slot] = max(g.first_live[slot], min(dead, len(table)))

    def release(self, slot: int) -> None:
        """The request ended (or is preempted): all its pages and its slot go back."""
        if not self.slots.is_live(slot):
            raise CacheError(f"slot {slot} released twice or never admitted")
        for g in self.groups.values():
            for p in g.tables.pop(slot):
                if p >= 0:
                    g.pool.free(p)
            g.first_live.pop(slot)
        del self.lengths[slot]
        self.slots.free(slot)

    # ------------------------------------------------------------------ addresses
    def table(self, group: str, slot: int) -> List[int]:
        return self.groups[group].tables[slot]

    def slot_of_position(self, group: str, slot: int, pos: int) -> int:
        """``page * page_size + offset`` of position ``pos``
        (``crates/mach-model/src/paged_kv.rs:68`` page_offsets)."""
        page = self.groups[group].tables[slot][pos // self.page_size]
        if page < 0:
            raise CacheError(f"group {group}: position {pos} of slot {slot} lies in a page already given back")
        return page * self.page_size + pos % self.page_size

    def free_pages(self, group: Optional[str] = None) -> int:
        if group is not None:
            return self.groups[group].pool.available()
        return min(g.pool.available() for g in self.groups.values()) if self.groups else 0

    def live_requests(self) -> List[int]:
        return sorted(self.lengths)

    def check(self) -> None:
        """Invariants: a page is owned by at most one table entry, and every live page of a pool
        is owned.  Raises CacheError otherwise."""
        for name, g in self.groups.items():
            owned: Dict[int, Tuple[int, int]] = {}
            for slot, table in g.tables.items():
                for i, p in enumerate(table):
                    if p < 0:
                        continue
                    if p in owned:
                        raise CacheError(f"group {name}: page {p} held by slot {owned[p][0]} and slot {slot}")
                    owned[p] = (slot, i)
            live = set(g.pool.live_pages())
            if live != set(owned):
                raise CacheError(f"group {name}: live pages {sorted(live)} differ from owned pages {sorted(owned)}")
            if len(live) + g.pool.available() != g.pool.num_pages:
                raise CacheError(f"group {name}: {len(live)} live + {g.pool.available()} free != {g.pool.num_pages}")
