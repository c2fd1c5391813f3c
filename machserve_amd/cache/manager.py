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

Host logic only.  The bookkeeping itself (pools, tables, windows, the step's address buffer) is
the native ``CacheCore`` of ``csrc/host/cache.hpp``; this class sorts the layers' requests into
groups, names them, and hands device tensors to the layers (``DeviceCache``).
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Dict, List, Optional, Tuple

from . import CacheCore, CacheError


def group_name(window: Optional[int]) -> str:
    return "full" if window is None else f"window{window}"


@dataclass
class GroupSpec:
    name: str
    window: Optional[int]
    kv_heads: int
    head_dim: int
    v_head_dim: int = 0      # width of a value; the key's width unless the request says otherwise
    layers: List[Tuple[int, int]] = field(default_factory=list)  # (layer run, index among its requests)


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


class _PoolView:
    """Counts of one group's page pool."""

    def __init__(self, core: CacheCore, index: int):
        self._core, self._index = core, index

    @property
    def num_pages(self) -> int:
        return self._core.group_pages(self._index)

    def available(self) -> int:
        return self._core.group_available(self._index)

    def live_pages(self) -> List[int]:
        return self._core.group_live_pages(self._index)


class _Group:
    def __init__(self, spec: GroupSpec, core: CacheCore, index: int):
        self.spec, self.index = spec, index
        self.pool = _PoolView(core, index)


class _SlotsView:
    def __init__(self, core: CacheCore):
        self._core = core

    def available(self) -> int:
        return self._core.slots_available()

    def is_live(self, slot: int) -> bool:
        return self._core.slot_is_live(slot)


def pages_by_need(max_tokens: int, max_requests: int, portion: int, page_size: int):
    """A rule for :class:`CacheManager`'s ``num_pages``: a group of all keys gets the pages of ``max_tokens``
    tokens; a window group only what its requests can hold at a time, which is, for each of ``max_requests``
    requests, the pages that ``window + portion - 1`` consecutive keys touch (``portion``: the most tokens of one
    request that a step brings), and never more than the group of all keys would get.  The scheduler refuses a
    request by the same count (``csrc/host/scheduler.hpp``, ``SchedulerCore::add``)."""
    full = max(1, -(-max_tokens // page_size))

    def rule(group: "GroupSpec") -> int:
        if group.window is None:
            return full
        per_request = -(-(group.window + portion - 1) // page_size) + 1
        return max(1, min(full, max_requests * per_request))
    return rule


class CacheManager:
    def __init__(self, layer_requests, page_size: int, num_pages, max_requests: int):
        """``layer_requests[p]`` is the cache request of the p-th layer run of a step (see
        ``parts.base`` and ``DecoderModel.cache_requests``); "layer" below means such a run.
        ``num_pages``: pages of every group's pool; or a dict from group name to pages (a group it
        does not name is an error); or a rule ``GroupSpec -> pages`` (see :func:`pages_by_need`)."""
        from ..parts.base import PagedKVRequest, SharedKVRequest, StateRequest
        self.core = CacheCore(page_size, max_requests)
        self.page_size = page_size
        self.max_requests = max_requests
        self.slots = _SlotsView(self.core)
        self.groups: Dict[str, _Group] = {}
        specs: Dict[str, GroupSpec] = {}
        # A layer run may ask for several things at once (pages and state, or caches of different widths): every
        # request is kept under (layer run, index among the run's requests); a run that asked for one thing has index 0.
        self.layer_requests: Dict[int, list] = {}
        self.paged: Dict[Tuple[int, int], str] = {}        # -> group
        self.shared: Dict[Tuple[int, int], int] = {}       # -> source layer run
        self.states: Dict[Tuple[int, int], StateRequest] = {}
        for i, req in enumerate(layer_requests):
            several = isinstance(req, (list, tuple))
            reqs = list(req) if several else [req]
            self.layer_requests[i] = (several, reqs)
            for j, r in enumerate(reqs):
                if isinstance(r, PagedKVRequest):
                    v_hd = r.v_head_dim or r.head_dim
                    name = group_name(r.window)
                    g = specs.get(name)
                    if g is not None and (g.kv_heads, g.head_dim, g.v_head_dim) != (r.kv_heads, r.head_dim, v_hd):
                        # same need, other geometry: a group of its own
                        name = f"{name}/kv{r.kv_heads}x{r.head_dim}" + (f"v{v_hd}" if v_hd != r.head_dim else "")
                        g = specs.get(name)
                    if g is None:
                        g = specs[name] = GroupSpec(name, r.window, r.kv_heads, r.head_dim, v_hd)
                    g.layers.append((i, j))
                    self.paged[(i, j)] = name
                elif isinstance(r, SharedKVRequest):
                    self.shared[(i, j)] = r.source_layer
                elif isinstance(r, StateRequest):
                    self.states[(i, j)] = r
                elif r is not None:
                    raise CacheError(f"layer {i}: unknown cache request {r!r}")
        for (i, j), src in self.shared.items():
            if (src, 0) not in self.paged or self.layer_requests[src][0]:
                raise CacheError(f"layer {i} reads the cache of layer {src}, which keeps no single paged cache")
        # the one-request view, as most layers have it
        self.layer_group = {i: g for (i, j), g in self.paged.items() if not self.layer_requests[i][0]}
        self.layer_source = {i: src for (i, j), src in self.shared.items() if not self.layer_requests[i][0]}
        self.layer_group.update({i: self.paged[(src, 0)] for i, src in self.layer_source.items()})
        self.state_requests = {i: r for (i, j), r in self.states.items() if not self.layer_requests[i][0]}
        if isinstance(num_pages, dict):
            unknown = sorted(set(num_pages) - set(specs))
            missing = sorted(set(specs) - set(num_pages))
            if unknown or missing:
                raise CacheError(f"num_pages names groups {unknown} that the model has not and lacks {missing}; "
                                 f"the model's groups are {sorted(specs)}")
        for name, spec in specs.items():
            pages = num_pages[name] if isinstance(num_pages, dict) else num_pages(spec) if callable(num_pages) else num_pages
            if isinstance(pages, bool) or not isinstance(pages, int) or pages < 1:
                raise CacheError(f"group {name}: {pages!r} pages; a pool needs at least one")
            index = self.core.add_group(name, spec.window or 0, pages)
            self.groups[name] = _Group(spec, self.core, index)
        self._names = list(self.groups)
        self.device = None  # filled by DeviceCache

    # ------------------------------------------------------------------ requests
    def admit(self) -> int:
        """A state slot for a new request; its block tables start empty and its state zero."""
        slot = self.core.admit()
        if self.device is not None:
            self.device.zero_state(slot)
        return slot

    def on_admitted(self, slot: int) -> None:
        """The native scheduler admitted a request into ``slot`` by itself: zero its state."""
        if self.device is not None:
            self.device.zero_state(slot)

    def length(self, slot: int) -> int:
        return self.core.length(slot)

    @property
    def lengths(self) -> Dict[int, int]:
        return self.core.lengths()

    def pages_needed(self, slot: int, n_new: int) -> Dict[str, int]:
        """Pages each group must add before ``n_new`` more tokens of ``slot`` can be written."""
        return dict(zip(self._names, self.core.pages_needed(slot, n_new)))

    def can_extend(self, slot: int, n_new: int, reserved: Optional[Dict[str, int]] = None) -> bool:
        return self.core.can_extend(slot, n_new, [(reserved or {}).get(n, 0) for n in self._names])

    def extend(self, slot: int, n_new: int) -> None:
        """Take the pages for the next ``n_new`` tokens of ``slot`` in every group, or none at all
        (``OutOfPages``)."""
        self.core.extend(slot, n_new)

    def commit(self, slot: int, n_new: int) -> None:
        """The step wrote ``n_new`` tokens: advance the length and give back the pages that no
        later row's window reaches."""
        self.core.commit(slot, n_new)

    def release(self, slot: int) -> None:
        """The request ended (or is preempted): all its pages and its slot go back."""
        self.core.release(slot)

    # ------------------------------------------------------------------ addresses
    def table(self, group: str, slot: int) -> List[int]:
        return self.core.table(self.groups[group].index, slot)

    def slot_of_position(self, group: str, slot: int, pos: int) -> int:
        """``page * page_size + offset`` of position ``pos``
        (``crates/mach-model/src/paged_kv.rs:68`` page_offsets)."""
        return self.core.slot_of_position(self.groups[group].index, slot, pos)

    def free_pages(self, group: Optional[str] = None) -> int:
        if group is not None:
            return self.groups[group].pool.available()
        return min(g.pool.available() for g in self.groups.values()) if self.groups else 0

    def live_requests(self) -> List[int]:
        return self.core.live_requests()

    def check(self) -> None:
        """Invariants: a page is owned by at most one table entry, and every live page of a pool
        is owned.  Raises CacheError otherwise."""
        self.core.check()

    def build_step(self, slots, counts, tokens, want_rows, heads_per_kv, rows_per_block: int, table_multiple: int = 1,
                   pad_rows: int = 0, axes: int = 1, explicit_positions=(), fill=None):
        """The step's int32 buffer as ``(numpy array, {section: (start, size)}, {group: table width})``;
        see ``CacheCore::build_step`` for the sections, the rows that fill a step up and the positions.
        ``fill = (rows, requests, wanted rows)`` fills the step up to that size with rows of the scratch slot."""
        rows, seqs, want = fill or (0, 0, 0)
        return self.core.build_step(slots, counts, tokens, want_rows, list(heads_per_kv), rows_per_block, table_multiple,
                                    pad_rows, axes, list(explicit_positions), rows, seqs, want)

    @property
    def scratch_slot(self) -> int:
        """The state slot of rows that belong to no request (one beyond the requests' slots)."""
        return self.core.scratch_slot()
