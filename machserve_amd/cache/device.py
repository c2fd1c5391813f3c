"""Device memory of the cache: K and V pools per layer, state arrays per layer."""
from __future__ import annotations

from typing import Dict

import torch

from .manager import CacheManager, KVBinding, StateBinding


class DeviceCache:
    """Pools are zero-filled once: a page that is handed out again holds old but finite
    values, which the attention kernel masks; uninitialised memory could hold NaNs that a
    zero probability does not cancel."""

    def __init__(self, manager: CacheManager, dtype: torch.dtype, device: torch.device):
        self.manager = manager
        # by (layer run, index among its requests); a pool has one page more than its group hands out, and a state
        # one slot more than there are requests: rows that fill a captured step up write there
        self._kpools: Dict[tuple, torch.Tensor] = {}
        self._vpools: Dict[tuple, torch.Tensor] = {}
        self._states: Dict[tuple, Dict[str, torch.Tensor]] = {}
        ps = manager.page_size
        for name, g in manager.groups.items():
            n, kv, hd, vhd = g.pool.num_pages + 1, g.spec.kv_heads, g.spec.head_dim, g.spec.v_head_dim
            for key in g.spec.layers:
                self._kpools[key] = torch.zeros((n, kv, ps, hd), dtype=dtype, device=device)
                self._vpools[key] = torch.zeros((n, kv, vhd, ps), dtype=dtype, device=device)
        for key, req in manager.states.items():
            self._states[key] = {k: torch.zeros((manager.max_requests + 1, *shape), dtype=req.dtype, device=device)
                                 for k, shape in req.shapes.items()}
        # the one-request view
        self.kpools = {i: t for (i, j), t in self._kpools.items() if not manager.layer_requests[i][0]}
        self.vpools = {i: t for (i, j), t in self._vpools.items() if not manager.layer_requests[i][0]}
        self.states = {i: t for (i, j), t in self._states.items() if not manager.layer_requests[i][0]}
        manager.device = self

    def _binding_of(self, key):
        m = self.manager
        if key in m.states:
            return StateBinding(self._states[key])
        if key in m.paged:
            return KVBinding(m.paged[key], self._kpools[key], self._vpools[key])
        if key in m.shared:
            src = (m.shared[key], 0)
            return KVBinding(m.paged[src], self._kpools[src], self._vpools[src])
        return None

    def binding(self, layer: int):
        """What the layer run's mixer asked for: one binding, or a list for a list of requests."""
        several, reqs = self.manager.layer_requests[layer]
        out = [self._binding_of((layer, j)) for j in range(len(reqs))]
        return out if several else out[0]

    def zero_state(self, slot: int) -> None:
        for tensors in self._states.values():
            for t in tensors.values():
                t[slot].zero_()

    def snapshot_states(self):
        """Copies of every state array (empty for a model without state)."""
        return {key: {k: t.clone() for k, t in d.items()} for key, d in self._states.items()}

    def restore_states(self, saved) -> None:
        for key, d in saved.items():
            for k, t in d.items():
                self._states[key][k].copy_(t)

    def bytes(self) -> int:
        n = sum(t.numel() * t.element_size() for t in list(self._kpools.values()) + list(self._vpools.values()))
        return n + sum(t.numel() * t.element_size() for d in self._states.values() for t in d.values())
