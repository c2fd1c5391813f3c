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
        self.kpools: Dict[int, torch.Tensor] = {}
        self.vpools: Dict[int, torch.Tensor] = {}
        self.states: Dict[int, Dict[str, torch.Tensor]] = {}
        ps = manager.page_size
        for name, g in manager.groups.items():
            n, kv, hd = g.pool.num_pages, g.spec.kv_heads, g.spec.head_dim
            for layer in g.spec.layers:
                self.kpools[layer] = torch.zeros((n, kv, ps, hd), dtype=dtype, device=device)
                self.vpools[layer] = torch.zeros((n, kv, hd, ps), dtype=dtype, device=device)
        for layer, req in manager.state_requests.items():
            self.states[layer] = {k: torch.zeros((manager.max_requests, *shape), dtype=req.dtype, device=device)
                                  for k, shape in req.shapes.items()}
        manager.device = self

    def binding(self, layer: int):
        m = self.manager
        if layer in m.state_requests:
            return StateBinding(self.states[layer])
        if layer in m.layer_group:
            src = m.layer_source.get(layer, layer)
            return KVBinding(m.layer_group[layer], self.kpools[src], self.vpools[src])
        return None

    def zero_state(self, slot: int) -> None:
        for tensors in self.states.values():
            for t in tensors.values():
                t[slot].zero_()

    def bytes(self) -> int:
        n = sum(t.numel() * t.element_size() for t in list(self.kpools.values()) + list(self.vpools.values()))
        return n + sum(t.numel() * t.element_size() for d in self.states.values() for t in d.values())
