"""Rotary position encoding with the rotate-half pairing ``(j, j + head_dim/2)`` and
``freq_j = theta^(-2j/head_dim)`` (``crates/mach-model/src/kernels.rs:589-660``,
``crates/mach-model/src/ref_model.rs:669-704``).  The table of inverse frequencies is made
once, in 32-bit; the angle ``pos * freq`` and its sine and cosine are computed in 32-bit by
the kernel that also writes the cache."""
from __future__ import annotations

import torch

from .base import PositionEncoding
from .registry import register_position_encoding


@register_position_encoding("rotary")
class Rotary(PositionEncoding):
    def __init__(self, spec, rt):
        super().__init__(spec, rt)
        hd = spec.head_dim
        j = torch.arange(hd // 2, dtype=torch.float32)
        inv = 1.0 / torch.pow(torch.tensor(float(spec.theta), dtype=torch.float32), 2.0 * j / hd)
        self.inv_freq = inv.to(rt.device)

    def rotary_inv_freq(self):
        return self.inv_freq
