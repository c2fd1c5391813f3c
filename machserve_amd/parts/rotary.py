"""Rotary position encoding with the rotate-half pairing ``(j, j + head_dim/2)`` and
``freq_j = theta^(-2j/head_dim)`` (``crates/mach-model/src/kernels.rs:589-660``,
``crates/mach-model/src/ref_model.rs:669-704``), optionally with YaRN's scaled frequencies
(``crates/mach-model/src/ref_model.rs:636-667``).  The table of inverse frequencies is made
once, in 32-bit; the angle ``pos * freq`` and its sine and cosine are computed in 32-bit by
the kernel that also writes the cache."""
from __future__ import annotations

import math
import weakref

import torch

from .base import PositionEncoding
from .registry import register_position_encoding


# Tables of equal frequencies on one device are one tensor: what a step's layers work out from the table (the rows'
# cosines and sines) is then found again by the table's address and made once a step, not once a layer.
_TABLES = weakref.WeakValueDictionary()


@register_position_encoding("rotary")
class Rotary(PositionEncoding):
    def __init__(self, spec, rt):
        super().__init__(spec, rt)
        hd = spec.head_dim
        j = torch.arange(hd // 2, dtype=torch.float32)
        theta = torch.tensor(float(spec.theta), dtype=torch.float32)
        inv = 1.0 / torch.pow(theta, 2.0 * j / hd)
        self.factor = 1.0
        yarn = getattr(spec, "yarn", None)
        if yarn is not None:
            # Between pair indices `low` and `high` a frequency goes over from its own value to 1 / factor of it; the
            # bounds are where beta_fast and beta_slow rotations fit the original context, clamped to the head size
            # (not to the number of pairs), every step in 32-bit as the reference takes it.
            f32 = lambda v: torch.tensor(float(v), dtype=torch.float32)
            two_ln_theta = 2.0 * torch.log(theta)

            def pair_of(rotations):
                return hd * torch.log(f32(yarn.original_max_positions) / (f32(rotations) * 2.0 * f32(math.pi))) / two_ln_theta
            low = max(float(torch.floor(pair_of(yarn.beta_fast))), 0.0)
            high = min(float(torch.ceil(pair_of(yarn.beta_slow))), hd - 1.0)
            if high == low:
                high += 0.001
            ramp = ((j - low) / (f32(high) - f32(low))).clamp(0.0, 1.0)
            inv = (1.0 / (f32(yarn.factor) * torch.pow(theta, 2.0 * j / hd))) * ramp + inv * (1.0 - ramp)
            ln = math.log(yarn.factor)
            self.factor = (0.1 * yarn.mscale * ln + 1.0) / (0.1 * yarn.mscale_all_dim * ln + 1.0)
        key = (str(rt.device), inv.numpy().tobytes())
        table = _TABLES.get(key)
        if table is None:
            table = inv.to(rt.device)
            _TABLES[key] = table
        self.inv_freq = table

    def rotary_inv_freq(self):
        return self.inv_freq

    def score_factor(self) -> float:
        """YaRN multiplies every cosine and sine, hence q and k, by a factor; a score is their product, so the
        factor's square on the scores is the same thing, and the cache keeps keys that are rotated only."""
        return self.factor * self.factor
