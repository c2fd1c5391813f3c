"""Per-request sampling options, with the reference's names, defaults and meanings
(``crates/mach-model/src/sampling.rs:46-110``)."""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Dict

MASK64 = (1 << 64) - 1
RNG_GOLDEN = 0x9E3779B97F4A7C15
MAX_EDITS = 4096  # most penalised or biased tokens per request (sampling.rs:1326-1328)
MAX_TOP_LOGPROBS = 20  # sampling.rs:1330


@dataclass
class SamplingParams:
    temperature: float = 0.0        # <= 0: greedy, the smallest index among the maxima
    top_k: int = 0                  # 0: off
    top_p: float = 1.0              # >= 1: off
    seed: int = 0                   # 0: the engine uses the request's id
    presence_penalty: float = 0.0   # subtracted once from every token generated so far
    frequency_penalty: float = 0.0  # subtracted once per earlier occurrence
    logit_bias: Dict[int, float] = field(default_factory=dict)
    top_logprobs: int = 0           # report this many most probable tokens per sampled token (at most 20)

    def validate(self) -> None:
        if not 0 <= self.top_logprobs <= MAX_TOP_LOGPROBS:
            raise ValueError(f"top_logprobs {self.top_logprobs} must be in 0..{MAX_TOP_LOGPROBS}")
        if self.top_k < 0:
            raise ValueError(f"top_k {self.top_k} must be >= 0")
        if not self.top_p > 0.0:
            raise ValueError(f"top_p {self.top_p} must be > 0")
        if len(self.logit_bias) > MAX_EDITS:
            raise ValueError(f"logit_bias has {len(self.logit_bias)} entries, at most {MAX_EDITS}")

    def plain(self) -> bool:
        """Nothing but a draw from the logits: such rows can be sampled inside a captured graph."""
        return not self.edits_logits() and self.top_logprobs == 0

    def edits_logits(self) -> bool:
        return self.presence_penalty != 0.0 or self.frequency_penalty != 0.0 or bool(self.logit_bias)


def advance(state: int) -> int:
    """The state after one draw (``sampling.rs:34-37``)."""
    return (state + RNG_GOLDEN) & MASK64
