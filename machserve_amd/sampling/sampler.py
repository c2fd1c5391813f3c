"""Sampling of one token per wanted row on the GPU.

Per step: penalties and biases are merged per (row, token) on the host and added to the
logits by one small kernel, then one kernel draws a token per row.  The SplitMix64 state of
each request lives on the host, goes up with the step's parameters and is advanced by one
draw per sampled row, greedy rows included (``crates/mach-model/src/sampling.rs:189-198,
1026-1030``)."""
from __future__ import annotations

from typing import Dict, Sequence

import numpy as np
import torch

from .params import MAX_EDITS, SamplingParams, advance


def _signed(state: int) -> int:
    return state - (1 << 64) if state >= (1 << 63) else state


class Sampler:
    def __init__(self, ops, device):
        self.ops, self.device = ops, device

    def sample(self, logits: torch.Tensor, params: Sequence[SamplingParams], states: Sequence[int],
               generated: Sequence[Sequence[int]]):
        """``logits [W, vocab]`` float32 (edited in place when a row has penalties or biases).
        Returns ``(tokens, logprobs, new_states, top)`` as host lists; ``top[r]`` is the list of
        (token, logprob) of the row's ``top_logprobs`` most probable tokens (empty if 0)."""
        W = logits.shape[0]
        rows, toks, deltas = [], [], []
        for r, p in enumerate(params):
            if not p.edits_logits():
                continue
            d: Dict[int, float] = {}
            if p.presence_penalty != 0.0 or p.frequency_penalty != 0.0:
                counts: Dict[int, int] = {}
                for t in generated[r]:
                    counts[t] = counts.get(t, 0) + 1
                for t, c in list(counts.items())[:MAX_EDITS]:
                    d[t] = d.get(t, 0.0) - (p.presence_penalty + p.frequency_penalty * c)
            for t, b in p.logit_bias.items():
                d[int(t)] = d.get(int(t), 0.0) + float(b)
            for t, v in d.items():
                rows.append(r), toks.append(t), deltas.append(v)
        if rows:
            self.ops.logit_edit(logits, torch.tensor(rows, dtype=torch.int32, device=self.device),
                                torch.tensor(toks, dtype=torch.int32, device=self.device),
                                torch.tensor(deltas, dtype=torch.float32, device=self.device))
        fl = np.empty((2, W), dtype=np.float32)
        fl[0] = [p.temperature for p in params]
        fl[1] = [p.top_p for p in params]
        fdev = torch.from_numpy(fl).to(self.device)
        kdev = torch.tensor([p.top_k for p in params], dtype=torch.int32, device=self.device)
        sdev = torch.tensor([_signed(s) for s in states], dtype=torch.int64, device=self.device)
        tok, lp = self.ops.sample(logits, fdev[0], kdev, fdev[1], sdev, any(p.temperature <= 0.0 for p in params))
        top = [[] for _ in params]
        kmax = max(p.top_logprobs for p in params)
        if kmax > 0:
            inv_t = torch.tensor([1.0 / p.temperature if p.temperature > 0.0 else 1.0 for p in params],
                                 dtype=torch.float32, device=self.device)
            ttok, tlp = self.ops.top_logprobs(logits, inv_t, kmax)
            ttok, tlp = ttok.cpu().tolist(), tlp.cpu().tolist()
            top = [list(zip(ttok[r][:p.top_logprobs], tlp[r][:p.top_logprobs])) for r, p in enumerate(params)]
        tokens = tok.cpu().tolist()  # the step's synchronisation
        return tokens, lp.cpu().tolist(), [advance(s) for s in states], top
