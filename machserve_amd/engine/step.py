"""The one step function: a batch of (request, its next tokens), prompt portions beside
single decoded tokens, cut anywhere.  It runs only the tokens it is given, as one batch,
from the cache that earlier steps left, and returns the logits at the wanted places.

Role in the reference: ``BatchedModel::decode_step_explicit``
(``crates/mach-model/src/batched.rs:4705-4834``), which takes rows of (token, position, slot)
and computes logits for every row; here the caller names the rows it wants.

Per step the host builds one int32 buffer (tokens, positions, per-request row ranges, the
groups' block tables and write addresses, attention work lists) and copies it to the
device once; everything after that is kernel launches on one stream.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Dict, List, Optional, Sequence

import numpy as np
import torch

from ..cache import CacheManager
from ..parts.base import GroupView, StepContext


class StepError(ValueError):
    pass


@dataclass
class StepEntry:
    slot: int                 # the request's state slot (from CacheManager.admit)
    tokens: Sequence[int]     # its next tokens, in order
    want: Sequence[int] = ()  # indices into ``tokens`` whose logits are wanted


class StepFunction:
    def __init__(self, model, cache: CacheManager, rt, attention_rows_per_block: int = 64):
        self.model, self.cache, self.rt = model, cache, rt
        self.rows_per_block = attention_rows_per_block
        self.heads_per_kv = model.attention_rows_per_token()

    # ------------------------------------------------------------------ context
    def build_context(self, entries: Sequence[StepEntry]) -> StepContext:
        cache, ps = self.cache, self.cache.page_size
        if not entries:
            raise StepError("a step needs at least one entry")
        seen = set()
        vocab = self.model.vocab
        tokens: List[int] = []
        positions: List[int] = []
        q_start, q_len, pos0, slots, want = [], [], [], [], []
        for e in entries:
            n = len(e.tokens)
            if n == 0:
                raise StepError(f"slot {e.slot}: an entry needs at least one token")
            if e.slot in seen:
                raise StepError(f"slot {e.slot} appears twice in one step")
            seen.add(e.slot)
            p0 = cache.length(e.slot)
            if p0 + n > self.model.spec.max_positions:
                raise StepError(f"slot {e.slot}: position {p0 + n - 1} is beyond the model's "
                                f"{self.model.spec.max_positions} positions")
            for t in e.tokens:
                if not 0 <= int(t) < vocab:
                    raise StepError(f"slot {e.slot}: token {t} is outside the vocabulary of {vocab}")
            for w in e.want:
                if not 0 <= w < n:
                    raise StepError(f"slot {e.slot}: wanted place {w} is outside its {n} tokens")
                want.append(len(tokens) + w)
            q_start.append(len(tokens))
            q_len.append(n)
            pos0.append(p0)
            slots.append(e.slot)
            tokens.extend(int(t) for t in e.tokens)
            positions.extend(range(p0, p0 + n))
        T, S = len(tokens), len(entries)

        sections: Dict[str, np.ndarray] = {
            "tokens": np.asarray(tokens, dtype=np.int32), "positions": np.asarray(positions, dtype=np.int32),
            "seq_q_start": np.asarray(q_start, dtype=np.int32), "seq_q_len": np.asarray(q_len, dtype=np.int32),
            "seq_pos0": np.asarray(pos0, dtype=np.int32), "seq_slot": np.asarray(slots, dtype=np.int32),
            "want_rows": np.asarray(want, dtype=np.int32),
        }
        group_shapes = {}
        for name in cache.groups:
            width = max(1, max(len(cache.table(name, s)) for s in slots))
            table = np.full((S, width), -1, dtype=np.int32)
            slot_map = np.empty(T, dtype=np.int32)
            for i, s in enumerate(slots):
                t = cache.table(name, s)
                table[i, :len(t)] = t
                pos = np.arange(pos0[i], pos0[i] + q_len[i])
                pages = np.asarray(t, dtype=np.int64)[pos // ps]
                if (pages < 0).any():
                    raise StepError(f"group {name}: slot {s} writes into a page already given back")
                slot_map[q_start[i]:q_start[i] + q_len[i]] = pages * ps + pos % ps
            sections[f"table/{name}"] = table.reshape(-1)
            sections[f"slot_map/{name}"] = slot_map
            group_shapes[name] = (S, width)
        for g in self.heads_per_kv:
            work = [(i, r0) for i in range(S) for r0 in range(0, q_len[i] * g, self.rows_per_block)]
            sections[f"work/{g}"] = np.asarray(work, dtype=np.int32).reshape(-1)

        # one buffer, one copy; every section starts on a 16-byte boundary
        offsets, total = {}, 0
        for k, a in sections.items():
            offsets[k] = total
            total += (a.size + 3) // 4 * 4
        host = np.zeros(max(total, 4), dtype=np.int32)
        for k, a in sections.items():
            host[offsets[k]:offsets[k] + a.size] = a
        dev = torch.from_numpy(host).to(self.rt.device)

        def sec(k):
            return dev[offsets[k]:offsets[k] + sections[k].size]

        ctx = StepContext(
            n_rows=T, n_seqs=S, tokens=sec("tokens"), positions=sec("positions"), seq_q_start=sec("seq_q_start"),
            seq_q_len=sec("seq_q_len"), seq_pos0=sec("seq_pos0"), seq_slot=sec("seq_slot"), want_rows=sec("want_rows"),
            host={"tokens": tokens, "positions": positions, "seq_q_start": q_start, "seq_q_len": q_len,
                  "seq_pos0": pos0, "seq_slot": slots, "want_rows": want},
            decode_only=all(n == 1 for n in q_len))
        for name, (S_, width) in group_shapes.items():
            ctx.groups[name] = GroupView(ps, sec(f"slot_map/{name}"), sec(f"table/{name}").view(S_, width))
        for g in self.heads_per_kv:
            ctx.attention_work[g] = sec(f"work/{g}").view(-1, 2)
        return ctx

    # ------------------------------------------------------------------ the step
    def __call__(self, entries: Sequence[StepEntry]) -> Optional[torch.Tensor]:
        """Float32 logits ``[number of wanted places, vocab]`` in the order of the entries and
        of their ``want`` lists (None if nothing is wanted).  Takes the pages the new tokens
        need (raises ``OutOfPages`` before anything ran if they are not there), runs the
        model, and advances the requests' lengths."""
        cache = self.cache
        reserved: Dict[str, int] = {}
        for e in entries:
            need = cache.pages_needed(e.slot, len(e.tokens))
            for k, v in need.items():
                reserved[k] = reserved.get(k, 0) + v
        for k, v in reserved.items():
            if cache.free_pages(k) < v:
                from ..cache import OutOfPages
                raise OutOfPages(f"group {k}: the step needs {v} new pages, {cache.free_pages(k)} are free")
        for e in entries:
            cache.extend(e.slot, len(e.tokens))
        ctx = self.build_context(entries)
        logits = self.model.forward(ctx)
        for e in entries:
            cache.commit(e.slot, len(e.tokens))
        return logits
