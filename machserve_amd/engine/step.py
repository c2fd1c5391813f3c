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


class _DecodeGraph:
    """One captured decode step for a fixed number of requests and fixed block-table widths:
    a static int32 buffer the host refills before every replay, and the logits it produces."""

    def __init__(self, graph, dev, pinned, offsets, sizes, logits):
        self.graph, self.dev, self.pinned, self.offsets, self.sizes, self.logits = graph, dev, pinned, offsets, sizes, logits
        self.sampled = None  # int32 [2, B] when the graph also samples: tokens, bits of the logprobs
        self.copied = torch.cuda.Event()  # the last upload of `pinned` has finished


class StepFunction:
    TABLE_BUCKET = 8  # captured block tables are this many pages wide, or a multiple

    def __init__(self, model, cache: CacheManager, rt, attention_rows_per_block: int = 64, use_graphs: bool = True):
        self.model, self.cache, self.rt = model, cache, rt
        self.rows_per_block = attention_rows_per_block
        self.heads_per_kv = model.attention_rows_per_token()
        # a decode step is launch-bound; it is captured once per batch size into a HIP graph and
        # replayed.  Only for models whose parts read nothing but device memory from the context.
        self.use_graphs = (use_graphs and rt.device.type == "cuda"
                           and all(getattr(b.mixer, "graph_safe", False) for b in getattr(model, "blocks", [])))
        self._graphs: Dict[tuple, _DecodeGraph] = {}

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

    # ------------------------------------------------------------------ captured decode steps
    def _decode_sections(self, slots: List[int], tokens: List[int], widths: Dict[str, int]) -> Dict[str, np.ndarray]:
        """The int32 sections of a step in which every request has one row, block tables padded
        to ``widths``.  The order of the keys is the layout of the captured buffer."""
        cache, ps = self.cache, self.cache.page_size
        B = len(slots)
        pos = np.fromiter((cache.lengths[s] for s in slots), dtype=np.int32, count=B)
        ar = np.arange(B, dtype=np.int32)
        sec: Dict[str, np.ndarray] = {
            "tokens": np.asarray(tokens, dtype=np.int32), "positions": pos, "seq_q_start": ar,
            "seq_q_len": np.ones(B, dtype=np.int32), "seq_pos0": pos, "seq_slot": np.asarray(slots, dtype=np.int32),
            "want_rows": ar,
        }
        for name, width in widths.items():
            table = np.full((B, width), -1, dtype=np.int32)
            slot_map = np.empty(B, dtype=np.int32)
            for i, s in enumerate(slots):
                t = cache.table(name, s)
                table[i, :len(t)] = t
                slot_map[i] = t[pos[i] // ps] * ps + pos[i] % ps
            sec[f"table/{name}"] = table.reshape(-1)
            sec[f"slot_map/{name}"] = slot_map
        for g in self.heads_per_kv:
            sec[f"work/{g}"] = np.stack([ar, np.zeros(B, dtype=np.int32)], 1).reshape(-1)
        return sec

    def _context_from(self, dev: torch.Tensor, offsets, sizes, B: int, widths: Dict[str, int]) -> StepContext:
        def sec(k):
            return dev[offsets[k]:offsets[k] + sizes[k]]
        ctx = StepContext(n_rows=B, n_seqs=B, tokens=sec("tokens"), positions=sec("positions"),
                          seq_q_start=sec("seq_q_start"), seq_q_len=sec("seq_q_len"), seq_pos0=sec("seq_pos0"),
                          seq_slot=sec("seq_slot"), want_rows=sec("want_rows"), decode_only=True)
        for name, width in widths.items():
            ctx.groups[name] = GroupView(self.cache.page_size, sec(f"slot_map/{name}"), sec(f"table/{name}").view(B, width))
        for g in self.heads_per_kv:
            ctx.attention_work[g] = sec(f"work/{g}").view(-1, 2)
        return ctx

    def _run_decode_graph(self, entries: Sequence[StepEntry], sampling=None):
        """Replay (or first capture) the graph of this batch size.  ``sampling`` = (temperatures,
        top_ks, top_ps, states) makes sampling part of the graph; the result is then the int32
        ``[2, B]`` tensor of :meth:`HipOps.sample_packed`, else the logits."""
        cache = self.cache
        slots = [e.slot for e in entries]
        tokens = [int(e.tokens[0]) for e in entries]
        vocab = self.model.vocab
        for s, t in zip(slots, tokens):
            if not 0 <= t < vocab:
                raise StepError(f"slot {s}: token {t} is outside the vocabulary of {vocab}")
            if cache.lengths[s] + 1 > self.model.spec.max_positions:
                raise StepError(f"slot {s}: position {cache.lengths[s]} is beyond the model's positions")
        B = len(slots)
        bucket = self.TABLE_BUCKET
        widths = {name: -(-max(len(cache.table(name, s)) for s in slots) // bucket) * bucket for name in cache.groups}
        key = (B, tuple(sorted(widths.items())), sampling is not None)
        sections = self._decode_sections(slots, tokens, widths)
        if sampling is not None:
            temps, top_ks, top_ps, states = sampling
            sections["sample/temperature"] = np.asarray(temps, dtype=np.float32).view(np.int32)
            sections["sample/top_p"] = np.asarray(top_ps, dtype=np.float32).view(np.int32)
            sections["sample/top_k"] = np.asarray(top_ks, dtype=np.int32)
            sections["sample/state"] = np.asarray(states, dtype=np.uint64).view(np.int32)
        dg = self._graphs.get(key)
        if dg is None:
            offsets, sizes, total = {}, {}, 0
            for k, a in sections.items():
                offsets[k], sizes[k] = total, a.size
                total += (a.size + 3) // 4 * 4
            pinned = torch.empty(total, dtype=torch.int32, pin_memory=True)
            pinned.zero_()
            dev = torch.zeros(total, dtype=torch.int32, device=self.rt.device)
            dg = _DecodeGraph(None, dev, pinned, offsets, sizes, None)
        dg.copied.synchronize()  # the host buffer is free to be refilled
        host = dg.pinned.numpy()
        for k, a in sections.items():
            host[dg.offsets[k]:dg.offsets[k] + a.size] = a
        dg.dev.copy_(dg.pinned, non_blocking=True)
        dg.copied.record()
        if dg.graph is None:
            ctx = self._context_from(dg.dev, dg.offsets, dg.sizes, B, widths)
            side = torch.cuda.Stream(device=self.rt.device)
            side.wait_stream(torch.cuda.current_stream())
            with torch.cuda.stream(side):
                self.model.forward(ctx)  # everything is loaded and compiled before the capture
            torch.cuda.current_stream().wait_stream(side)
            def sec(k):
                return dg.dev[dg.offsets[k]:dg.offsets[k] + dg.sizes[k]]
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph):
                dg.logits = self.model.forward(ctx)
                if sampling is not None:
                    dg.sampled = self.rt.ops.sample_packed(
                        dg.logits, sec("sample/temperature").view(torch.float32), sec("sample/top_k"),
                        sec("sample/top_p").view(torch.float32), sec("sample/state").view(torch.int64), True)
            dg.graph = graph
            self._graphs[key] = dg
        dg.graph.replay()
        return dg.sampled if sampling is not None else dg.logits

    def decode_and_sample(self, entries: Sequence[StepEntry], temperatures, top_ks, top_ps, states):
        """A decode-only step (one token per request) with sampling inside the captured graph: one
        upload, one replay, one copy back.  Returns ``(tokens, logprobs)`` as host lists, or None
        if this step cannot take that path (the caller then uses ``__call__`` and the sampler)."""
        if not (self.use_graphs and all(len(e.tokens) == 1 for e in entries)
                and len({e.slot for e in entries}) == len(entries)):
            return None
        cache = self.cache
        reserved: Dict[str, int] = {}
        for e in entries:
            for k, v in cache.pages_needed(e.slot, 1).items():
                reserved[k] = reserved.get(k, 0) + v
        for k, v in reserved.items():
            if cache.free_pages(k) < v:
                from ..cache import OutOfPages
                raise OutOfPages(f"group {k}: the step needs {v} new pages, {cache.free_pages(k)} are free")
        for e in entries:
            cache.extend(e.slot, 1)
        both = self._run_decode_graph(entries, (temperatures, top_ks, top_ps, states)).cpu()  # the step's one sync
        for e in entries:
            cache.commit(e.slot, 1)
        return both[0].tolist(), both[1].view(torch.float32).tolist()

    # ------------------------------------------------------------------ the step
    def __call__(self, entries: Sequence[StepEntry], borrow_logits: bool = False) -> Optional[torch.Tensor]:
        """Float32 logits ``[number of wanted places, vocab]`` in the order of the entries and
        of their ``want`` lists (None if nothing is wanted).  Takes the pages the new tokens
        need (raises ``OutOfPages`` before anything ran if they are not there), runs the
        model, and advances the requests' lengths.  With ``borrow_logits`` the result may be a
        buffer that the next step overwrites (the engine samples from it at once)."""
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
        if self.use_graphs and all(len(e.tokens) == 1 for e in entries) and len({e.slot for e in entries}) == len(entries):
            logits = self._run_decode_graph(entries)
            wanted = [i for i, e in enumerate(entries) if len(e.want)]
            if not wanted:
                logits = None
            elif len(wanted) != len(entries):
                logits = logits[torch.tensor(wanted, device=logits.device)]
            elif not borrow_logits:
                logits = logits.clone()  # the graph's own buffer is overwritten by its next replay
        else:
            logits = self.model.forward(self.build_context(entries))
        for e in entries:
            cache.commit(e.slot, len(e.tokens))
        return logits
