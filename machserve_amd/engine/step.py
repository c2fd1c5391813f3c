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

from collections import OrderedDict
from dataclasses import dataclass
from typing import Dict, List, Optional, Sequence

import numpy as np
import torch

from ..cache import CacheError, CacheManager, OutOfPages
from ..parts.base import GroupView, StepContext


class StepError(ValueError):
    pass


@dataclass
class StepEntry:
    slot: int                 # the request's state slot (from CacheManager.admit)
    tokens: Sequence[int]     # its next tokens, in order
    want: Sequence[int] = ()  # indices into ``tokens`` whose logits are wanted
    # what the position encodings see for each token, one number per axis of the model's positions; None: on every
    # axis the token's index in the request (where a token lies in the cache never depends on this)
    positions: Optional[Sequence[Sequence[int]]] = None


class _DecodeGraph:
    """One captured step for fixed numbers of tokens per request, of wanted rows and fixed
    block-table widths: a static int32 buffer the host refills before every replay, and the
    logits it produces."""

    def __init__(self, graph, dev, pinned, offsets, widths, logits):
        self.graph, self.dev, self.pinned, self.offsets, self.widths, self.logits = graph, dev, pinned, offsets, widths, logits
        self.sampled = None  # int32 [2, B] when the graph also samples: tokens, bits of the logprobs
        self.copied = torch.cuda.Event()  # the last upload of `pinned` has finished

    def held_bytes(self) -> int:
        """Device memory this captured step holds for good: its buffer and its results."""
        return sum(t.numel() * t.element_size() for t in (self.dev, self.logits, self.sampled) if t is not None)


@dataclass
class LaunchedDecode:
    """A step that samples inside (a decode step, or a step of any mix) and runs on the device: the slot of
    every sampled row's request, the device tensor that will hold its samples (int32 ``[2, B]``: tokens, bits
    of the logprobs; rows beyond the slots belong to nobody), the pinned copy of it, the event after that
    copy, and the captured graph that ran it (a decode step's token section holds the sampled tokens as well)."""
    slots: List[int]
    sampled: torch.Tensor
    result: torch.Tensor
    done: object
    graph: object


class StepFunction:
    TABLE_BUCKET = 8        # captured block tables are this many pages wide, or a multiple
    MAX_GRAPHS = 256        # captured steps kept; the one unused longest goes first
    # ... and the most memory they may hold for good between them: each keeps its step buffer and its results (the
    # logits [rows, vocabulary] in 32-bit are nearly all of it, 39 MB at 64 rows of a 152k vocabulary, where the
    # caller gets logits; a step that samples inside keeps the samples only).  What a
    # captured step needs only while it runs comes from one pool that all captures share, since they run one
    # after another on one stream.  This reserve is device memory beside the weights and the page pools.
    MAX_GRAPH_BYTES = 2 << 30
    # A larger step keeps the device busy about as long as the host needs to launch it (2,048 rows of the 0.5B sizes:
    # 4.06 ms launched, 3.95 ms replayed).
    CAPTURE_MAX_ROWS = 2048
    # A capture costs 7 ms; a replayed step is about 1 ms shorter than a launched one (a decode step of the 0.5B sizes:
    # 1.03 against 2.17 ms).  A step in a shape of its own is captured only when that shape has come often (most never come
    # again); the sizes that steps are filled up to, and the decode steps' few sizes, keep coming in a server, so they are
    # captured the second time they are seen.  (256 and 1,024 requests of 64 to 640 prompt tokens and 32 to 256 new
    # ones, four arriving a step, 64 running: 1.28 -> 1.23 s and 4.50 -> 4.39 s against thresholds of 8 and 4.)
    CAPTURE_AFTER = 16        # a step other than plain decoding, in its own shape
    FILLED_CAPTURE_AFTER = 2  # ... filled up to a size that many steps share
    DECODE_CAPTURE_AFTER = 1  # a decode step

    def __init__(self, model, cache: CacheManager, rt, attention_rows_per_block: int = 64, use_graphs: bool = True):
        self.model, self.cache, self.rt = model, cache, rt
        self.rows_per_block = attention_rows_per_block
        self.heads_per_kv = model.attention_rows_per_token()
        self.position_axes = model.position_axes() if hasattr(model, "position_axes") else 1
        # A step of few tokens is bound by its launches: it is captured into a HIP graph and replayed.
        # A decode step (one token a request), and any other step of few rows, when its shape
        # (tokens per request, wanted rows, table widths) keeps coming, as it does while the same
        # requests decode, or while a long prompt is fed in small portions beside them (a capture
        # costs as much as a few dozen launched steps, so a shape must earn it).  Only for models
        # whose parts read nothing but device memory from the context.
        self.use_graphs = (use_graphs and rt.device.type == "cuda"
                           and all(getattr(b, "graph_safe", False) for b in getattr(model, "blocks", [])))
        self._graphs: "OrderedDict[tuple, _DecodeGraph]" = OrderedDict()
        self._graph_pool = None  # the memory pool that all captures share
        self._seen: Dict[tuple, int] = {}
        self._results: Dict[int, list] = {}  # pinned buffers for the samples, three per batch size, in turn
        self._launches = 0

    # ------------------------------------------------------------------ context
    def _check_entries(self, entries: Sequence[StepEntry]):
        """Validates the entries before anything is taken or run; returns their slots, token counts, flattened tokens,
        wanted rows, and the entries' own positions flattened ``[rows * axes]`` (empty if no entry brings any)."""
        if not entries:
            raise StepError("a step needs at least one entry")
        cache, vocab, limit = self.cache, self.model.vocab, self.model.spec.max_positions
        seen = set()
        slots, counts, tokens, want = [], [], [], []
        axes = self.position_axes
        explicit = [] if any(e.positions is not None for e in entries) else None
        for e in entries:
            n = len(e.tokens)
            if n == 0:
                raise StepError(f"slot {e.slot}: an entry needs at least one token")
            if e.slot in seen:
                raise StepError(f"slot {e.slot} appears twice in one step")
            seen.add(e.slot)
            try:
                base = cache.length(e.slot)
            except CacheError as err:  # not a request's slot
                raise StepError(str(err)) from err
            if base + n > limit:
                raise StepError(f"slot {e.slot}: position {base + n - 1} is beyond the model's {limit} positions")
            if explicit is not None:
                rows = e.positions if e.positions is not None else [[base + j] * axes for j in range(n)]
                if len(rows) != n or any(len(r) != axes for r in rows):
                    raise StepError(f"slot {e.slot}: positions must be {n} rows of {axes} numbers")
                for r in rows:
                    if min(r) < 0 or max(r) >= limit:
                        raise StepError(f"slot {e.slot}: position {list(r)} is outside the model's {limit} positions")
                    explicit.extend(int(v) for v in r)
            toks = [int(t) for t in e.tokens]
            if min(toks) < 0 or max(toks) >= vocab:
                bad = next(t for t in toks if not 0 <= t < vocab)
                raise StepError(f"slot {e.slot}: token {bad} is outside the vocabulary of {vocab}")
            for w in e.want:
                if not 0 <= w < n:
                    raise StepError(f"slot {e.slot}: wanted place {w} is outside its {n} tokens")
                want.append(len(tokens) + w)
            slots.append(e.slot)
            counts.append(n)
            tokens.extend(toks)
        return slots, counts, tokens, want, explicit or []

    def _take_pages(self, entries: Sequence[StepEntry]) -> None:
        """The pages the entries' tokens need, in every group: all of them or, with ``OutOfPages``, none."""
        cache = self.cache
        reserved: Dict[str, int] = {}
        for e in entries:
            for k, v in cache.pages_needed(e.slot, len(e.tokens)).items():
                reserved[k] = reserved.get(k, 0) + v
        for k, v in reserved.items():
            if cache.free_pages(k) < v:
                raise OutOfPages(f"group {k}: the step needs {v} new pages, {cache.free_pages(k)} are free")
        for e in entries:
            cache.extend(e.slot, len(e.tokens))

    def _context_from(self, dev: torch.Tensor, offsets, widths: Dict[str, int], host=None, sequential: bool = True) -> StepContext:
        """A step context over the device copy of a buffer laid out by ``CacheManager.build_step``."""
        def sec(k):
            start, size = offsets[k]
            return dev[start:start + size]
        S, T = offsets["seq_slot"][1], offsets["tokens"][1]
        ctx = StepContext(n_rows=T, n_seqs=S, tokens=sec("tokens"), positions=sec("positions").view(T, -1),
                          seq_q_start=sec("seq_q_start"), seq_q_len=sec("seq_q_len"), seq_pos0=sec("seq_pos0"),
                          seq_slot=sec("seq_slot"), want_rows=sec("want_rows"), host=host or {}, decode_only=S == T,
                          positions_sequential=sequential)
        for name, width in widths.items():
            ctx.groups[name] = GroupView(self.cache.page_size, sec(f"slot_map/{name}"), sec(f"table/{name}").view(S, width))
        for g in self.heads_per_kv:
            ctx.attention_work[g] = sec(f"work/{g}").view(-1, 2)
        return ctx

    def build_context(self, entries: Sequence[StepEntry], checked=None) -> StepContext:
        slots, counts, tokens, want, explicit = checked or self._check_entries(entries)
        try:
            host, offsets, widths = self.cache.build_step(slots, counts, tokens, want, self.heads_per_kv, self.rows_per_block,
                                                          1, 0, self.position_axes, explicit)
        except CacheError as e:
            raise StepError(str(e)) from e
        dev = torch.from_numpy(host).to(self.rt.device)  # one buffer, one copy
        lists = {k: host[offsets[k][0]:offsets[k][0] + offsets[k][1]].tolist()
                 for k in ("tokens", "positions", "seq_q_start", "seq_q_len", "seq_pos0", "seq_slot", "want_rows")}
        return self._context_from(dev, offsets, widths, lists, sequential=not explicit)

    # ------------------------------------------------------------------ captured decode steps
    @staticmethod
    def _decode_bucket(n: int) -> int:
        """Rows of the captured decode step that takes ``n`` requests: 1, 2, 4, 8, 16, 32, then multiples
        of 16 (above 32 rows the products run in tiles of 64 rows, whose stores are cheap for whole groups
        of 16 rows).  No step of 24 rows: from 17 to 31 rows the narrow projections run in the few-rows
        kernel with two row tiles, which holds one block a CU, and the 0.5B step is slower at 24 rows than
        at 32 (1.30 against 1.26 ms)."""
        if n <= 32:
            b = 1
            while b < n:
                b *= 2
            return b
        return -(-n // 16) * 16

    def _decode_shape(self, checked, sampled: bool):
        """The buffer of a decode step (every row's logits are computed), its graph's key, and the
        number of rows added.  The step is filled up to a bucket's size, so that a few graphs serve every
        batch size while requests end one by one, with rows that belong to no request: token 0 at position 0
        of the cache manager's scratch slot and scratch page, so that they change no key, value or state that
        a request owns (a mixer with state of fixed size may be captured too); their logits are dropped.  A
        decode step's time hardly depends on a few rows more."""
        slots, counts, tokens = checked[:3]
        pad = self._decode_bucket(len(slots)) - len(slots)
        try:
            built = self.cache.build_step(slots, counts, tokens, list(range(len(slots) + pad)), self.heads_per_kv,
                                          self.rows_per_block, self.TABLE_BUCKET, pad, self.position_axes)
        except CacheError as e:
            raise StepError(str(e)) from e
        return built, self._graph_key(counts + [1] * pad, len(slots) + pad, built[2], sampled), pad

    def _ready(self, key: tuple, after: int) -> bool:
        """Whether the step of this shape runs from a graph: it has one, or has come ``after`` times."""
        if key in self._graphs:
            return True
        n = self._seen.get(key, 0)
        if n >= after:
            return True
        if len(self._seen) > 4096:
            self._seen.clear()
        self._seen[key] = n + 1
        return False

    @staticmethod
    def _row_bucket(n: int) -> int:
        """Rows of the captured step that takes a step of ``n`` rows which is not plain decoding: multiples of 16 up
        to 64 rows, of 64 up to 512, of 128 up to 1,024, of 256 beyond (a step's time grows slowly with its rows while
        they are few: 1.25 ms at 16 rows of the 0.5B sizes, 1.35 at 64, 1.47 at 128, 1.52 at 256, 2.0 at 512)."""
        if n <= 64:
            return -(-n // 16) * 16
        if n <= 512:
            return -(-n // 64) * 64
        return -(-n // 128) * 128 if n <= 1024 else -(-n // 256) * 256

    def _fill_shape(self, n_seqs: int, n_rows: int, n_want: int):
        """``(rows, requests, wanted rows)`` that a step of any mix is filled up to, or None if it runs in its own
        shape: the requests to the next power of two that leaves room for one more (the rows that fill the step up
        need a request to belong to), the rows to their bucket, the wanted rows to a power of two; a step whose rows are
        a bucket's already keeps its requests.  Beyond 1,024 rows a step is filled by at most 64 rows: more would cost
        more than the launches that a replay saves (launched kernel by kernel a step takes the host some 2.4 ms, which
        the device is busy for from about 1,000 rows on; a prompt of 640 tokens: 2.44 ms launched, 2.35 replayed in 768
        rows)."""
        if self._row_bucket(n_rows) == n_rows:
            seqs, rows = n_seqs, n_rows  # the step has a shared size already (a portion of the token budget, say)
        else:
            seqs = 2
            while seqs < n_seqs + 1:
                seqs *= 2
            rows = self._row_bucket(n_rows + seqs - n_seqs)
        if rows > self.CAPTURE_MAX_ROWS or (n_rows > 1024 and rows - n_rows > 64):
            return None
        want = 0
        if n_want:
            want = 1
            while want < n_want:
                want *= 2
            want = max(n_want, min(want, rows))
        return rows, seqs, want

    @staticmethod
    def _graph_key(counts, n_want: int, widths, sampled: bool) -> tuple:
        # for given tokens per request, wanted rows and table widths the buffer's layout is always the same
        return (tuple(counts), n_want, tuple(sorted(widths.items())), sampled)

    def _run_graph(self, key: tuple, built, sampling=None, after: Optional["LaunchedDecode"] = None, fill_rows: int = 0,
                   samples_feed_tokens: bool = True, feeds=None):
        """Replays the captured step of this key on ``built`` (captures it first if it has none).  With ``sampling`` the
        graph also samples at its logits' rows; with ``samples_feed_tokens`` (a decode step: row i is sample i) the
        samples are left in the step's token section as well, where the next replay finds its input.  ``after`` is the
        launched step before this one, whose samples are this step's input: row for row if ``feeds`` is None (the same
        requests in the same order), else for the pairs ``(row of this step, index among that step's samples)`` of
        ``feeds``; the other rows' tokens are the entries' own."""
        host, offsets, widths = built
        extra: Dict[str, np.ndarray] = {}
        if sampling is not None:
            temps, top_ks, top_ps, states = sampling
            extra["sample/temperature"] = np.asarray(temps, dtype=np.float32).view(np.int32)
            extra["sample/top_p"] = np.asarray(top_ps, dtype=np.float32).view(np.int32)
            extra["sample/top_k"] = np.asarray(top_ks, dtype=np.int32)
            extra["sample/state"] = np.asarray(states, dtype=np.uint64).view(np.int32)
            # which rows take their token from the step before, and from where among its samples: at most one a request
            cap = offsets["seq_slot"][1]
            extra["feed/rows"], extra["feed/src"] = np.full(cap, -1, dtype=np.int32), np.zeros(cap, dtype=np.int32)
            for i, (row, src) in enumerate(feeds or ()):
                extra["feed/rows"][i], extra["feed/src"][i] = row, src
        dg = self._graphs.get(key)
        if dg is not None:
            self._graphs.move_to_end(key)
        if dg is None:
            offsets = dict(offsets)
            total = host.size
            for k, a in extra.items():
                offsets[k] = (total, a.size)
                total += (a.size + 3) // 4 * 4
            pinned = torch.empty(total, dtype=torch.int32, pin_memory=True)
            pinned.zero_()
            dev = torch.zeros(total, dtype=torch.int32, device=self.rt.device)
            dg = _DecodeGraph(None, dev, pinned, offsets, widths, None)
        dg.copied.synchronize()  # the host buffer is free to be refilled
        staged = dg.pinned.numpy()
        staged[:host.size] = host
        for k, a in extra.items():
            staged[dg.offsets[k][0]:dg.offsets[k][0] + a.size] = a
        start, size = dg.offsets["tokens"]
        if after is not None and feeds is None and after.graph is dg:
            # the sampling kernel of this graph's last replay left its tokens in the graph's own
            # token section: everything but that section is uploaded
            if start:
                dg.dev[:start].copy_(dg.pinned[:start], non_blocking=True)
            dg.dev[start + size:].copy_(dg.pinned[start + size:], non_blocking=True)
        else:
            dg.dev.copy_(dg.pinned, non_blocking=True)
            if after is not None and feeds is None:  # another graph ran that step (the block tables have grown a bucket)
                dg.dev[start:start + size].copy_(after.sampled[0])
        dg.copied.record()
        if after is not None and feeds:
            def part(k):
                return dg.dev[dg.offsets[k][0]:dg.offsets[k][0] + dg.offsets[k][1]]
            self.rt.ops.feed_tokens(part("tokens"), after.sampled[0], part("feed/rows"), part("feed/src"))
        if dg.graph is None:
            ctx = self._context_from(dg.dev, dg.offsets, widths)
            # Everything is loaded and compiled before the capture: one run of the step outside it.  That run and the
            # first replay both write the step's keys and values (the same ones, to the same places), but state of
            # fixed size would advance twice: it is put back in between.
            states = self.cache.device.snapshot_states() if self.cache.device is not None else None
            side = torch.cuda.Stream(device=self.rt.device)
            side.wait_stream(torch.cuda.current_stream())
            with torch.cuda.stream(side):
                self.model.forward(ctx)
            torch.cuda.current_stream().wait_stream(side)
            if states is not None:
                self.cache.device.restore_states(states)
            def sec(k):
                return dg.dev[dg.offsets[k][0]:dg.offsets[k][0] + dg.offsets[k][1]]
            graph = torch.cuda.CUDAGraph()
            if self._graph_pool is None:
                self._graph_pool = torch.cuda.graph_pool_handle()
            with torch.cuda.graph(graph, pool=self._graph_pool):
                dg.logits = self.model.forward(ctx)
                if sampling is not None:
                    dg.sampled = self.rt.ops.sample_packed(
                        dg.logits, sec("sample/temperature").view(torch.float32), sec("sample/top_k"),
                        sec("sample/top_p").view(torch.float32), sec("sample/state").view(torch.int64), True,
                        also_tokens=sec("tokens") if samples_feed_tokens else None)
            if sampling is not None:
                # Nobody reads a sampling step's logits outside it: their memory (nearly all that such a step would hold
                # for good: 78 MB at 128 sampled rows of a 152k vocabulary) goes back to the pool that the captured
                # steps share, like every other buffer a step needs only while it runs.
                dg.logits = None
            dg.graph = graph
            self._graphs[key] = dg
            while len(self._graphs) > 1 and (len(self._graphs) > self.MAX_GRAPHS or self.graph_bytes() > self.MAX_GRAPH_BYTES):
                self._graphs.popitem(last=False)
        if fill_rows and self.cache.device is not None:
            # rows that fill the step up advance the scratch slot's state of fixed size, step after step: it starts
            # from zero each time, so that it stays finite whatever the mixer does with it
            self.cache.device.zero_state(self.cache.scratch_slot)
        dg.graph.replay()
        return (dg.sampled if sampling is not None else dg.logits), dg

    def graph_bytes(self) -> int:
        """Device memory that the captured steps hold for good between them."""
        return sum(g.held_bytes() for g in self._graphs.values())

    def decode_and_sample(self, entries: Sequence[StepEntry], temperatures, top_ks, top_ps, states):
        """A decode-only step (one token per request) with sampling inside the captured graph: one
        upload, one replay, one copy back.  Returns ``(tokens, logprobs)`` as host lists, or None
        if this step cannot take that path (the caller then uses ``__call__`` and the sampler)."""
        launched = self.launch_decode(entries, temperatures, top_ks, top_ps, states)
        return None if launched is None else self.collect(launched)

    def launch_decode(self, entries: Sequence[StepEntry], temperatures, top_ks, top_ps, states,
                      after: Optional["LaunchedDecode"] = None, feeds=None) -> Optional["LaunchedDecode"]:
        """The same step, launched and not waited for.  With ``after`` - the launched step before
        this one - the tokens are that step's samples, taken on the device: the host need not have seen
        them.  Without ``feeds`` that step held the same requests in the same order; with ``feeds``, pairs of
        (entry of this step, index among that step's samples), only the listed entries take their token
        from it and the others bring their own.  None if the step cannot take this
        path or its shape has not come often enough to be captured; ``OutOfPages`` before anything
        ran if the pages are not there."""
        if not (self.use_graphs and self.model.observer is None
                and all(len(e.tokens) == 1 and e.positions is None for e in entries)
                and len({e.slot for e in entries}) == len(entries)):
            return None
        slots = [e.slot for e in entries]
        if after is not None and feeds is None and after.slots != slots:
            raise StepError("a step fed from the device must hold the requests of the step before, in the same order")
        cache = self.cache
        checked = self._check_entries(entries)
        self._take_pages(entries)
        built, key, pad = self._decode_shape(checked, True)
        if not self._ready(key, self.DECODE_CAPTURE_AFTER):
            return None  # the pages stay with the requests; the caller runs the step as it is
        # the rows that fill the step up are rows of the scratch slot: they sample greedily (their token is some
        # token of the vocabulary, which is all that the next step's embedding needs of it) and are dropped
        filled = [list(v) + [fill] * pad for v, fill in ((temperatures, 0.0), (top_ks, 0), (top_ps, 1.0), (states, 0))]
        sampled, graph = self._run_graph(key, built, tuple(filled), after, fill_rows=pad, feeds=feeds)
        for e in entries:
            cache.commit(e.slot, 1)
        return self._launched(slots, sampled, graph)

    def _launched(self, slots: List[int], sampled: torch.Tensor, graph) -> "LaunchedDecode":
        """The samples of a step that was just replayed go to a pinned buffer of their own (the graph's is overwritten
        by its next replay), behind the step on its stream; nothing is waited for."""
        rows = sampled.shape[1]
        ring = self._results.get(rows)
        if ring is None:
            ring = self._results[rows] = [torch.empty((2, rows), dtype=torch.int32, pin_memory=True) for _ in range(3)]
        result = ring[self._launches % 3]  # at most two steps are in flight: a buffer is read before its next turn
        self._launches += 1
        result.copy_(sampled, non_blocking=True)
        done = torch.cuda.Event()
        done.record()
        return LaunchedDecode(slots, sampled, result, done, graph)

    def collect(self, launched: "LaunchedDecode"):
        """``(tokens, logprobs)`` of a launched step as host lists; waits for them."""
        launched.done.synchronize()
        n = len(launched.slots)  # rows beyond belong to no request
        return launched.result[0, :n].tolist(), launched.result[1, :n].view(torch.float32).tolist()

    def step_and_sample(self, entries: Sequence[StepEntry], temperatures, top_ks, top_ps, states, capture_now: bool = False):
        """A step of any mix (portions of prompts, alone or beside decoded tokens) whose wanted rows are sampled inside
        the captured step: ``temperatures`` ... ``states`` hold one value for every wanted row, in the order of the
        entries.  Returns ``(tokens, logprobs)`` as host lists in that order: one small copy brings them, where the
        logits' way is three uploads, two launches and two copies behind the step (0.1 ms: 7 % of a short prompt's
        first token).  None, before anything is taken or run, if the step cannot take this path: it is plain decoding
        (``decode_and_sample``), it is not filled up to a shared size, or that size has not come often enough to be
        captured (the caller then runs it through ``__call__`` with ``eager`` and samples from the logits)."""
        launched = self.launch_step(entries, temperatures, top_ks, top_ps, states, capture_now=capture_now)
        return None if launched is None else self.collect(launched)

    def launch_step(self, entries: Sequence[StepEntry], temperatures, top_ks, top_ps, states, after: Optional["LaunchedDecode"] = None,
                    feeds=None, capture_now: bool = False) -> Optional["LaunchedDecode"]:
        """``step_and_sample``, launched and not waited for (``collect`` brings the samples).  With ``after``, the
        launched step before this one, and ``feeds``, pairs of (entry of this step, index among that step's
        samples), the first token of the listed entries is that sample, taken on the device; such an entry has one
        token, whose value here is a placeholder."""
        if not (self.use_graphs and self.model.observer is None and all(e.positions is None for e in entries)):
            return None
        if all(len(e.tokens) == 1 for e in entries) and len({e.slot for e in entries}) == len(entries):
            return None
        cache = self.cache
        checked = self._check_entries(entries)
        slots, counts, tokens, want, _ = checked
        if not want or len(want) != len(temperatures):
            return None
        fill = self._fill_shape(len(slots), len(tokens), len(want))
        if fill is None:
            return None
        pages = max(-(-(cache.length(sl) + n) // cache.page_size) for sl, n in zip(slots, counts))
        width = self.TABLE_BUCKET
        while width < pages:
            width *= 2
        # the graph's key holds every group's table width, which only the built step knows: how often the size has
        # come is counted under the width asked for
        seen_as = ("filled, sampled",) + fill + (width,)
        if not self._ready(seen_as, 0 if capture_now else self.FILLED_CAPTURE_AFTER):
            return None
        self._seen[seen_as] = max(self._seen.get(seen_as, 0), self.FILLED_CAPTURE_AFTER)  # it runs from a graph from now on
        self._take_pages(entries)
        try:
            built = cache.build_step(slots, counts, tokens, want, self.heads_per_kv, self.rows_per_block, width, 0,
                                     self.position_axes, (), fill)
        except CacheError as e:
            raise StepError(str(e)) from e
        key = seen_as + tuple(sorted(built[2].items()))
        # the rows that fill the wanted rows up sample greedily and are dropped
        pad = fill[2] - len(want)
        sampling = tuple(list(v) + [f] * pad for v, f in ((temperatures, 0.0), (top_ks, 0), (top_ps, 1.0), (states, 0)))
        row_feeds = None
        if after is not None and feeds:
            first_row, at = [], 0
            for n in counts:
                first_row.append(at)
                at += n
            if any(counts[e] != 1 for e, _ in feeds):
                raise StepError("an entry fed from the device brings one token")
            row_feeds = [(first_row[e], src) for e, src in feeds]
        sampled, graph = self._run_graph(key, built, sampling, after if row_feeds else None, fill_rows=fill[0] - len(tokens),
                                         samples_feed_tokens=False, feeds=row_feeds)
        for e in entries:
            cache.commit(e.slot, len(e.tokens))
        return self._launched([e.slot for e in entries for _ in e.want], sampled, graph)

    # ------------------------------------------------------------------ the step
    def __call__(self, entries: Sequence[StepEntry], borrow_logits: bool = False, capture_now: bool = False,
                 eager: bool = False) -> Optional[torch.Tensor]:
        """Float32 logits ``[number of wanted places, vocab]`` in the order of the entries and
        of their ``want`` lists (None if nothing is wanted).  Takes the pages the new tokens
        need (raises ``OutOfPages`` before anything ran if they are not there), runs the
        model, and advances the requests' lengths.  With ``borrow_logits`` the result may be a
        buffer that the next step overwrites (the engine samples from it at once); with
        ``capture_now`` a step that may run from a captured graph is captured at once, not
        when its shape has come a few times; with ``eager`` it is launched kernel by kernel whatever its shape
        (a step that ``step_and_sample`` has declined: its shape is counted there)."""
        cache = self.cache
        checked = self._check_entries(entries)  # a step that is refused has taken nothing
        self._take_pages(entries)
        # a captured step takes positions from the cache, and shows no layer's stream to an observer
        graphs = self.use_graphs and not eager and self.model.observer is None and all(e.positions is None for e in entries)
        if graphs and all(len(e.tokens) == 1 for e in entries) and len({e.slot for e in entries}) == len(entries):
            built, key, pad = self._decode_shape(checked, False)
            if self._ready(key, self.DECODE_CAPTURE_AFTER):
                logits, _ = self._run_graph(key, built, fill_rows=pad)
            else:
                host, offsets, widths = built
                logits = self.model.forward(self._context_from(torch.from_numpy(host).to(self.rt.device), offsets, widths))
                borrow_logits = True  # a fresh tensor: nothing overwrites it
            if pad:
                logits = logits[:len(entries)]
            wanted = [i for i, e in enumerate(entries) if len(e.want)]
            if not wanted:
                logits = None
            elif len(wanted) != len(entries):
                logits = logits[torch.tensor(wanted, device=logits.device)]
            elif not borrow_logits:
                logits = logits.clone()  # the graph's own buffer is overwritten by its next replay
        elif graphs:
            slots, counts, tokens, want, _ = checked
            # block tables as wide as the next power of two of pages: a prompt that grows by a
            # portion a step keeps its shape for many steps
            pages = max(-(-(cache.length(sl) + n) // cache.page_size) for sl, n in zip(slots, counts))
            width = self.TABLE_BUCKET
            while width < pages:
                width *= 2
            # filled up to a size that many steps share (rows, requests, wanted rows), so that one captured graph
            # serves every step of that size; a step that would have to be filled too far runs in its own shape
            fill = self._fill_shape(len(slots), len(tokens), len(want))
            try:
                built = cache.build_step(slots, counts, tokens, want, self.heads_per_kv, self.rows_per_block, width, 0,
                                         self.position_axes, (), fill)
            except CacheError as e:
                raise StepError(str(e)) from e
            if fill is not None:
                key = ("filled",) + fill + tuple(sorted(built[2].items()))
                after = 0 if capture_now else self.FILLED_CAPTURE_AFTER
            else:
                key = self._graph_key(counts, len(want), built[2], False)
                after = 0 if capture_now else self.CAPTURE_AFTER
            if (fill is not None or len(tokens) <= self.CAPTURE_MAX_ROWS) and self._ready(key, after):
                logits, _ = self._run_graph(key, built, fill_rows=0 if fill is None else fill[0] - len(tokens))
                if logits is not None:
                    if fill is not None:
                        logits = logits[:len(want)] if want else None  # rows beyond belong to nobody
                    if logits is not None and not borrow_logits:
                        logits = logits.clone()
            else:  # most shapes never come again: they run as they are
                host, offsets, widths = built
                logits = self.model.forward(self._context_from(torch.from_numpy(host).to(self.rt.device), offsets, widths))
                if fill is not None and logits is not None:
                    logits = logits[:len(want)] if want else None
        else:
            logits = self.model.forward(self.build_context(entries, checked))
        for e in entries:
            cache.commit(e.slot, len(e.tokens))
        return logits
