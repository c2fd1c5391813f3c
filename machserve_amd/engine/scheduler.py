"""The scheduler: admits requests, cuts prompts into portions under a token budget,
decodes, finishes and frees.  Host logic only; it decides, the engine runs.

Compared with the reference (``crates/mach-model/src/continuous.rs:753-929, 943-1201,
1294-1405``): the reference reserves every page of a request at admission and rejects a new
request when the pool is exhausted; it never takes pages from a running request.  Here
pages are taken step by step, so the pool can run dry in the middle of a step.  The
decision then is: **the youngest running request is preempted** - its pages and slot go
back, it keeps its prompt and what it has generated, and it returns to the *front* of the
waiting queue to be recomputed - until the decoded tokens of the older requests fit.  A
request whose prompt and ``max_new`` could never fit the pool alone is refused at
``add``.  Because the sampler's state advances once per sampled token and is kept with the
request, a preempted request continues with the same tokens it would have produced.

One rule serves prompts, decoding and recomputation: a request holds ``tokens`` (prompt
plus generated) and ``fed`` (how many of them are in the cache); a step feeds
``tokens[fed : fed + n]``, and when that reaches the end, the last row is sampled and the
new token appended.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Dict, List, Optional, Sequence

from ..cache import CacheManager
from ..kernels.build import ensure_host_module
from ..sampling.params import SamplingParams

_host = ensure_host_module()
SchedulerError = _host.SchedulerError  # a ValueError


@dataclass
class Request:
    id: int
    prompt: List[int]
    max_new: int
    params: SamplingParams
    eos: Optional[int] = None
    stop_seqs: Sequence[Sequence[int]] = ()
    # progress
    tokens: List[int] = field(default_factory=list)  # prompt + generated
    fed: int = 0
    slot: Optional[int] = None
    rng_state: int = 0
    logprobs: List[float] = field(default_factory=list)
    top_logprobs: List[list] = field(default_factory=list)  # per generated token: [(token, logprob), ...]
    finish_reason: Optional[str] = None
    preemptions: int = 0
    pending: int = 0                  # tokens sampled on the device that the host has not seen yet
    closing: Optional[str] = None     # it has left the queues for this reason; finished once its tokens are in

    @property
    def generated(self) -> List[int]:
        return self.tokens[len(self.prompt):]

    @property
    def decoding(self) -> bool:
        n = len(self.tokens) + self.pending
        return self.fed == n - 1 and n > len(self.prompt)


@dataclass
class PlanItem:
    request: Request
    start: int    # first token of the portion, index into request.tokens
    count: int
    sample: bool  # the portion reaches the end of tokens: its last row is sampled


@dataclass
class StepPlan:
    items: List[PlanItem] = field(default_factory=list)
    preempted: List[Request] = field(default_factory=list)
    admitted: List[Request] = field(default_factory=list)
    native: list = field(default_factory=list)  # the core's own items, handed back to it after the step

    @property
    def n_tokens(self) -> int:
        return sum(i.count for i in self.items)


class Scheduler:
    """Queues and decisions live in the native ``SchedulerCore`` (``csrc/host/scheduler.hpp``); this
    class keeps the requests' tokens, sampling options and results, and mirrors ``fed``, ``slot``
    and ``preemptions`` from the core's plans."""

    def __init__(self, cache: CacheManager, max_batch_tokens: int = 512, chunk_size: Optional[int] = None,
                 max_running: Optional[int] = None, max_positions: Optional[int] = None):
        self.cache = cache
        self.core = _host.SchedulerCore(cache.core, max_batch_tokens, chunk_size or 0, max_running or 0, max_positions or 0)
        self.max_batch_tokens = self.core.max_batch_tokens
        self.chunk_size = self.core.chunk_size
        self.max_running = self.core.max_running
        self.max_positions = max_positions
        self.requests: Dict[int, Request] = {}  # waiting or running
        self.finished: Dict[int, Request] = {}
        self._next_id = 1

    @property
    def waiting(self) -> List[Request]:
        return [self.requests[i] for i in self.core.waiting()]

    @property
    def running(self) -> List[Request]:
        """Oldest first."""
        return [self.requests[i] for i in self.core.running()]

    # ------------------------------------------------------------------ admission
    def add(self, prompt: Sequence[int], max_new: int, params: Optional[SamplingParams] = None,
            eos: Optional[int] = None, stop_seqs: Sequence[Sequence[int]] = ()) -> int:
        """Queue a request; returns its id.  Refused: an empty prompt, a prompt beyond the model's
        positions (``continuous.rs:788-800``), and a request the pool could never hold."""
        prompt = [int(t) for t in prompt]
        params = params or SamplingParams()
        params.validate()
        rid = self._next_id
        self.core.add(rid, len(prompt), max_new)
        self._next_id += 1
        seed = params.seed if params.seed != 0 else rid  # continuous.rs:803
        req = Request(rid, prompt, max_new, params, eos, [list(s) for s in stop_seqs if len(s)],
                      tokens=list(prompt), rng_state=seed & ((1 << 64) - 1))
        self.requests[rid] = req
        return rid

    def cancel(self, rid: int) -> bool:
        r = self.requests.get(rid)
        if r is None:
            return False
        self._finish(r, "cancelled")
        return True

    def has_work(self) -> bool:
        return self.core.has_work()

    # ------------------------------------------------------------------ planning
    def schedule(self) -> StepPlan:
        """The next step: every decoding request's token first, then prompt portions of running
        requests, then newly admitted requests, under the token budget and the free pages."""
        native = self.core.schedule()
        plan = StepPlan(native=native.items)
        for rid in native.preempted:
            r = self.requests[rid]
            r.slot, r.fed = None, 0
            r.preemptions += 1
            plan.preempted.append(r)
        for rid, slot in native.admitted:
            r = self.requests[rid]
            r.slot, r.fed = slot, 0
            self.cache.on_admitted(slot)
            plan.admitted.append(r)
        plan.items = [PlanItem(self.requests[i.id], i.start, i.count, i.sample) for i in native.items]
        return plan

    # ------------------------------------------------------------------ after the step
    def _close(self, r: Request, reason: str) -> None:
        """The request leaves the queues: its pages and slot go back now (work already launched on them
        runs before anything that is launched later).  It is finished once its last token is in."""
        if r.closing is None:
            r.closing = reason
            self.core.finish(r.id)
            r.slot = None
            del self.requests[r.id]

    def _finish(self, r: Request, reason: str) -> None:
        self._close(r, reason)
        r.finish_reason = r.closing
        self.finished[r.id] = r

    def begin(self, plan: StepPlan) -> None:
        """The step has been launched: its tokens are in the cache, a sampled row will yield one
        token more.  What follows from counts alone is decided here, before the tokens are known:
        a request whose next token is its last leaves the queues."""
        self.core.advance(plan.native)
        for it in plan.items:
            r = it.request
            r.fed += it.count
            if not it.sample:
                continue
            r.pending += 1
            n = len(r.tokens) + r.pending
            if n - len(r.prompt) >= r.max_new or (self.max_positions is not None and n > self.max_positions):
                self._close(r, "length")

    def complete(self, plan: StepPlan, sampled: Sequence[int], logprobs: Optional[Sequence[float]] = None,
                 new_states: Optional[Sequence[int]] = None):
        """The sampled tokens of a launched step have arrived: ``sampled[i]`` is the token of the i-th
        item with ``sample`` set.  Returns the (request id, token) pairs emitted and the requests that
        finished.  A token that arrives for a request already stopped (its end was only seen after
        the next step had been launched) is dropped."""
        emitted, done = [], []
        k = 0
        for it in plan.items:
            if not it.sample:
                continue
            r = it.request
            tok = int(sampled[k])
            lp = float(logprobs[k]) if logprobs is not None else None
            if new_states is not None:
                r.rng_state = new_states[k]
            k += 1
            r.pending -= 1
            if r.finish_reason is not None:
                continue
            r.tokens.append(tok)
            if lp is not None:
                r.logprobs.append(lp)
            emitted.append((r.id, tok))
            n_gen = len(r.tokens) - len(r.prompt)
            if r.eos is not None and tok == r.eos:
                r.closing = None if r.closing == "length" else r.closing  # the token itself decides
                self._stop(r)
            elif any(n_gen >= len(s) and r.tokens[-len(s):] == s for s in r.stop_seqs):
                r.closing = None if r.closing == "length" else r.closing
                self._stop(r)
            if r.closing is not None and (r.closing == "stop" or r.pending == 0):
                r.finish_reason = r.closing
                self.finished[r.id] = r
                done.append(r)
        return emitted, done

    def _stop(self, r: Request) -> None:
        if r.id in self.requests:
            self._close(r, "stop")
        else:
            r.closing = "stop"  # it had left the queues for its length already

    def update(self, plan: StepPlan, sampled: Sequence[int], logprobs: Optional[Sequence[float]] = None,
               new_states: Optional[Sequence[int]] = None):
        """``begin`` and ``complete`` at once, for a step whose tokens are known when it returns."""
        self.begin(plan)
        return self.complete(plan, sampled, logprobs, new_states)
