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

from collections import deque
from dataclasses import dataclass, field
from typing import Deque, Dict, List, Optional, Sequence

from ..cache import CacheManager
from ..sampling.params import SamplingParams


class SchedulerError(ValueError):
    pass


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

    @property
    def generated(self) -> List[int]:
        return self.tokens[len(self.prompt):]

    @property
    def decoding(self) -> bool:
        return self.fed == len(self.tokens) - 1 and len(self.tokens) > len(self.prompt)


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

    @property
    def n_tokens(self) -> int:
        return sum(i.count for i in self.items)


class Scheduler:
    def __init__(self, cache: CacheManager, max_batch_tokens: int = 512, chunk_size: Optional[int] = None,
                 max_running: Optional[int] = None, max_positions: Optional[int] = None):
        if max_batch_tokens < 1:
            raise SchedulerError("max_batch_tokens must be at least 1")
        self.cache = cache
        self.max_batch_tokens = max_batch_tokens
        self.chunk_size = chunk_size or max_batch_tokens
        self.max_running = min(max_running or cache.max_requests, cache.max_requests)
        self.max_positions = max_positions
        self.waiting: Deque[Request] = deque()
        self.running: List[Request] = []  # oldest first
        self.finished: Dict[int, Request] = {}
        self._next_id = 1

    # ------------------------------------------------------------------ admission
    def add(self, prompt: Sequence[int], max_new: int, params: Optional[SamplingParams] = None,
            eos: Optional[int] = None, stop_seqs: Sequence[Sequence[int]] = ()) -> int:
        """Queue a request; returns its id.  Refusals follow ``continuous.rs:788-800``: empty
        prompt, prompt beyond the model's positions; and, ours, a request the pool could
        never hold."""
        prompt = [int(t) for t in prompt]
        if not prompt:
            raise SchedulerError("empty prompt")
        if max_new < 1:
            raise SchedulerError(f"max_new {max_new} must be at least 1")
        if self.max_positions is not None and len(prompt) >= self.max_positions:
            raise SchedulerError(f"prompt of {len(prompt)} tokens leaves no room within {self.max_positions} positions")
        total = len(prompt) + max_new - 1  # the last generated token is never fed
        if self.max_positions is not None:
            total = min(total, self.max_positions)
        ps = self.cache.page_size
        for name, g in self.cache.groups.items():
            if -(-total // ps) > g.pool.num_pages:
                raise SchedulerError(f"request of up to {total} cached tokens needs {-(-total // ps)} pages; "
                                     f"group {name} has {g.pool.num_pages}")
        params = params or SamplingParams()
        params.validate()
        rid = self._next_id
        self._next_id += 1
        seed = params.seed if params.seed != 0 else rid  # continuous.rs:803
        req = Request(rid, prompt, max_new, params, eos, [list(s) for s in stop_seqs if len(s)],
                      tokens=list(prompt), rng_state=seed & ((1 << 64) - 1))
        self.waiting.append(req)
        return rid

    def cancel(self, rid: int) -> bool:
        for r in list(self.waiting):
            if r.id == rid:
                self.waiting.remove(r)
                self._finish(r, "cancelled")
                return True
        for r in self.running:
            if r.id == rid:
                self._finish(r, "cancelled")
                return True
        return False

    def has_work(self) -> bool:
        return bool(self.waiting or self.running)

    # ------------------------------------------------------------------ planning
    def _preempt_youngest(self, plan: StepPlan) -> Request:
        victim = self.running.pop()
        self.cache.release(victim.slot)
        victim.slot, victim.fed = None, 0
        victim.preemptions += 1
        self.waiting.appendleft(victim)
        plan.preempted.append(victim)
        plan.items = [i for i in plan.items if i.request is not victim]
        return victim

    def _reserved(self, plan: StepPlan) -> Dict[str, int]:
        res: Dict[str, int] = {}
        for it in plan.items:
            for k, v in self.cache.pages_needed(it.request.slot, it.count).items():
                res[k] = res.get(k, 0) + v
        return res

    def schedule(self) -> StepPlan:
        """The next step: every decoding request's token first, then prompt portions of running
        requests, then newly admitted requests, under the token budget and the free pages."""
        plan = StepPlan()
        while True:
            plan.items = []
            budget = self.max_batch_tokens
            # 1. decoded tokens, oldest request first; they must all fit, or the youngest goes
            decoders = [r for r in self.running if r.decoding]
            need: Dict[str, int] = {}
            for r in decoders:
                for k, v in self.cache.pages_needed(r.slot, 1).items():
                    need[k] = need.get(k, 0) + v
            if any(self.cache.free_pages(k) < v for k, v in need.items()):
                self._preempt_youngest(plan)
                continue
            for r in decoders:
                if budget == 0:
                    break
                plan.items.append(PlanItem(r, r.fed, 1, True))
                budget -= 1
            # 2. portions of prompts (or of a recomputation) already running, oldest first; an
            #    older request that lacks pages takes them from the youngest
            restart = False
            for r in self.running:
                if r.decoding or budget == 0:
                    continue
                n = min(len(r.tokens) - r.fed, self.chunk_size, budget)
                if not self.cache.can_extend(r.slot, n, self._reserved(plan)):
                    if r is not self.running[-1]:
                        self._preempt_youngest(plan)
                        restart = True
                        break
                    continue
                plan.items.append(PlanItem(r, r.fed, n, r.fed + n == len(r.tokens)))
                budget -= n
            if restart:
                continue
            # 3. admission, first come first served
            while self.waiting and budget > 0 and len(self.running) < self.max_running \
                    and self.cache.slots.available() > 0:
                r = self.waiting[0]
                if r in plan.preempted:  # it lost its pages in this very step
                    break
                n = min(len(r.tokens), self.chunk_size, budget)
                res = self._reserved(plan)
                ps = self.cache.page_size
                if any(self.cache.free_pages(k) - res.get(k, 0) < -(-n // ps) for k in self.cache.groups):
                    break
                self.waiting.popleft()
                r.slot = self.cache.admit()
                r.fed = 0
                self.running.append(r)
                plan.admitted.append(r)
                plan.items.append(PlanItem(r, 0, n, n == len(r.tokens)))
                budget -= n
            if plan.items or not self.running:
                return plan
            # running requests exist but none can move: they hold each other's pages
            self._preempt_youngest(plan)

    # ------------------------------------------------------------------ after the step
    def _finish(self, r: Request, reason: str) -> None:
        r.finish_reason = reason
        if r in self.running:
            self.running.remove(r)
        if r.slot is not None:
            self.cache.release(r.slot)
            r.slot = None
        self.finished[r.id] = r

    def update(self, plan: StepPlan, sampled: Sequence[int], logprobs: Optional[Sequence[float]] = None,
               new_states: Optional[Sequence[int]] = None):
        """The step ran: ``sampled[i]`` is the token of the i-th item with ``sample`` set.
        Returns the list of (request id, token) emitted and the requests that finished."""
        emitted, done = [], []
        k = 0
        for it in plan.items:
            r = it.request
            r.fed += it.count
            if not it.sample:
                continue
            tok = int(sampled[k])
            if logprobs is not None:
                r.logprobs.append(float(logprobs[k]))
            if new_states is not None:
                r.rng_state = new_states[k]
            k += 1
            r.tokens.append(tok)
            emitted.append((r.id, tok))
            gen = r.generated
            reason = None
            if r.eos is not None and tok == r.eos:
                reason = "stop"
            elif any(len(gen) >= len(s) and gen[-len(s):] == list(s) for s in r.stop_seqs):
                reason = "stop"
            elif len(gen) >= r.max_new:
                reason = "length"
            elif self.max_positions is not None and len(r.tokens) > self.max_positions:
                reason = "length"
            if reason:
                self._finish(r, reason)
                done.append(r)
        return emitted, done
