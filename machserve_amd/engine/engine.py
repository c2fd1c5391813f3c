"""The engine: scheduler above, step function and sampler below.

``add`` queues a request, ``step`` runs one scheduled batch and returns the tokens it
produced, ``step_pipelined`` does the same but launches a decode step before the tokens of
the step before it have reached the host (``run`` and ``generate`` use it), ``cancel`` ends a
request, ``generate`` runs a list of prompts to the end.  Role of ``ContinuousModel`` in the
reference (``crates/mach-model/src/continuous.rs:715, 943, 1294``)."""
from __future__ import annotations

import gc
from typing import Dict, List, Optional, Sequence

from ..sampling import Sampler, SamplingParams
from .loading import LoadedModel, load_model
from .scheduler import Request, Scheduler, StepPlan
from .step import StepEntry


class Engine:
    def __init__(self, loaded: LoadedModel, max_batch_tokens: int = 512, chunk_size: Optional[int] = None,
                 max_running: Optional[int] = None, freeze_gc: bool = True):
        self.loaded = loaded
        self.scheduler = Scheduler(loaded.cache, max_batch_tokens, chunk_size, max_running,
                                   loaded.model.spec.max_positions)
        self.sampler = Sampler(loaded.rt.ops, loaded.rt.device)
        self.steps = 0
        self.tokens_run = 0
        self._inflight = None  # (plan, launched step) of step_pipelined
        # Every step makes a few hundred short-lived objects; with the interpreter's whole heap in the
        # collector's oldest generation its full passes cost more than the scheduling itself.  What
        # exists now (modules, the model) is taken out of the collector's reach (``freeze_gc=False``
        # leaves the collector as it is).
        if freeze_gc:
            gc.collect()
            gc.freeze()

    @classmethod
    def from_dir(cls, model_dir: str, *, dtype="bfloat16", device="cuda:0", page_size: int = 64,
                 num_pages: Optional[int] = None, max_tokens: Optional[int] = None, capacity: int = 64,
                 max_batch_tokens: int = 512, chunk_size: Optional[int] = None) -> "Engine":
        loaded = load_model(model_dir, dtype=dtype, device=device, page_size=page_size, num_pages=num_pages,
                            max_tokens=max_tokens, max_requests=capacity,
                            portion=min(chunk_size or max_batch_tokens, max_batch_tokens))
        return cls(loaded, max_batch_tokens, chunk_size, capacity)

    def warm_up(self, prompt_lengths: Sequence[int]) -> int:
        """Captures, before any request has come, the steps that prompts of these lengths run as (each alone in its
        step), so that the first prompt of such a size is replayed and not launched kernel by kernel: a step is
        filled up to a size that many steps share, so a few lengths (say every 64 up to the token budget) cover every
        prompt in between.  For each length two steps are captured: a prompt of exactly that many tokens, and one a
        token shorter, which is filled up to it (and stands for every prompt that is).  Each capture runs a prompt
        of token 0 in a request of its own, which is then released.  Returns how many steps were captured; 0 where
        steps are not captured at all."""
        from ..cache import OutOfPages
        lm = self.loaded
        if not lm.step.use_graphs or self.scheduler.has_work():
            return 0
        before = len(lm.step._graphs)
        for n in sorted({m for length in prompt_lengths for m in (int(length) - 1, int(length))}):
            if not 1 <= n <= min(self.scheduler.max_batch_tokens, lm.model.spec.max_positions) or lm.cache.slots.available() < 1:
                continue
            slot = lm.cache.admit()
            try:  # as the engine runs a prompt that fits one step: sampled inside the step
                if lm.step.step_and_sample([StepEntry(slot, [0] * n, [n - 1])], [0.0], [0], [1.0], [0], capture_now=True) is None:
                    lm.step([StepEntry(slot, [0] * n, [n - 1])], borrow_logits=True, capture_now=True)
            except OutOfPages:
                pass
            finally:
                lm.cache.release(slot)
        return len(lm.step._graphs) - before

    def add(self, prompt: Sequence[int], max_new: int, params: Optional[SamplingParams] = None,
            eos: Optional[int] = None, stop_seqs: Sequence[Sequence[int]] = ()) -> int:
        vocab = self.loaded.model.vocab
        for t in prompt:
            if not 0 <= int(t) < vocab:
                raise ValueError(f"token {t} is outside the vocabulary of {vocab}")
        return self.scheduler.add(prompt, max_new, params, eos, stop_seqs)

    def cancel(self, rid: int) -> bool:
        """End a request now (reason ``"cancelled"``); its pages and slot go back at once.  A token that
        a step in flight still computes for it is dropped.  False if the request is not live
        (``continuous.rs:1266-1292``)."""
        return self.scheduler.cancel(rid)

    def has_work(self) -> bool:
        return self.scheduler.has_work() or self._inflight is not None

    def step(self):
        """One scheduled batch.  Returns ``(emitted, finished)``: the (request id, token) pairs
        produced and the requests that ended."""
        if self._inflight is not None:
            return self._drain()
        plan: StepPlan = self.scheduler.schedule()
        return self._run_plan(plan)

    def step_pipelined(self):
        """Like :meth:`step`, but a step is launched before the tokens of the step before it have come back: the
        requests that decode take them on the device, and the host's share of a step (the scheduler, the step's buffers,
        reading the samples) runs while the device works.  What is returned is what has become known by now, which lags
        the launches by one step; what would end a request is seen one step late, and the token computed for it in
        between is dropped.  Steps that cannot be launched so (sampling with penalties, biases or top log-probabilities,
        a preemption, a shape that has no captured step yet) are run as :meth:`step` runs them, after what is in
        flight."""
        sched = self.scheduler
        if self._inflight is None:
            plan = sched.schedule()
            launched = self._launch(plan, None)
            if not launched:
                # False: the step function has declined (no graph for this shape yet); not asked again
                return self._run_plan(plan, try_fast=launched is None)
            self._inflight = (plan, launched)
            return [], []
        prev_plan, prev = self._inflight
        plan = sched.schedule()
        launched = self._launch(plan, (prev_plan, prev))
        emitted, done = sched.complete(prev_plan, *self.loaded.step.collect(prev))
        if launched:
            self._inflight = (plan, launched)
            return emitted, done
        self._inflight = None
        # the plan was made before these tokens were known: what has ended meanwhile drops out of it
        plan.items = [it for it in plan.items if it.request.closing is None or it.request.pending > 0]
        plan.native = [n for n in plan.native if n.id in sched.requests]
        em2, done2 = self._run_plan(plan, try_fast=launched is None)
        return emitted + em2, done + done2

    def _launch(self, plan: StepPlan, after):
        """Launch ``plan`` without waiting for it; ``after`` is the plan in flight and its launched step, or None.
        None (nothing done) if the plan cannot be launched so, False if the step function declined.  A request's next
        token that the host has not seen yet (``pending``) must be a sample of the step in flight: it is taken from
        there on the device."""
        if not plan.items or plan.preempted or not all(it.request.params.plain() for it in plan.items if it.sample):
            return None
        reqs = [it.request for it in plan.items]
        prev_plan, prev = after if after is not None else (None, None)
        where = {}
        if prev_plan is not None:
            k = 0
            for it in prev_plan.items:
                if it.sample:
                    where[it.request.id] = k
                    k += 1
        feeds, entries = [], []
        for i, (r, it) in enumerate(zip(reqs, plan.items)):
            if it.start + it.count > len(r.tokens):
                # its first token is still on the device: one token, sampled by the step in flight
                if it.count != 1 or it.start != len(r.tokens) or r.pending != 1 or r.id not in where:
                    return None
                feeds.append((i, where[r.id]))
                entries.append(StepEntry(r.slot, [0], [0] if it.sample else []))
            else:
                entries.append(StepEntry(r.slot, r.tokens[it.start:it.start + it.count], [it.count - 1] if it.sample else []))
        sampled = [r for r, it in zip(reqs, plan.items) if it.sample]
        if not sampled:
            return None  # nothing comes back from it: it runs as it is
        args = ([r.params.temperature for r in sampled], [r.params.top_k for r in sampled], [r.params.top_p for r in sampled],
                [r.rng_state for r in sampled])
        step = self.loaded.step
        if all(it.sample and it.count == 1 for it in plan.items):
            same = prev is not None and len(feeds) == len(entries) and all(e == s for e, s in feeds) and len(where) == len(entries)
            launched = step.launch_decode(entries, *args, prev if feeds else None, None if (same or not feeds) else feeds)
        else:
            launched = step.launch_step(entries, *args, prev if feeds else None, feeds or None)
        if launched is None:
            return False
        from ..sampling import advance
        for r in sampled:
            r.rng_state = advance(r.rng_state)  # one draw a sampled row, whatever the token
        self.scheduler.begin(plan)
        self.steps += 1
        self.tokens_run += plan.n_tokens
        return launched

    def _drain(self):
        """Wait for the step in flight and take its tokens."""
        plan, launched = self._inflight
        self._inflight = None
        return self.scheduler.complete(plan, *self.loaded.step.collect(launched))

    def _run_plan(self, plan: StepPlan, try_fast: bool = True):
        if not plan.items:
            return [], []
        entries, sampled_items = [], []
        for it in plan.items:
            toks = it.request.tokens[it.start:it.start + it.count]
            entries.append(StepEntry(it.request.slot, toks, [it.count - 1] if it.sample else []))
            if it.sample:
                sampled_items.append(it)
        self.steps += 1
        self.tokens_run += plan.n_tokens
        reqs = [it.request for it in sampled_items]
        if try_fast and len(sampled_items) == len(plan.items) and all(r.params.plain() for r in reqs):
            # every request decodes one token: forward pass and sampling are one captured graph
            fast = self.loaded.step.decode_and_sample(
                entries, [r.params.temperature for r in reqs], [r.params.top_k for r in reqs],
                [r.params.top_p for r in reqs], [r.rng_state for r in reqs])
            if fast is not None:
                from ..sampling import advance
                return self.scheduler.update(plan, fast[0], fast[1], [advance(r.rng_state) for r in reqs])
        declined = False
        if try_fast and sampled_items and all(r.params.plain() for r in reqs):
            # portions of prompts, alone or beside decoded tokens: the captured step of their shared size samples too
            fast = self.loaded.step.step_and_sample(
                entries, [r.params.temperature for r in reqs], [r.params.top_k for r in reqs],
                [r.params.top_p for r in reqs], [r.rng_state for r in reqs])
            if fast is not None:
                from ..sampling import advance
                return self.scheduler.update(plan, fast[0], fast[1], [advance(r.rng_state) for r in reqs])
            declined = self.loaded.step.use_graphs  # its shape is counted there, and captured there when it has come often enough
        logits = self.loaded.step(entries, borrow_logits=True, eager=declined)
        if not sampled_items:
            return self.scheduler.update(plan, [])
        tokens, logprobs, states, top = self.sampler.sample(logits, [r.params for r in reqs], [r.rng_state for r in reqs],
                                                            [r.generated for r in reqs])
        for r, t in zip(reqs, top):
            if r.params.top_logprobs:
                r.top_logprobs.append(t)
        return self.scheduler.update(plan, tokens, logprobs, states)

    def run(self) -> Dict[int, Request]:
        """Step until every queued request has finished."""
        while self.has_work():
            self.step_pipelined()
        return self.scheduler.finished

    def generate(self, prompts: Sequence[Sequence[int]], max_new: int, temperature: float = 0.0, seed: int = 0,
                 eos: Optional[int] = None, top_k: int = 0, top_p: float = 1.0, presence_penalty: float = 0.0,
                 frequency_penalty: float = 0.0, stop_seqs: Sequence[Sequence[int]] = ()) -> List[List[int]]:
        ids = []
        for i, p in enumerate(prompts):
            params = SamplingParams(temperature=temperature, top_k=top_k, top_p=top_p,
                                    seed=(seed + i) if seed else 0, presence_penalty=presence_penalty,
                                    frequency_penalty=frequency_penalty)
            ids.append(self.add(p, max_new, params, eos, stop_seqs))
        done = self.run()
        return [done.pop(i).generated for i in ids]
