"""The cache manager (no page lost, held twice or freed twice, under random orders of
requests) and the scheduler's decisions, with the engine's host logic run on the CPU
stand-ins of the kernels."""
import random

import pytest
import torch

from emulated_ops import EmulatedOps
from plain import qwen2_plain as P
from tiny_configs import make_model_dir, random_prompt, read_for_plain


def test_block_pool_vectors():
    """crates/mach-model/src/paged_kv.rs:1343-1352."""
    from machserve_amd.cache import BlockPool, CacheError
    a = BlockPool(3)
    assert [a.alloc(), a.alloc(), a.alloc(), a.alloc()] == [0, 1, 2, None]
    a.free(1)
    assert a.alloc() == 1 and a.alloc() is None
    with pytest.raises(CacheError):
        a.free(7)
    a.free(2)
    with pytest.raises(CacheError, match="twice"):
        a.free(2)
    b = BlockPool(2)
    with pytest.raises(CacheError):
        b.free(0)  # never handed out


def _manager(window=None, pages=8, page_size=16, slots=4, state=False):
    from machserve_amd.cache import CacheManager
    from machserve_amd.parts import PagedKVRequest, SharedKVRequest, StateRequest
    reqs = [PagedKVRequest(2, 16), PagedKVRequest(2, 16, window), SharedKVRequest(0)]
    if state:
        reqs.append(StateRequest({"s": (3,)}))
    return CacheManager(reqs, page_size, pages, slots)


def test_positions_map_to_pages():
    """crates/mach-model/src/paged_kv.rs:1011-1020 (page_offsets)."""
    m = _manager(page_size=16)
    s = m.admit()
    m.extend(s, 20)
    t = m.table("full", s)
    assert len(t) == 2
    assert m.slot_of_position("full", s, 0) == t[0] * 16 and m.slot_of_position("full", s, 15) == t[0] * 16 + 15
    assert m.slot_of_position("full", s, 16) == t[1] * 16 and m.slot_of_position("full", s, 19) == t[1] * 16 + 3
    with pytest.raises(IndexError):
        m.slot_of_position("full", s, 32)


def test_groups_have_pages_of_their_own_and_windows_give_pages_back():
    from machserve_amd.cache import OutOfPages
    m = _manager(window=20, pages=6)
    assert sorted(m.groups) == ["full", "window20"] and m.layer_group == {0: "full", 1: "window20", 2: "full"}
    s = m.admit()
    for step in range(6):           # 6 * 16 = 96 tokens, one page a step
        m.extend(s, 16)
        m.commit(s, 16)
        m.check()
    assert m.free_pages("full") == 0 and len(m.table("full", s)) == 6
    # window of 20: after 96 tokens the next row sees keys > 76: pages 0..3 (keys < 64) are back
    assert m.table("window20", s)[:4] == [-1] * 4 and m.free_pages("window20") == 4
    with pytest.raises(OutOfPages):
        m.extend(s, 1)              # all-or-nothing: the full group is dry
    assert len(m.table("window20", s)) == 6
    m.release(s)
    m.check()
    assert m.free_pages("full") == 6 and m.free_pages("window20") == 6


def test_slots_and_double_release():
    from machserve_amd.cache import CacheError
    m = _manager(slots=2)
    a, b = m.admit(), m.admit()
    assert (a, b) == (0, 1)
    with pytest.raises(CacheError, match="slots"):
        m.admit()
    m.release(a)
    with pytest.raises(CacheError, match="twice"):
        m.release(a)
    assert m.admit() == 0


@pytest.mark.parametrize("seed", range(8))
def test_random_orders_lose_no_page(seed):
    from machserve_amd.cache import OutOfPages
    rng = random.Random(seed)
    m = _manager(window=rng.choice([None, 5, 40]), pages=rng.randint(3, 12), slots=4)
    live = []
    for _ in range(400):
        op = rng.random()
        if op < 0.2 and len(live) < 4:
            live.append(m.admit())
        elif op < 0.8 and live:
            s, n = rng.choice(live), rng.randint(1, 40)
            before = {g: list(m.table(g, s)) for g in m.groups}
            try:
                m.extend(s, n)
                m.commit(s, n)
            except OutOfPages:
                assert {g: list(m.table(g, s)) for g in m.groups} == before  # nothing was taken
        elif live:
            m.release(live.pop(rng.randrange(len(live))))
        m.check()
    for s in live:
        m.release(s)
    m.check()
    assert all(g.pool.available() == g.pool.num_pages for g in m.groups.values())


# ---------------------------------------------------------------------------- scheduler

def _scheduler(pages=8, page_size=16, **kw):
    from machserve_amd.engine import Scheduler
    return Scheduler(_manager(pages=pages, page_size=page_size, slots=kw.pop("slots", 4)), **kw)


def _run_plan(s, plan, token=7):
    for it in plan.items:
        s.cache.extend(it.request.slot, it.count)
        s.cache.commit(it.request.slot, it.count)
    return s.update(plan, [token] * sum(i.sample for i in plan.items))


def test_refusals_at_add():
    from machserve_amd.engine import SchedulerError
    s = _scheduler(pages=4, max_positions=100)
    with pytest.raises(SchedulerError, match="empty"):
        s.add([], 4)
    with pytest.raises(SchedulerError, match="max_new"):
        s.add([1], 0)
    with pytest.raises(SchedulerError, match="positions"):
        s.add([1] * 100, 4)
    with pytest.raises(SchedulerError, match="pages"):
        s.add([1] * 60, 10)        # 69 cached tokens need 5 pages of 16, the pool has 4


def test_prompts_are_cut_under_the_budget_and_decodes_go_first():
    s = _scheduler(pages=32, max_batch_tokens=24, chunk_size=16)
    a = s.add(list(range(40)), 3)
    b = s.add(list(range(5)), 3)
    p = s.schedule()
    assert [(i.request.id, i.start, i.count, i.sample) for i in p.items] == [(a, 0, 16, False), (b, 0, 5, True)]
    _run_plan(s, p)
    p = s.schedule()   # b decodes first, then a's next portion
    assert [(i.request.id, i.start, i.count, i.sample) for i in p.items] == [(b, 5, 1, True), (a, 16, 16, False)]
    _run_plan(s, p)
    p = s.schedule()
    assert [(i.request.id, i.start, i.count, i.sample) for i in p.items] == [(b, 6, 1, True), (a, 32, 8, True)]
    em, done = _run_plan(s, p)
    assert [r.id for r in done] == [b] and s.finished[b].finish_reason == "length" and len(s.finished[b].generated) == 3
    s.cache.check()
    while s.has_work():
        _run_plan(s, s.schedule())
    assert len(s.finished[a].generated) == 3
    assert s.cache.free_pages() == 32 and s.cache.slots.available() == 4


def test_eos_stop_sequences_and_slot_reuse():
    s = _scheduler(pages=32, slots=1)
    a = s.add([1, 2, 3], 10, eos=7)
    b = s.add([4], 10, stop_seqs=[[9, 9]])
    p = s.schedule()
    assert [i.request.id for i in p.items] == [a]     # one slot: b waits
    em, done = _run_plan(s, p, token=7)
    assert done[0].finish_reason == "stop" and done[0].generated == [7]
    for _ in range(2):
        p = s.schedule()
        assert [i.request.id for i in p.items] == [b] and p.items[0].request.slot == 0   # the slot is used again
        em, done = _run_plan(s, p, token=9)
    assert done and done[0].generated == [9, 9] and done[0].finish_reason == "stop"
    assert not s.has_work()


def test_pages_run_out_the_youngest_is_preempted_and_recomputed():
    s = _scheduler(pages=4, page_size=16, max_batch_tokens=64)
    a = s.add(list(range(30)), 20)     # up to 49 cached tokens: 4 pages alone
    b = s.add(list(range(100, 130)), 6)
    p = s.schedule()
    assert [i.request.id for i in p.items] == [a, b] and not p.preempted
    _run_plan(s, p, token=5)           # both hold 2 pages, one token generated each
    p = s.schedule()
    assert [i.request.id for i in p.items] == [a, b]
    _run_plan(s, p, token=5)           # 31 cached each
    _run_plan(s, s.schedule(), token=5)  # 32 cached each: both second pages are full
    p = s.schedule()                   # position 32 needs a third page for both: none is free
    assert [r.id for r in p.preempted] == [b] and [i.request.id for i in p.items] == [a]
    rb = p.preempted[0]
    assert rb.slot is None and rb.fed == 0 and rb.generated == [5, 5, 5] and s.waiting[0] is rb
    s.cache.check()
    while s.has_work():
        _run_plan(s, s.schedule(), token=5)
        s.cache.check()
    assert len(s.finished[a].generated) == 20 and len(s.finished[b].generated) == 6
    assert s.finished[b].preemptions >= 1 and s.cache.free_pages() == 4


def test_decoders_never_outnumber_the_budget_and_nobody_starves():
    """A budget of two tokens a step and four requests: a request starts only in a step that has budget left
    beside every decoding request, so at most two decode at a time, the others wait their turn in the queue,
    every step is full, nobody is preempted while pages suffice, and all finish."""
    s = _scheduler(pages=9, page_size=16, max_batch_tokens=2, chunk_size=2, slots=4)
    ids = [s.add([1, 2], 12) for _ in range(4)]
    steps = 0
    while s.has_work():
        p = s.schedule()
        assert not p.preempted and 1 <= p.n_tokens <= 2
        assert sum(r.decoding for r in s.running) <= 2
        _run_plan(s, p)
        s.cache.check()
        steps += 1
    assert all(len(s.finished[i].generated) == 12 for i in ids)
    assert steps <= 4 * 13 // 2 + 4   # 52 tokens through a budget of two, a few half-empty steps at the seams


@pytest.mark.parametrize("seed", range(8))
def test_more_slots_than_budget_under_random_arrivals_and_preemptions(seed):
    """More requests may run than a step holds tokens, pages are short and requests arrive at random: in every
    plan the decoding requests fit the budget (the core refuses a plan that would break this before it has
    preempted anybody), every step runs something, and all requests finish."""
    rng = random.Random(100 + seed)
    budget = rng.choice([2, 3, 5])
    s = _scheduler(pages=rng.randint(5, 9), page_size=16, max_batch_tokens=budget, chunk_size=rng.choice([None, 2]), slots=8)
    want, queue = {}, [(rng.randint(1, 40), rng.randint(1, 30), rng.randrange(0, 60)) for _ in range(14)]
    queue.sort(key=lambda q: q[2])
    steps = preempted = 0
    while queue or s.has_work():
        while queue and (queue[0][2] <= steps or not s.has_work()):
            n, m, _ = queue.pop(0)
            want[s.add([rng.randrange(50) for _ in range(n)], m)] = m
        p = s.schedule()
        assert p.items and p.n_tokens <= budget
        assert sum(r.decoding for r in s.running) <= budget
        preempted += len(p.preempted)
        _run_plan(s, p, token=rng.randrange(50))
        s.cache.check()
        steps += 1
        assert steps < 5000
    assert {i: len(r.generated) for i, r in s.finished.items()} == want
    _PREEMPTED.append(preempted)


_PREEMPTED = []


def test_the_random_arrivals_above_did_preempt():
    if not _PREEMPTED:
        pytest.skip("the test above did not run in this process")
    assert sum(_PREEMPTED) > 0


def test_a_window_group_is_sized_by_its_window_not_by_the_request():
    """A long request on a model whose layers all see a window needs pages for window + portion keys
    only: it is admitted with a pool far smaller than its length, and runs to the end."""
    from machserve_amd.cache import CacheManager
    from machserve_amd.engine import Scheduler, SchedulerError
    from machserve_amd.parts import PagedKVRequest
    m = CacheManager([PagedKVRequest(2, 16, 40)], 16, 6, 2)      # window 40, 6 pages of 16
    s = Scheduler(m, max_batch_tokens=32, chunk_size=32)
    rid = s.add(list(range(600)), 8)        # 607 cached tokens = 38 pages if all keys were kept
    while s.has_work():
        p = s.schedule()
        assert p.items and not p.preempted
        _run_plan(s, p)
        m.check()
    assert len(s.finished[rid].generated) == 8 and m.free_pages() == 6
    # with a group of all keys beside it the request is refused, by that group's name
    m2 = CacheManager([PagedKVRequest(2, 16, 40), PagedKVRequest(2, 16)], 16, 6, 2)
    with pytest.raises(SchedulerError, match="group full"):
        Scheduler(m2, max_batch_tokens=32, chunk_size=32).add(list(range(600)), 8)
    # and a window group too small for window + portion refuses as well
    m3 = CacheManager([PagedKVRequest(2, 16, 40)], 16, 4, 2)
    with pytest.raises(SchedulerError, match="window40"):
        Scheduler(m3, max_batch_tokens=32, chunk_size=32).add(list(range(600)), 8)


@pytest.mark.parametrize("seed", range(6))
def test_random_load_always_finishes(seed):
    rng = random.Random(seed)
    s = _scheduler(pages=rng.randint(4, 10), page_size=16, max_batch_tokens=rng.choice([8, 32, 64]),
                   chunk_size=rng.choice([None, 4, 16]))
    want = {}
    steps = 0
    for _ in range(12):
        n, m = rng.randint(1, 40), rng.randint(1, 20)
        if -(-(n + m - 1) // 16) <= s.cache.groups["full"].pool.num_pages:
            want[s.add([rng.randrange(50) for _ in range(n)], m)] = m
    while s.has_work():
        p = s.schedule()
        assert p.items, "a step with work must run something"
        assert p.n_tokens <= s.max_batch_tokens
        _run_plan(s, p, token=rng.randrange(50))
        s.cache.check()
        steps += 1
        assert steps < 5000
    assert {i: len(r.generated) for i, r in s.finished.items()} == want


def test_pages_by_need_give_a_window_group_what_its_requests_can_hold_and_the_bytes_follow(tmp_path):
    """A model whose later layers see a window: with the rule, the window group's pool holds what its requests can
    hold of it at a time, not the whole pool once more; a dict names each group's pages; the device cache's byte
    count is pages + 1 (the scratch page) times the layers' page bytes; and the engine still equals the plain model."""
    from machserve_amd.cache import CacheError, CacheManager, pages_by_need
    from machserve_amd.engine import Engine, load_model
    from machserve_amd.parts import PagedKVRequest
    reqs = [PagedKVRequest(2, 16), PagedKVRequest(2, 16, 40), PagedKVRequest(2, 16, 40)]
    m = CacheManager(reqs, 16, pages_by_need(max_tokens=4096, max_requests=3, portion=24, page_size=16), 3)
    # all keys: 4096 / 16; window 40 + portion 24 - 1 = 63 keys touch at most 4 + 1 pages a request
    assert {n: g.pool.num_pages for n, g in m.groups.items()} == {"full": 256, "window40": 3 * 5}
    m = CacheManager(reqs, 16, {"full": 7, "window40": 3}, 3)
    assert {n: g.pool.num_pages for n, g in m.groups.items()} == {"full": 7, "window40": 3}
    with pytest.raises(CacheError, match="window40"):
        CacheManager(reqs, 16, {"full": 7}, 3)
    with pytest.raises(CacheError, match="nobody"):
        CacheManager(reqs, 16, {"full": 7, "window40": 3, "nobody": 1}, 3)
    d = make_model_dir(tmp_path, "C")     # configuration C has layers that see a window
    w, sizes = read_for_plain(d)
    lm = load_model(d, dtype="float32", device="cpu", page_size=16, max_tokens=320, max_requests=2, portion=16, ops=EmulatedOps())
    windows = {g.spec.window for g in lm.cache.groups.values()}
    assert None in windows and len(windows) == 2, "configuration C must have both kinds of layers"
    want_bytes = 0
    for g in lm.cache.groups.values():
        pages = 320 // 16 if g.spec.window is None else min(20, 2 * (-(-(g.spec.window + 15) // 16) + 1))
        assert g.pool.num_pages == pages
        want_bytes += len(g.spec.layers) * (pages + 1) * 2 * g.spec.kv_heads * 16 * g.spec.head_dim * 4
    assert lm.device_cache.bytes() == want_bytes
    assert lm.device_cache.bytes() < sum(len(g.spec.layers) for g in lm.cache.groups.values()) * 21 * 2 * 16 * 4 * max(
        g.spec.kv_heads * g.spec.head_dim for g in lm.cache.groups.values())
    eng = Engine(lm, max_batch_tokens=16, max_running=2)
    prompts = [random_prompt(n, sizes["vocab"], 70 + n) for n in (90, 33)]
    got = eng.generate(prompts, max_new=8)
    for p, g in zip(prompts, got):
        assert g == P.greedy_generate(w, sizes, p, 8)


@pytest.mark.parametrize("which", ["A", "C"])
def test_a_step_filled_up_to_a_shared_size_gives_the_same_logits(tmp_path, which):
    """Steps of any mix are filled up to a size that many steps share (rows, requests, wanted rows, work items) so
    that one captured graph serves them all: the rows that fill a step up belong to nobody, write to the scratch page
    and the scratch slot, and change no logit of a request.  Here on the CPU stand-ins, through the same buffer."""
    from machserve_amd.engine import StepEntry, load_model
    d = make_model_dir(tmp_path, which)
    w, sizes = read_for_plain(d)
    lm = load_model(d, dtype="float32", device="cpu", page_size=16, num_pages=24, max_requests=4, ops=EmulatedOps())
    sf = lm.step
    assert sf._fill_shape(1, 100, 1) == (128, 2, 1) and sf._fill_shape(3, 17, 3) == (32, 4, 4) and sf._fill_shape(4, 60, 0) == (64, 8, 0) and sf._fill_shape(4, 64, 0) == (64, 4, 0)
    assert sf._fill_shape(1, 600, 1) == (640, 2, 1) and sf._fill_shape(1, 1000, 1) == (1024, 2, 1) and sf._fill_shape(1, 1100, 1) is None
    assert sf._fill_shape(1, 1230, 1) == (1280, 2, 1) and sf._fill_shape(1, 2048, 1) == (2048, 1, 1) and sf._fill_shape(2, 5000, 1) is None
    seqs = [random_prompt(n, sizes["vocab"], 20 + n) for n in (50, 23, 9)]
    refs = [P.forward(w, sizes, s) for s in seqs]
    slots = [lm.cache.admit() for _ in seqs]
    fed = [0, 0, 0]
    for cuts in ([30, 23, 0], [19, 0, 8], [1, 0, 1], [0, 0, 0]):
        if not any(cuts):   # a step that has a shared size already: sixteen rows of one request
            lm.cache.release(slots[1])
            slots[1], fed[1], seqs[1] = lm.cache.admit(), 0, random_prompt(16, sizes["vocab"], 99)
            refs[1] = P.forward(w, sizes, seqs[1])
            cuts = [0, 16, 0]
        entries = [StepEntry(slots[r], seqs[r][fed[r]:fed[r] + n], [0, n - 1] if n > 1 else [0]) for r, n in enumerate(cuts) if n]
        who = [r for r, n in enumerate(cuts) if n]
        checked = sf._check_entries(entries)
        sf._take_pages(entries)
        sl, counts, tokens, want, _ = checked
        fill = sf._fill_shape(len(sl), len(tokens), len(want))
        host, offsets, widths = lm.cache.build_step(sl, counts, tokens, want, sf.heads_per_kv, sf.rows_per_block, 8, 0, 1, (), fill)
        assert offsets["tokens"][1] == fill[0] and offsets["seq_slot"][1] == fill[1] and offsets["want_rows"][1] == fill[2]
        for g in sf.heads_per_kv:   # as many work items as any step of this size can have
            assert offsets[f"work/{g}"][1] == 2 * (-(-fill[0] * g // sf.rows_per_block) + fill[1])
        logits = lm.model.forward(sf._context_from(torch.from_numpy(host), offsets, widths))[:len(want)]
        k = 0
        for r, e in zip(who, entries):
            for place in e.want:
                ref = refs[r][fed[r] + place]
                assert (logits[k] - ref).abs().max() <= 2e-5 * (1 + ref.abs().max())
                k += 1
            lm.cache.commit(e.slot, len(e.tokens))
            fed[r] += len(e.tokens)
        lm.cache.check()
    for s_ in slots:
        lm.cache.release(s_)
    assert all(g.pool.available() == g.pool.num_pages for g in lm.cache.groups.values())


def test_layers_of_equal_frequencies_share_one_rotation_table():
    """Rotary parts of equal frequencies hold the same tensor (what a step works out from it is then made once for all
    layers); other frequencies, another table."""
    from machserve_amd.config import RotarySpec, YarnSpec
    from machserve_amd.parts import POSITION_ENCODINGS, Runtime
    rt = Runtime(torch.device("cpu"), torch.float32, EmulatedOps())
    a, b = (POSITION_ENCODINGS.build(RotarySpec("rotary", 64, 1e6), rt) for _ in range(2))
    assert a is not b and a.rotary_inv_freq() is b.rotary_inv_freq()
    for other in (RotarySpec("rotary", 64, 1e4), RotarySpec("rotary", 32, 1e6),
                  RotarySpec("rotary", 64, 1e6, yarn=YarnSpec(4.0, 64, 32.0, 1.0, 1.0, 0.0))):
        c = POSITION_ENCODINGS.build(other, rt)
        assert c.rotary_inv_freq() is not a.rotary_inv_freq() and not (c.rotary_inv_freq().shape == a.rotary_inv_freq().shape
                                                                         and torch.equal(c.rotary_inv_freq(), a.rotary_inv_freq()))


@pytest.mark.parametrize("mscale_all_dim", [0.0, 0.707])
def test_yarn_through_the_engine_equals_the_plain_model(tmp_path, mscale_all_dim):
    """A configuration with YaRN (crates/mach-model/src/ref_model.rs:636-704): scaled frequencies, the factor on
    cosines and sines (which the engine puts on the scores, squared) and mscale_all_dim's square on the scores'
    scale; positions far beyond the original context, in portions and token by token."""
    from machserve_amd.engine import StepEntry, load_model
    from machserve_amd.weights import write_random_model
    from tiny_configs import TINY_A, sharpen_attention
    raw = dict(TINY_A, max_position_embeddings=512,
               rope_scaling={"type": "yarn", "factor": 8.0, "original_max_position_embeddings": 32, "mscale_all_dim": mscale_all_dim})
    d = write_random_model(raw, 3, str(tmp_path / "yarn"))
    sharpen_attention(d, 4.0)
    w, sizes = read_for_plain(d)
    assert sizes["rope_scaling"]["factor"] == 8.0
    toks = random_prompt(300, 512, 5)
    ref = P.forward(w, sizes, toks)
    without = P.forward(w, dict(sizes, rope_scaling=None), toks)
    assert (ref - without).abs().max() > 1e-2 * ref.abs().max(), "the test must tell YaRN from plain rotation"
    lm = load_model(d, dtype="float32", device="cpu", page_size=16, num_pages=20, max_requests=1, ops=EmulatedOps())
    slot = lm.cache.admit()
    got = [lm.step([StepEntry(slot, toks[:170], list(range(170)))]), lm.step([StepEntry(slot, toks[170:290], list(range(120)))])]
    got += [lm.step([StepEntry(slot, toks[i:i + 1], [0])]) for i in range(290, 300)]
    got = torch.cat(got)
    assert (got - ref).abs().max() <= 2e-5 * (1 + ref.abs().max())


def test_replay_writes_every_layer_s_stream_at_the_wanted_places(tmp_path):
    """The replay program's debugging aid (crates/mach-model/src/batched.rs:3040-3088): the residual stream after the
    embedding and after every layer, at the wanted places of a step, equals the plain model's; a fault put into one
    layer's weights shows in that layer's file first."""
    import json
    import numpy as np
    from machserve_amd.engine import load_model
    from machserve_amd.engine.replay import replay
    d = make_model_dir(tmp_path, "C")
    w, sizes = read_for_plain(d)
    toks = random_prompt(70, sizes["vocab"], 9)
    lm = load_model(d, dtype="float32", device="cpu", page_size=16, num_pages=12, max_requests=2, ops=EmulatedOps())
    lines = [json.dumps({"step": 0, "entries": [{"id": "a", "tokens": toks[:50], "want": []}], "end": []}),
             json.dumps({"step": 1, "entries": [{"id": "a", "tokens": toks[50:], "want": [3, 19]}], "end": ["a"]})]
    out, layers = tmp_path / "out", tmp_path / "layers"
    out.mkdir(), layers.mkdir()
    replay(lm, lines, str(out), say=lambda m: None, layers_dir=str(layers))
    streams = []
    ref = P.forward(w, sizes, toks, streams=streams)
    rows = [53, 69]
    got = np.fromfile(out / "1.f32", dtype="<f4").reshape(2, -1)
    assert np.abs(got - ref[rows].numpy()).max() <= 2e-5 * (1 + ref.abs().max().item())
    names = ["embedding"] + [f"layer{i:02d}" for i in range(sizes["layers"])]
    assert sorted(f.name for f in layers.iterdir()) == sorted(f"1_{n}.f32" for n in names)   # step 0 wanted nothing
    for n, want in zip(names, streams):
        g = np.fromfile(layers / f"1_{n}.f32", dtype="<f4").reshape(2, sizes["hidden"])
        assert np.abs(g - want[rows].numpy()).max() <= 2e-5 * (1 + want.abs().max().item()), n
    # a changed weight in layer 2: layers 0 and 1 still agree, layer 2 is the first that does not
    w2 = dict(w)
    w2["model.layers.2.mlp.down_proj.weight"] = w["model.layers.2.mlp.down_proj.weight"] * 1.5
    streams2 = []
    P.forward(w2, sizes, toks, streams=streams2)
    differs = [n for n, want in zip(names, streams2)
               if np.abs(np.fromfile(layers / f"1_{n}.f32", dtype="<f4").reshape(2, -1) - want[rows].numpy()).max() > 1e-4]
    assert differs == ["layer02", "layer03"]
    assert lm.model.observer is not None and lm.step.use_graphs is False


def test_a_refused_step_takes_no_pages(tmp_path):
    """A step with a bad token, a slot twice, a place beyond its tokens, or a slot that no request holds is refused
    before anything is taken: the tables, the free pages and the lengths are what they were."""
    from machserve_amd.engine import StepEntry, StepError, load_model
    d = make_model_dir(tmp_path, "A")
    lm = load_model(d, dtype="float32", device="cpu", page_size=16, num_pages=6, max_requests=3, ops=EmulatedOps())
    a, b = lm.cache.admit(), lm.cache.admit()
    lm.step([StepEntry(a, [1, 2, 3], [2]), StepEntry(b, [4] * 17, [])])
    free, lengths, tables = lm.cache.free_pages(), dict(lm.cache.lengths), [lm.cache.table("full", s) for s in (a, b)]
    bad = [
        [StepEntry(a, [5] * 20, []), StepEntry(b, [512], [0])],               # a token outside the vocabulary, after a good entry
        [StepEntry(a, [5] * 20, []), StepEntry(a, [1], [0])],                  # a slot twice
        [StepEntry(a, [5] * 20, [20])],                                        # a wanted place beyond the tokens
        [StepEntry(a, [5] * 20, []), StepEntry(2, [1], [0])],                  # a slot nobody holds
        [StepEntry(a, [5] * 20, []), StepEntry(b, [], [])],                    # an empty entry
        [StepEntry(a, [5] * 300, [])],                                         # beyond the model's positions
    ]
    for entries in bad:
        with pytest.raises(StepError):
            lm.step(entries)
        lm.cache.check()
        assert lm.cache.free_pages() == free and dict(lm.cache.lengths) == lengths
        assert [lm.cache.table("full", s) for s in (a, b)] == tables
    # and the step function still works
    out = lm.step([StepEntry(a, [5] * 20, [19])])
    assert out.shape == (1, 512) and lm.cache.length(a) == 23


# ---------------------------------------------------------------------------- engine on the CPU stand-ins

@pytest.mark.parametrize("which,pages,budget,runs_out", [("A", 8, 512, False), ("A", 5, 12, False), ("A", 3, 64, True),
                                                          ("B", 6, 24, False), ("B", 3, 64, True), ("C", 16, 32, False),
                                                          ("C", 3, 32, True)])
def test_engine_generations_equal_plain_greedy(tmp_path, which, pages, budget, runs_out):
    """The reference's central test (crates/mach-model/tests/continuous.rs:80-97, 216-247,
    393-427): what the engine generates equals single-request greedy generation, token for
    token, also when prompts are cut, requests wait for a slot, and pages run out."""
    from machserve_amd.engine import Engine, load_model
    d = make_model_dir(tmp_path, which)
    w, sizes = read_for_plain(d)
    ps = {"A": 16, "B": 32, "C": 16}[which]
    lm = load_model(d, dtype="float32", device="cpu", page_size=ps, num_pages=pages, max_requests=3, ops=EmulatedOps())
    eng = Engine(lm, max_batch_tokens=budget)
    # when pages are to run out: three prompts that fill a page each, so that their decoded tokens need a second one
    # at about the same time, from a pool of three
    lengths = (ps - 1, ps - 2, ps, 9) if runs_out else (5, 17, 33, 9)
    prompts = [random_prompt(n, sizes["vocab"], 40 + n) for n in lengths]
    ids = [eng.add(p, 8) for p in prompts]
    done = eng.run()
    for p, i in zip(prompts, ids):
        assert done[i].generated == P.greedy_generate(w, sizes, p, 8)
    lm.cache.check()
    assert all(g.pool.available() == g.pool.num_pages for g in lm.cache.groups.values())
    preemptions = sum(done[i].preemptions for i in ids)
    assert (preemptions > 0) == runs_out, f"{preemptions} preemptions with {pages} pages"


def test_engine_sampling_is_deterministic_and_survives_preemption(tmp_path):
    from machserve_amd.engine import Engine, load_model
    from machserve_amd.sampling import SamplingParams
    d = make_model_dir(tmp_path, "A")
    w, sizes = read_for_plain(d)
    prompts = [random_prompt(n, 512, 60 + n) for n in (20, 25)]

    def run(pages):
        lm = load_model(d, dtype="float32", device="cpu", page_size=16, num_pages=pages, max_requests=2, ops=EmulatedOps())
        eng = Engine(lm, max_batch_tokens=64)
        ids = [eng.add(p, 14, SamplingParams(temperature=1.0, top_k=50, seed=11 + i)) for i, p in enumerate(prompts)]
        done = eng.run()
        return [done[i].generated for i in ids], sum(done[i].preemptions for i in ids)

    roomy, n0 = run(16)
    tight, n1 = run(5)
    assert n0 == 0 and n1 > 0, "the small pool must force a preemption"
    assert roomy == tight
    # and the tokens are the CPU mirror's draws on the plain model's logits
    seq, st = list(prompts[0]), 11
    for t in roomy[0][:4]:
        tok, st = P.sample(P.forward(w, sizes, seq)[-1].numpy(), 1.0, 50, 1.0, st)
        assert tok == t
        seq.append(tok)


def test_engine_reports_logprobs_and_top_logprobs(tmp_path):
    """Options that need the logits after the draw: the engine leaves its captured-graph path."""
    from machserve_amd.engine import Engine, load_model
    from machserve_amd.sampling import SamplingParams
    d = make_model_dir(tmp_path, "A")
    w, sizes = read_for_plain(d)
    lm = load_model(d, dtype="float32", device="cpu", page_size=16, num_pages=8, max_requests=2, ops=EmulatedOps())
    eng = Engine(lm)
    p = random_prompt(9, 512, 5)
    rid = eng.add(p, 4, SamplingParams(top_logprobs=3, presence_penalty=0.5, logit_bias={7: 1.0}))
    r = eng.run()[rid]
    assert len(r.generated) == 4 and len(r.top_logprobs) == 4 and all(len(t) == 3 for t in r.top_logprobs)
    seq, counts = list(p), {}
    for step, tok in enumerate(r.generated):
        logits = P.forward(w, sizes, seq)[-1].clone()
        for t, c in counts.items():
            logits[t] -= 0.5
        logits[7] += 1.0
        lp = torch.log_softmax(logits.double(), -1)
        best = torch.argsort(-logits.double(), stable=True)[:3].tolist()
        assert [t for t, _ in r.top_logprobs[step]] == best and tok == best[0]
        assert abs(r.top_logprobs[step][0][1] - lp[best[0]].item()) < 1e-4
        counts[tok] = counts.get(tok, 0) + 1
        seq.append(tok)
    with pytest.raises(ValueError, match="top_logprobs"):
        eng.add(p, 1, SamplingParams(top_logprobs=21))


class _LaggedDecode:
    """Stand-in on the CPU for the launched steps of the device: what a step samples stays out of
    the engine's sight until ``collect``, and a step launched after another takes that step's tokens
    from it directly, as the device does (row for row, or for the listed entries)."""

    def __init__(self, eng):
        self.eng, self.fed_from_device, self.mixed = eng, 0, 0
        eng.loaded.step.launch_decode = self.launch_decode
        eng.loaded.step.launch_step = self.launch_step
        eng.loaded.step.collect = lambda launched: (launched["tokens"], launched["logprobs"])

    def _run(self, entries, temperatures, top_ks, top_ps, states, after, feeds):
        from machserve_amd.engine.step import StepEntry
        from machserve_amd.sampling import SamplingParams
        entries = list(entries)
        if after is not None:
            if feeds is None:
                assert after["slots"] == [e.slot for e in entries]
                feeds = [(i, i) for i in range(len(entries))]
            for i, src in feeds:
                assert len(entries[i].tokens) == 1
                entries[i] = StepEntry(entries[i].slot, [after["tokens"][src]], entries[i].want)
            self.fed_from_device += 1
        logits = self.eng.loaded.step(entries)
        params = [SamplingParams(temperature=t, top_k=k, top_p=p) for t, k, p in zip(temperatures, top_ks, top_ps)]
        tokens, logprobs, _, _ = self.eng.sampler.sample(logits, params, list(states), [[] for _ in params])
        return {"slots": [e.slot for e in entries for _ in e.want], "tokens": [int(t) for t in tokens], "logprobs": list(logprobs)}

    def launch_decode(self, entries, temperatures, top_ks, top_ps, states, after=None, feeds=None):
        if not all(len(e.tokens) == 1 for e in entries):
            return None
        return self._run(entries, temperatures, top_ks, top_ps, states, after, feeds)

    def launch_step(self, entries, temperatures, top_ks, top_ps, states, after=None, feeds=None, capture_now=False):
        if all(len(e.tokens) == 1 for e in entries):
            return None
        self.mixed += 1
        return self._run(entries, temperatures, top_ks, top_ps, states, after, feeds)


@pytest.mark.parametrize("pages", [16, 4])
def test_pipelined_steps_give_what_synchronous_steps_give(tmp_path, pages):
    """Steps launched before the tokens of the step before are known: the same tokens, log
    probabilities and reasons to finish as with one step at a time, although an end-of-sequence
    token or a stop sequence is seen one step late, requests end at different steps, one arrives in
    the middle, and (with few pages) one is preempted."""
    from machserve_amd.engine import Engine, load_model
    from machserve_amd.sampling import SamplingParams
    d = make_model_dir(tmp_path, "A")
    prompts = [random_prompt(n, 512, 80 + n) for n in (7, 19, 12, 5)]
    max_new = [14, 6, 11, 9]

    def run(pipelined, eos=None, stop=()):
        lm = load_model(d, dtype="float32", device="cpu", page_size=16, num_pages=pages, max_requests=3, ops=EmulatedOps())
        eng = Engine(lm, max_batch_tokens=32)
        lag = _LaggedDecode(eng)
        ids = [eng.add(p, m, SamplingParams(temperature=0.9, top_k=40, seed=3 + i), eos=eos, stop_seqs=stop)
               for i, (p, m) in enumerate(zip(prompts[:3], max_new))]
        emitted, n = [], 0
        while eng.has_work():
            em, _ = eng.step_pipelined() if pipelined else eng.step()
            emitted += em
            n += 1
            if n == 5:
                ids.append(eng.add(prompts[3], max_new[3], SamplingParams(temperature=0.7, seed=9), eos=eos, stop_seqs=stop))
            lm.cache.check()
            assert n < 500
        assert all(g.pool.available() == g.pool.num_pages for g in lm.cache.groups.values())
        done = eng.scheduler.finished
        per_request = {i: [t for j, t in emitted if j == i] for i in ids}
        assert all(per_request[i] == done[i].generated for i in ids)
        return ([(done[i].generated, done[i].finish_reason, [round(x, 5) for x in done[i].logprobs]) for i in ids],
                lag.fed_from_device, sum(done[i].preemptions for i in ids), lag.mixed)

    plain, _, _, _ = run(False)
    piped, from_device, preempted, mixed = run(True)
    assert piped == plain and from_device > 3
    assert mixed >= 2, "the prompts' steps and the step of the arrival beside the decoding requests were launched ahead too"
    assert (preempted > 0) == (pages == 4)
    assert [r for _, r, _ in plain] == ["length"] * 4
    # an end-of-sequence token and a stop sequence taken from the middle of what request 0 generates
    first = plain[0][0]
    eos = first[5]
    stop = [first[3:5]]
    for kw in ({"eos": eos}, {"stop": stop}, {"eos": plain[1][0][-1]}):
        a, _, _, _ = run(False, **kw)
        b, n_dev, _, _ = run(True, **kw)
        assert a == b and n_dev > 0
        assert "stop" in [r for _, r, _ in a]


@pytest.mark.parametrize("seed", range(6))
def test_pipelined_steps_under_random_arrivals(tmp_path, seed):
    """Requests of random lengths arriving at random steps under a small token budget and few pages, some ending at an
    end-of-sequence token: steps of every mix launched one ahead (prompt portions beside requests that take their token
    from the step in flight) give every request the tokens, log-probabilities and reason to finish of one step at a
    time."""
    from machserve_amd.engine import Engine, load_model
    from machserve_amd.sampling import SamplingParams
    d = make_model_dir(tmp_path, "B")
    rnd = random.Random(70 + seed)
    vocab = read_for_plain(d)[1]["vocab"]
    n = 9
    prompts = [random_prompt(rnd.randint(2, 45), vocab, 900 + 17 * seed + i) for i in range(n)]
    max_new = [rnd.randint(1, 12) for _ in range(n)]
    arrive = sorted(rnd.randint(0, 25) for _ in range(n))
    temps = [rnd.choice([0.0, 0.8]) for _ in range(n)]
    budget, pages = rnd.choice([16, 24, 48]), rnd.choice([10, 14, 30])

    def run(pipelined, eos):
        lm = load_model(d, dtype="float32", device="cpu", page_size=16, num_pages=pages, max_requests=3, ops=EmulatedOps())
        eng = Engine(lm, max_batch_tokens=budget)
        lag = _LaggedDecode(eng)
        ids, step = [], 0
        while len(ids) < n or eng.has_work():
            while len(ids) < n and arrive[len(ids)] <= step:
                i = len(ids)
                ids.append(eng.add(prompts[i], max_new[i], SamplingParams(temperature=temps[i], seed=5 + i), eos=eos))
            if eng.has_work():
                eng.step_pipelined() if pipelined else eng.step()
            step += 1
            lm.cache.check()
            assert step < 2000
        assert all(g.pool.available() == g.pool.num_pages for g in lm.cache.groups.values())
        done = eng.scheduler.finished
        return [(done[i].generated, done[i].finish_reason, [round(x, 5) for x in done[i].logprobs]) for i in ids], lag

    plain, _ = run(False, None)
    piped, lag = run(True, None)
    assert piped == plain
    assert lag.mixed > 0 and lag.fed_from_device > 0
    # a token that some request generates in its middle ends every request that meets it
    longest = max(plain, key=lambda r: len(r[0]))[0]
    if len(longest) >= 3:
        eos = longest[len(longest) // 2]
        assert run(True, eos)[0] == run(False, eos)[0]


def test_cancel_while_a_step_is_in_flight(tmp_path):
    """A request cancelled between two launches: the token the step in flight computes for it is
    dropped, the others go on as if it had never been there, and its pages are back at once."""
    from machserve_amd.engine import Engine, load_model
    from machserve_amd.sampling import SamplingParams
    d = make_model_dir(tmp_path, "A")
    prompts = [random_prompt(n, 512, 30 + n) for n in (6, 11)]

    def run(cancel_at):
        lm = load_model(d, dtype="float32", device="cpu", page_size=16, num_pages=8, max_requests=2, ops=EmulatedOps())
        eng = Engine(lm, max_batch_tokens=32)
        _LaggedDecode(eng)
        ids = [eng.add(p, 12, SamplingParams(temperature=0.9, seed=4 + i)) for i, p in enumerate(prompts)]
        n = 0
        while eng.has_work():
            eng.step_pipelined()
            n += 1
            if n == cancel_at:
                assert eng._inflight is not None, "the cancellation is meant to meet a step in flight"
                free = lm.cache.groups["full"].pool.available()
                assert eng.cancel(ids[1]) and not eng.cancel(ids[1])
                assert lm.cache.groups["full"].pool.available() > free
            lm.cache.check()
        done = eng.scheduler.finished
        return [(done[i].generated, done[i].finish_reason) for i in ids]

    whole, cut = run(None), run(5)
    assert cut[0] == whole[0] and whole[0][1] == "length"
    assert cut[1][1] == "cancelled" and 0 < len(cut[1][0]) < 12 and cut[1][0] == whole[1][0][:len(cut[1][0])]
