"""The engine against the plain model through the step function, cache and kernels that
generation uses: each request alone and whole; most of it in one step and the last 32
tokens one by one; portions of changing size down to two tokens; and mixed, up to four
live requests with portions of some beside decoded tokens of others and so few pages
that they are handed out again.  In 32-bit and in bfloat16."""
import pytest
import torch

from gpu_util import DEV
from plain import qwen2_plain as P
from tiny_configs import CONFIGS, make_model_dir, random_prompt, read_for_plain

pytestmark = pytest.mark.gpu

PAGE = {"A": 16, "B": 32, "C": 16}
LENGTHS = {"A": [5, 17, 33, 90], "B": [1, 9, 40, 100], "C": [3, 64, 130, 47]}


BF16_ROUNDED_TOL = 1.5e-2   # against the plain model that rounds where the engine rounds (see ``check``)
F16_TOL, F16_ROUNDED_TOL = 3e-2 / 8, 1.5e-2 / 8   # half precision has three bits of mantissa more than bfloat16


def logit_tol(dtype, ref):
    """float32: the reference's own bound for a 32-bit GPU against a CPU forward is
    2e-3 + 2e-3 * scale (crates/mach-model/tests/decode_slice.rs:79-85); ours is a hundred
    times tighter.  bfloat16 (weights rounded once, activations rounded at every matrix
    input, cache in bfloat16): 8 bits of mantissa, ~2^-8 per rounding, a few dozen roundings
    adding up like a random walk."""
    scale = ref.abs().max().item()
    if dtype == torch.float16:
        return F16_TOL * scale
    return (2e-5 + 2e-5 * scale) if dtype == torch.float32 else (3e-2 * scale)


@pytest.fixture(scope="module")
def models(tmp_path_factory):
    tmp = tmp_path_factory.mktemp("models")
    out = {}
    for which in CONFIGS:
        d = make_model_dir(tmp, which)
        w, sizes = read_for_plain(d)
        prompts = [random_prompt(n, sizes["vocab"], 10 * i + len(which)) for i, n in enumerate(LENGTHS[which])]
        out[which] = (d, w, sizes, prompts, {})
    return out


class Ref:
    """The plain model's logits of a prompt; for bfloat16 also those of the plain model that stores in
    bfloat16 what the engine stores in bfloat16 (``rounded``)."""

    def __init__(self, logits, rounded=None):
        self.logits, self.rounded = logits, rounded

    def __getitem__(self, idx):
        return Ref(self.logits[idx], None if self.rounded is None else self.rounded[idx])


def plain_ref(w, sizes, prompt, dtype):
    if dtype == torch.float32:
        return Ref(P.forward(w, sizes, prompt))
    ww = {k: v.to(dtype).float() if v.dim() == 2 else v for k, v in w.items()}  # the matrices are stored in the element type
    stored = P.to_bf16_and_back if dtype == torch.bfloat16 else P.to_f16_and_back
    return Ref(P.forward(ww, sizes, prompt), P.forward(ww, sizes, prompt, rounded=stored))


def plain_logits(models, which, dtype, i):
    d, w, sizes, prompts, memo = models[which]
    key = (dtype, i)
    if key not in memo:
        memo[key] = plain_ref(w, sizes, prompts[i], dtype)
    return memo[key]


def engine(models, which, dtype, num_pages):
    from machserve_amd.engine import load_model
    return load_model(models[which][0], dtype=dtype, device=DEV, page_size=PAGE[which], num_pages=num_pages)


WORST = {}


def check(got, ref, dtype, what):
    """float32: equal to the plain model within the rounding of sums in another order, and the same most likely
    token everywhere.  bfloat16: within 3e-2 of the logits' scale of the plain model with bfloat16 matrices, and
    within 1.5e-2 (four units in the last place of a bfloat16 number of the logits' size) of the plain model that also
    stores in bfloat16 every value that the engine stores in bfloat16 (the inputs of the matrix products, q, the
    cache, the probabilities that multiply the values).  The second bound is what a rounding in a place of the
    engine's own (a stream or a sum kept in bfloat16) would break: equal rounding places leave only the units in
    the last place by which sums in another order move a value across a rounding boundary (the smallest
    configuration agrees to 1e-7; the largest difference over all cuts of the three configurations is 8.5e-3)."""
    if not isinstance(ref, Ref):
        ref = Ref(ref)
    got = got.float().cpu()
    err = (got - ref.logits).abs().max().item()
    assert err <= logit_tol(dtype, ref.logits), f"{what}: max error {err:.3e}, allowed {logit_tol(dtype, ref.logits):.3e}"
    if dtype == torch.float32:
        assert torch.equal(got.argmax(-1), ref.logits.argmax(-1)), f"{what}: argmax differs"
    elif ref.rounded is not None:
        scale = ref.rounded.abs().max().item()
        err = (got - ref.rounded).abs().max().item()
        WORST[f"{dtype} vs rounded"] = max(WORST.get(f"{dtype} vs rounded", 0.0), err / scale)
        WORST[f"{dtype} vs plain"] = max(WORST.get(f"{dtype} vs plain", 0.0), (got - ref.logits).abs().max().item() / ref.logits.abs().max().item())
        bound = (BF16_ROUNDED_TOL if dtype == torch.bfloat16 else F16_ROUNDED_TOL) * scale
        assert err <= bound, f"{what}: {err:.3e} from the plain model with the engine's roundings, allowed {bound:.3e}"


def run_cuts(lm, prompt, cuts):
    from machserve_amd.engine import StepEntry
    slot = lm.cache.admit()
    out, i = [], 0
    for c in cuts:
        out.append(lm.step([StepEntry(slot, prompt[i:i + c], list(range(c)))]))
        i += c
    assert i == len(prompt)
    lm.cache.release(slot)
    lm.cache.check()
    return torch.cat(out)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("which", ["A", "B", "C"])
def test_whole_prompts(models, which, dtype):
    lm = engine(models, which, dtype, 16)
    for i, prompt in enumerate(models[which][3]):
        check(run_cuts(lm, prompt, [len(prompt)]), plain_logits(models, which, dtype, i), dtype, f"{which} prompt {i} whole")


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("which", ["A", "B", "C"])
def test_last_32_one_by_one(models, which, dtype):
    lm = engine(models, which, dtype, 16)
    for i, prompt in enumerate(models[which][3]):
        n = len(prompt)
        head = max(0, n - 32)
        cuts = ([head] if head else []) + [1] * (n - head)
        check(run_cuts(lm, prompt, cuts), plain_logits(models, which, dtype, i), dtype, f"{which} prompt {i} decoded")


def changing_cuts(n):
    sizes, out, i = [7, 2, 5, 3, 11, 2, 24, 2, 1, 31, 4], [], 0
    while n > 0:
        c = min(sizes[i % len(sizes)], n)
        if n - c == 1:  # no portion of one token at the end of a prompt unless it is the whole rest
            c = n
        out.append(c)
        n -= c
        i += 1
    return out


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("which", ["A", "B", "C"])
def test_portions_of_changing_size(models, which, dtype):
    lm = engine(models, which, dtype, 16)
    for i, prompt in enumerate(models[which][3]):
        check(run_cuts(lm, prompt, changing_cuts(len(prompt))), plain_logits(models, which, dtype, i), dtype,
              f"{which} prompt {i} in portions")


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("which", ["A", "B", "C"])
def test_mixed_with_page_reuse(models, which, dtype):
    """Requests arrive one after another; every step carries a portion of the newest beside
    one token of each older one.  The pool holds the live requests and no more, so a
    finished request's pages go to the next."""
    from machserve_amd.engine import StepEntry
    d, w, sizes, prompts, _ = models[which]
    ps = PAGE[which]
    seqs = [prompts[i % len(prompts)] for i in range(9)]
    refs = [plain_logits(models, which, dtype, i % len(prompts)) for i in range(9)]
    live_cap = 4
    pages = sum(sorted(-(-len(s) // ps) for s in seqs)[-live_cap:])
    lm = engine(models, which, dtype, pages)
    got = [[] for _ in seqs]
    state = {}  # request -> [slot, fed]
    waiting = list(range(len(seqs)))
    portion = [9, 2, 17, 5]
    step, used = 0, []
    first_pages = None
    while waiting or state:
        while waiting and len(state) < live_cap:
            r = waiting[0]
            need = -(-len(seqs[r]) // ps)
            held = sum(-(-len(seqs[q]) // ps) for q in state)
            if held + need > pages:
                break
            waiting.pop(0)
            state[r] = [lm.cache.admit(), 0]
        entries, order = [], []
        newest = max(state)
        for r, (slot, fed) in sorted(state.items()):
            left = len(seqs[r]) - fed
            if r == newest:
                n = min(portion[step % len(portion)], left)
                if left - n == 1:
                    n = left
            else:
                n = 1
            entries.append(StepEntry(slot, seqs[r][fed:fed + n], list(range(n))))
            order.append((r, n))
        logits = lm.step(entries)
        lm.cache.check()
        k = 0
        for r, n in order:
            got[r].append(logits[k:k + n])
            k += n
            state[r][1] += n
            used.append((r, frozenset(p for p in lm.cache.table(next(iter(lm.cache.groups)), state[r][0]) if p >= 0)))
            if state[r][1] == len(seqs[r]):
                lm.cache.release(state.pop(r)[0])
        step += 1
    lm.cache.check()
    assert all(g.pool.available() == g.pool.num_pages for g in lm.cache.groups.values())
    total_pages = sum(-(-len(s) // ps) for s in seqs)
    assert total_pages > pages, "the trace must need more pages than the pool has"
    owners = {}
    for r, held in used:
        for p in held:
            owners.setdefault(p, set()).add(r)
    assert max(len(o) for o in owners.values()) >= 2, "some page must have served two requests, one after the other"
    for r in range(len(seqs)):
        check(torch.cat(got[r]), refs[r], dtype, f"{which} request {r} mixed")


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("which", ["B", "C"])
def test_a_step_shape_that_recurs_is_replayed_from_its_graph(models, which, dtype):
    """A long prompt fed in equal portions beside two requests that decode: once the step's shape
    has come a few times it runs from a captured graph.  Every replay is compared with
    the plain model, with other steps (another shape, run as it is) in between; and so is the
    same trace with capturing switched off (it differs in rounding only: the captured tables
    are wider, which changes how the keys are cut among waves)."""
    from machserve_amd.engine import StepEntry
    d, w, sizes, prompts, _ = models[which]
    long_i = max(range(len(prompts)), key=lambda i: len(prompts[i]))
    others = [i for i in range(len(prompts)) if i != long_i and len(prompts[i]) >= 9][:2]
    assert len(others) == 2

    def run(use_graphs):
        lm = engine(models, which, dtype, 24)
        lm.step.CAPTURE_AFTER = lm.step.FILLED_CAPTURE_AFTER = lm.step.DECODE_CAPTURE_AFTER = 3
        if not use_graphs:
            lm.step.use_graphs = False
        replays = [0]
        inner = lm.step._run_graph

        def counted(key, *a, **kw):
            replays[0] += key in lm.step._graphs
            return inner(key, *a, **kw)
        lm.step._run_graph = counted
        slots = {i: lm.cache.admit() for i in [long_i] + others}
        fed = {i: 0 for i in slots}
        got = {i: [] for i in slots}
        # the two short ones: all but their last eight tokens at once
        for i in others:
            n = len(prompts[i]) - 8
            got[i].append(lm.step([StepEntry(slots[i], prompts[i][:n], list(range(n)))]))
            fed[i] = n
        portion, step = 7, 0
        while fed[long_i] < len(prompts[long_i]):
            entries, order = [], []
            for i in others:
                if fed[i] < len(prompts[i]):
                    entries.append(StepEntry(slots[i], prompts[i][fed[i]:fed[i] + 1], [0]))
                    order.append((i, 1))
            n = min(portion, len(prompts[long_i]) - fed[long_i])
            entries.append(StepEntry(slots[long_i], prompts[long_i][fed[long_i]:fed[long_i] + n], list(range(n))))
            order.append((long_i, n))
            logits = lm.step(entries)
            k = 0
            for i, m in order:
                got[i].append(logits[k:k + m])
                k += m
                fed[i] += m
            step += 1
        for i in others:  # what is left of the short ones, one by one
            while fed[i] < len(prompts[i]):
                got[i].append(lm.step([StepEntry(slots[i], prompts[i][fed[i]:fed[i] + 1], [0])]))
                fed[i] += 1
        lm.cache.check()
        return {i: torch.cat(got[i]) for i in slots}, replays[0]

    captured, n_replays = run(True)
    plain_run, none = run(False)
    assert n_replays >= 2 and none == 0, "the recurring shape must have been replayed"
    for i in captured:
        check(captured[i], plain_logits(models, which, dtype, i), dtype, f"{which} request {i} with captured steps")
        check(plain_run[i], plain_logits(models, which, dtype, i), dtype, f"{which} request {i} without captured steps")


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("captured", [True, False])
def test_decode_steps_filled_up_to_a_bucket(models, dtype, captured):
    """Three, five, six and seven requests decode side by side: the step is filled up to four or eight
    rows with rows that belong to no request, whose logits are dropped.  Captured at once, or launched as it
    is; every request's logits against the plain model, and the cache consistent afterwards."""
    from machserve_amd.engine import StepEntry
    which = "A"
    d, w, sizes, prompts, _ = models[which]
    seqs = [prompts[i % len(prompts)][:20 + 3 * i] if len(prompts[i % len(prompts)]) >= 20 + 3 * i else prompts[i % len(prompts)]
            for i in range(7)]
    lm = engine(models, which, dtype, 40)
    lm.step.DECODE_CAPTURE_AFTER = 0 if captured else 10 ** 6
    slots = [lm.cache.admit() for _ in seqs]
    got = [[] for _ in seqs]
    fed = []
    for i, sq in enumerate(seqs):  # all but the last four tokens at once
        n = max(1, len(sq) - 4)
        got[i].append(lm.step([StepEntry(slots[i], sq[:n], list(range(n)))]))
        fed.append(n)
    for live in ([0, 1, 2], [0, 1, 2, 3, 4], [1, 2, 3, 4, 5, 6], [0, 1, 2, 3, 4, 5, 6], [6, 5, 4, 3, 2]):
        live = [i for i in live if fed[i] < len(seqs[i])]
        if not live:
            continue
        out = lm.step([StepEntry(slots[i], seqs[i][fed[i]:fed[i] + 1], [0]) for i in live])
        assert out.shape[0] == len(live)
        for k, i in enumerate(live):
            got[i].append(out[k:k + 1])
            fed[i] += 1
    lm.cache.check()
    for i, sq in enumerate(seqs):
        check(torch.cat(got[i]), plain_ref(w, sizes, sq, dtype)[:fed[i]], dtype, f"request {i} in filled decode steps")


# ---------------------------------------------------------------------------- the same four ways through the program

def _four_mode_trace(prompts, page):
    """Steps for ``bin/trace_run`` that replay ``prompts`` four ways (whole; most of it at once and the last 32
    tokens one by one; portions of changing size; mixed with up to four live requests), and for every step
    the (prompt, positions) whose logits it asks for, in the order of the file.  Also the most tokens that
    live requests hold at any time, each request rounded up to the page: the pool is made for that many, so
    the mixed part, which always has its four largest requests live at some time, gets pages that others used."""
    steps, wanted, live, peak = [], {}, {}, 0

    def emit(entries, end=()):
        nonlocal peak
        n = len(steps)
        recs = []
        for rid, i, lo, hi in entries:
            live[rid] = hi
            recs.append({"id": rid, "tokens": prompts[i][lo:hi], "want": list(range(hi - lo))})
            wanted.setdefault(n, []).append((i, lo, hi))
        peak = max(peak, sum(-(-v // page) * page for v in live.values()))
        for rid in end:
            live.pop(rid)
        steps.append({"step": n, "entries": recs, "end": list(end)})

    for i, p in enumerate(prompts):                                   # whole
        emit([(f"w{i}", i, 0, len(p))], [f"w{i}"])
    for i, p in enumerate(prompts):                                   # the last 32 one by one
        head = max(0, len(p) - 32)
        if head:
            emit([(f"d{i}", i, 0, head)])
        for t in range(head, len(p)):
            emit([(f"d{i}", i, t, t + 1)], [f"d{i}"] if t == len(p) - 1 else [])
    for i, p in enumerate(prompts):                                   # portions of changing size
        at = 0
        for c in changing_cuts(len(p)):
            emit([(f"c{i}", i, at, at + c)], [f"c{i}"] if at + c == len(p) else [])
            at += c
    order = [k % len(prompts) for k in range(9)]                      # mixed: a portion of the newest beside one token of each older one
    fed, waiting, portion, k = {}, list(range(len(order))), [9, 2, 17, 5], 0
    while waiting or fed:
        while waiting and len(fed) < 4:
            fed[waiting.pop(0)] = 0
        newest, entries, end = max(fed), [], []
        for r in sorted(fed):
            left = len(prompts[order[r]]) - fed[r]
            n = 1
            if r == newest:
                n = min(portion[k % 4], left)
                n = left if left - n == 1 else n
            entries.append((f"m{r}", order[r], fed[r], fed[r] + n))
            fed[r] += n
            if fed[r] == len(prompts[order[r]]):
                end.append(f"m{r}")
                del fed[r]
        emit(entries, end)
        k += 1
    return steps, wanted, peak


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("which", ["A", "B", "C"])
def test_the_four_ways_through_the_program(models, which, dtype, tmp_path):
    """``bin/trace_run`` itself, fed the four ways of cutting as one stream of steps, with a pool of exactly the
    tokens that are live at the worst moment: every position's logits against the plain model."""
    import json, os, subprocess, sys
    import numpy as np
    d, w, sizes, prompts, _ = models[which]
    page = 64
    steps, wanted, peak = _four_mode_trace(prompts, page)
    total = sum(-(-len(p) // page) * page for p in prompts)
    assert peak < 2 * total, "the pool is far smaller than what the trace writes in all"
    root = os.path.join(os.path.dirname(os.path.abspath(__file__)), "..")
    name = {torch.float32: "float32", torch.bfloat16: "bfloat16", torch.float16: "float16"}[dtype]
    r = subprocess.run([sys.executable, os.path.join(root, "bin", "trace_run"), "--model", d, "--dtype", name, "--out", str(tmp_path),
                        "--max-tokens", str(peak)], input="\n".join(json.dumps(s) for s in steps) + "\n",
                       capture_output=True, text=True, timeout=600)
    assert r.returncode == 0, r.stderr[-2000:]
    assert r.stdout.split() == [t for s in steps for t in ("done", str(s["step"]))]
    V = sizes["vocab"]
    for n, parts in wanted.items():
        got = torch.from_numpy(np.fromfile(tmp_path / f"{n}.f32", dtype="<f4").reshape(-1, V))
        assert got.shape[0] == sum(hi - lo for _, lo, hi in parts)
        at = 0
        for i, lo, hi in parts:
            check(got[at:at + hi - lo], plain_logits(models, which, dtype, i)[lo:hi], dtype, f"{which} step {n} prompt {i} [{lo}, {hi})")
            at += hi - lo


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_the_program_writes_every_layer_s_stream(models, dtype, tmp_path):
    """``bin/trace_run --dump-layers``: the residual stream after the embedding and after every layer at the wanted
    places (crates/mach-model/src/batched.rs:3040-3088 dumps the same points), from the kernels, a prompt portion
    beside decoded tokens of another request; the logits of the same run are those of a run without the dump."""
    import json, os, subprocess, sys
    import numpy as np
    d, w, sizes, prompts, _ = models["C"]
    a, b = prompts[2], prompts[3]                       # 130 and 47 tokens
    steps = [{"step": 0, "entries": [{"id": "a", "tokens": a[:100], "want": []}, {"id": "b", "tokens": b[:46], "want": []}], "end": []},
             {"step": 1, "entries": [{"id": "b", "tokens": b[46:], "want": [0]}, {"id": "a", "tokens": a[100:], "want": [0, 29]}], "end": ["a", "b"]}]
    root = os.path.join(os.path.dirname(os.path.abspath(__file__)), "..")
    name = {torch.float32: "float32", torch.bfloat16: "bfloat16"}[dtype]
    outs = {}
    for how in ("plainly", "dumping"):
        out = tmp_path / how
        cmd = [sys.executable, os.path.join(root, "bin", "trace_run"), "--model", d, "--dtype", name, "--out", str(out), "--max-tokens", "256"]
        if how == "dumping":
            cmd += ["--dump-layers", str(tmp_path / "layers")]
        r = subprocess.run(cmd, input="\n".join(json.dumps(s) for s in steps) + "\n", capture_output=True, text=True, timeout=600)
        assert r.returncode == 0, r.stderr[-2000:]
        outs[how] = np.fromfile(out / "1.f32", dtype="<f4").reshape(3, sizes["vocab"])
    scale = np.abs(outs["plainly"]).max()
    assert np.abs(outs["plainly"] - outs["dumping"]).max() <= (1e-5 if dtype == torch.float32 else 1e-2) * scale
    ww = w if dtype == torch.float32 else {k: v.to(dtype).float() if v.dim() == 2 else v for k, v in w.items()}
    sa, sb = [], []
    P.forward(ww, sizes, a, streams=sa)
    P.forward(ww, sizes, b, streams=sb)
    names = ["embedding"] + [f"layer{i:02d}" for i in range(sizes["layers"])]
    for n, xa, xb in zip(names, sa, sb):
        want = torch.stack([xb[46], xa[100], xa[129]]).numpy()
        got = np.fromfile(tmp_path / "layers" / f"1_{n}.f32", dtype="<f4").reshape(3, sizes["hidden"])
        bound = (2e-5 if dtype == torch.float32 else 3e-2) * (1 + np.abs(want).max())
        assert np.abs(got - want).max() <= bound, f"{n}: {np.abs(got - want).max():.3e}"


def test_zz_report_worst_bfloat16_error():
    print("largest errors of the reduced-precision runs, in units of the logits' scale:", WORST)
