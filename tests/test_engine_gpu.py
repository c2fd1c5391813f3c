"""The engine on the GPU through its entry points: greedy generation, long decoding, the
first tokens of a sequence, the replay program, the command line, sampling, and each part
of a layer alone."""
import json
import os
import subprocess
import sys

import numpy as np
import pytest
import torch

from gpu_util import DEV, assert_close
from plain import qwen2_plain as P
from tiny_configs import CONFIGS, make_model_dir, random_prompt, read_for_plain

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.fixture(scope="module")
def dirs(tmp_path_factory):
    tmp = tmp_path_factory.mktemp("engine_models")
    return {w: make_model_dir(tmp, w) for w in CONFIGS}


def assert_greedy(w, sizes, prompt, generated, dtype, what=""):
    """``generated`` is a greedy continuation of ``prompt``.  32-bit: token for token the plain model's.  bfloat16:
    every token is, given the tokens before it, the plain model's most likely one or within the rounding of it
    (the plain model with the matrices stored in the element type; 3e-2 of the logits' scale in bfloat16, an eighth
    of that in half precision: the bounds of the logit tests), since a near-tie may fall either way."""
    if dtype == "float32":
        assert generated == P.greedy_generate(w, sizes, prompt, len(generated)), what
        return
    stored, near = (torch.bfloat16, 3e-2) if dtype == "bfloat16" else (torch.float16, 3e-2 / 8)
    ww = {k: v.to(stored).float() if v.dim() == 2 else v for k, v in w.items()}
    seq = list(prompt)
    for n, tok in enumerate(generated):
        logits = P.forward(ww, sizes, seq)[-1]
        assert logits[tok] >= logits.max() - near * logits.abs().max(), f"{what}: generated token {n} is not near the most likely one"
        seq.append(tok)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16", "float16"])
@pytest.mark.parametrize("which", ["A", "B", "C"])
def test_greedy_generation_through_the_entry_point(dirs, which, dtype):
    import machserve_amd
    w, sizes = read_for_plain(dirs[which])
    prompts = [random_prompt(n, sizes["vocab"], 70 + n) for n in (1, 9, 40, 33)]
    got = machserve_amd.generate(dirs[which], prompts, max_new=12, dtype=dtype, page_size=16, capacity=3,
                                 max_batch_tokens=24)
    for p, g in zip(prompts, got):
        assert len(g) == 12
        assert_greedy(w, sizes, p, g, dtype, f"{which} prompt of {len(p)}")


ODD = {
    "architectures": ["Qwen2ForCausalLM"], "model_type": "qwen2", "hidden_size": 88, "num_hidden_layers": 2,
    "num_attention_heads": 3, "num_key_value_heads": 1, "head_dim": 80, "intermediate_size": 104, "vocab_size": 333,
    "max_position_embeddings": 128, "rms_norm_eps": 2e-6, "rope_theta": 3000.0, "tie_word_embeddings": True,
    "hidden_act": "silu", "use_sliding_window": False,
}


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_sizes_at_the_edge_of_what_the_kernels_take(tmp_path, dtype):
    """Width, intermediate size and vocabulary that are multiples of 8 only, three heads in one group, a head
    size that fills five sixths of its tile: logits of a prompt in portions against the plain model."""
    from machserve_amd.engine import StepEntry, load_model
    from machserve_amd.weights import write_random_model
    d = write_random_model(dict(ODD), 5, str(tmp_path / "odd"), torch.float32)
    w, sizes = read_for_plain(d)
    if dtype == "bfloat16":
        w = {k: v.to(torch.bfloat16).float() if v.dim() == 2 else v for k, v in w.items()}
    p = random_prompt(50, 333, 8)
    ref = P.forward(w, sizes, p)
    lm = load_model(d, dtype=dtype, device=DEV, page_size=16, num_pages=4)
    slot = lm.cache.admit()
    got = [lm.step([StepEntry(slot, p[:33], list(range(33)))]), lm.step([StepEntry(slot, p[33:35], [0, 1])])]
    got += [lm.step([StepEntry(slot, p[i:i + 1], [0])]) for i in range(35, 50)]
    got = torch.cat(got).float().cpu()
    scale = ref.abs().max().item()
    allowed = 2e-5 + 2e-5 * scale if dtype == "float32" else 3e-2 * scale
    assert (got - ref).abs().max().item() <= allowed


@pytest.mark.parametrize("key,value,said", [("intermediate_size", 100, "intermediate size = 100"), ("hidden_size", 92, "width = 92"),
                                            ("head_dim", 72, "head size 72")])
def test_sizes_the_kernels_do_not_take_are_refused_when_the_model_is_built(tmp_path, key, value, said):
    from machserve_amd.engine import load_model
    from machserve_amd.weights import write_random_model
    d = write_random_model(dict(ODD, **{key: value}), 5, str(tmp_path / "refused"), torch.float32)
    with pytest.raises(Exception, match=said):
        load_model(d, dtype="bfloat16", device=DEV, page_size=16, num_pages=4)


def test_rows_too_wide_for_the_norm_and_the_rotation_are_refused_when_the_part_is_built():
    """The norm and the rotation kernels hold a row in a block's LDS: a wider one is refused when the part is built,
    with the size, not at the first step."""
    from machserve_amd.config import AttentionSpec, NormSpec, RotarySpec
    from machserve_amd.parts import MIXERS, NORMS
    rt = _runtime(torch.bfloat16)
    most = rt.ops._core.ms_max_norm_width()
    NORMS.build(NormSpec("rmsnorm", most, 1e-6), rt)
    with pytest.raises(Exception, match=f"width {most + 8}"):
        NORMS.build(NormSpec("rmsnorm", most + 8, 1e-6), rt)
    with pytest.raises(Exception, match=r"head size = 15360"):
        MIXERS.build(AttentionSpec("attention", 1024, 100, 10, 128, RotarySpec("rotary", 128, 1e4)), rt)


def test_eos_stops_generation(dirs):
    import machserve_amd
    w, sizes = read_for_plain(dirs["A"])
    p = random_prompt(11, 512, 3)
    full = P.greedy_generate(w, sizes, p, 10)
    got = machserve_amd.generate(dirs["A"], [p], max_new=10, dtype="float32", eos=full[4])
    assert got[0] == full[:full.index(full[4]) + 1]


def test_generation_under_page_pressure_equals_roomy_generation(dirs):
    """Pages run out, the youngest request is preempted and recomputed; tokens do not change."""
    from machserve_amd.engine import Engine
    from machserve_amd.sampling import SamplingParams
    prompts = [random_prompt(n, 1000, 90 + n) for n in (40, 50, 45)]

    def run(pages, dtype):
        eng = Engine.from_dir(dirs["B"], dtype=dtype, page_size=32, num_pages=pages, capacity=3, max_batch_tokens=64)
        ids = [eng.add(p, 30, SamplingParams(temperature=0.8, top_p=0.95, seed=5 + i)) for i, p in enumerate(prompts)]
        done = eng.run()
        eng.loaded.cache.check()
        return [done[i].generated for i in ids], sum(done[i].preemptions for i in ids)
    roomy, n0 = run(12, "float32")
    tight, n1 = run(5, "float32")
    assert n0 == 0 and n1 > 0 and roomy == tight


@pytest.mark.parametrize("which,dtype,seed", [("B", "float32", 1), ("B", "float32", 2), ("B", "float32", 3), ("A", "float32", 4),
                                              ("C", "float32", 5), ("A", "bfloat16", 6), ("B", "bfloat16", 7), ("C", "bfloat16", 8)])
def test_random_arrivals_under_page_pressure_equal_the_plain_model(dirs, which, dtype, seed):
    """Requests of random lengths arrive at random steps in an engine with few slots, few pages and a small
    token budget: portions, decoded tokens, ends, slot and page reuse and preemptions in whatever order the
    seed brings; every request's greedy tokens against the plain model, and no page lost at the end."""
    import random
    from machserve_amd.engine import Engine
    w, sizes = read_for_plain(dirs[which])
    rnd_ = random.Random(seed)
    reqs = [(random_prompt(rnd_.randrange(1, 90), sizes["vocab"], 100 * seed + i), rnd_.randrange(1, 18)) for i in range(12)]
    eng = Engine.from_dir(dirs[which], dtype=dtype, page_size=16, num_pages=10, capacity=4,
                          max_batch_tokens=rnd_.choice([24, 40, 64]))
    arrivals = sorted(rnd_.randrange(0, 60) for _ in reqs)
    ids, step, nxt = [], 0, 0
    while nxt < len(reqs) or eng.has_work():
        while nxt < len(reqs) and (arrivals[nxt] <= step or not eng.has_work()):
            ids.append(eng.add(reqs[nxt][0], reqs[nxt][1]))
            nxt += 1
        (eng.step_pipelined if step % 3 else eng.step)()
        step += 1
        assert step < 5000
    done = eng.scheduler.finished
    eng.loaded.cache.check()
    assert not eng.loaded.cache.live_requests()
    for rid, (prompt, max_new) in zip(ids, reqs):
        assert len(done[rid].generated) == max_new
        assert_greedy(w, sizes, prompt, done[rid].generated, dtype, f"request {rid} ({len(prompt)} tokens, {max_new} new)")
    print(f"seed {seed}: {step} steps, {sum(done[r].preemptions for r in ids)} preemptions")
    _PREEMPTIONS[(which, dtype, seed)] = sum(done[r].preemptions for r in ids)


_PREEMPTIONS = {}


def test_the_random_arrivals_did_run_out_of_pages():
    """The seeds above are there for what happens when pages run out: over all of them (at least those that ran in
    this process before this test) some request must have been preempted, and in both element types."""
    if not _PREEMPTIONS:
        pytest.skip("the random-arrival tests did not run in this process")
    for dtype in {k[1] for k in _PREEMPTIONS}:
        assert sum(n for k, n in _PREEMPTIONS.items() if k[1] == dtype) > 0, f"no preemption in any {dtype} run: {_PREEMPTIONS}"


def test_captured_steps_are_dropped_and_captured_again(dirs):
    """The step function keeps two captured steps at most while requests come and go, so that steps of one, two and
    four rows take turns: the graph of a shape that returns has been dropped meanwhile and is captured again, also
    while steps are launched ahead.  Every request's tokens against the plain model."""
    from machserve_amd.engine import Engine
    w, sizes = read_for_plain(dirs["A"])
    eng = Engine.from_dir(dirs["A"], dtype="float32", page_size=16, num_pages=40, capacity=4, max_batch_tokens=64)
    st = eng.loaded.step
    st.MAX_GRAPHS, st.DECODE_CAPTURE_AFTER = 2, 1
    captures, dropped = [], []
    inner = st._run_graph

    def watched(key, *a, **kw):
        if key not in st._graphs:
            captures.append(key)
        before = set(st._graphs)
        out = inner(key, *a, **kw)
        dropped.extend(before - set(st._graphs))
        return out
    st._run_graph = watched
    # (arrival step, prompt length, new tokens): one request alone, then two, then four, then two, one, and four again
    plan = [(0, 5, 70), (8, 9, 40), (16, 7, 12), (16, 11, 12), (52, 6, 30), (52, 8, 30), (52, 4, 30)]
    reqs = [(at, random_prompt(n, sizes["vocab"], 300 + i), m) for i, (at, n, m) in enumerate(plan)]
    ids, step, nxt = [], 0, 0
    while nxt < len(reqs) or eng.has_work():
        while nxt < len(reqs) and reqs[nxt][0] <= step:
            ids.append(eng.add(reqs[nxt][1], reqs[nxt][2]))
            nxt += 1
        eng.step_pipelined()
        step += 1
        assert step < 2000
    assert len(st._graphs) <= 2 and 0 < st.graph_bytes() <= 2 * 4 * (sizes["vocab"] * 4 + 4096)
    again = [k for k in set(captures) if captures.count(k) > 1]
    assert dropped and again, f"a shape must have been dropped and captured again ({len(captures)} captures, {len(dropped)} dropped)"
    done = eng.scheduler.finished
    for rid, (_, prompt, max_new) in zip(ids, reqs):
        assert done[rid].generated == P.greedy_generate(w, sizes, prompt, max_new), f"request {rid}"
    eng.loaded.cache.check()
    # the same limit by bytes: with room for one step's results only, one captured step is kept
    st.MAX_GRAPHS, st.MAX_GRAPH_BYTES = 256, 1
    for n in (3, 9):
        eng.add(random_prompt(n, sizes["vocab"], 400 + n), 20)
    eng.run()
    assert len(st._graphs) == 1


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_steps_launched_ahead_give_what_steps_one_at_a_time_give(dirs, dtype):
    """Engine.run launches a decode step before the samples of the step before have reached the
    host (they are taken on the device).  Same tokens and log probabilities as with one step at a
    time, with requests that end at different steps, one that arrives in the middle, and an
    end-of-sequence token that is only seen one step late."""
    from machserve_amd.engine import Engine
    from machserve_amd.sampling import SamplingParams
    prompts = [random_prompt(n, 1000, 20 + n) for n in (37, 8, 21, 14)]
    max_new = [40, 17, 29, 23]

    def run(pipelined, eos=None):
        eng = Engine.from_dir(dirs["B"], dtype=dtype, page_size=32, num_pages=16, capacity=4, max_batch_tokens=48)
        eng.loaded.step.DECODE_CAPTURE_AFTER = 0  # every decode step from a captured graph: nothing is launched ahead without one
        fed_from_device = [0]
        launch = eng.loaded.step.launch_decode

        def counted(*a, **kw):
            fed_from_device[0] += (len(a) > 5 and a[5] is not None) or kw.get("after") is not None
            return launch(*a, **kw)
        eng.loaded.step.launch_decode = counted
        ids = [eng.add(p, m, SamplingParams(temperature=0.8, top_k=60, top_p=0.9, seed=2 + i), eos=eos)
               for i, (p, m) in enumerate(zip(prompts[:3], max_new))]
        n = 0
        while eng.has_work():
            eng.step_pipelined() if pipelined else eng.step()
            n += 1
            if n == 9:
                ids.append(eng.add(prompts[3], max_new[3], SamplingParams(seed=1), eos=eos))
        eng.loaded.cache.check()
        done = eng.scheduler.finished
        return [(done[i].generated, done[i].finish_reason, done[i].logprobs) for i in ids], fed_from_device[0]

    one_by_one, n0 = run(False)
    ahead, n1 = run(True)
    assert n0 == 0 and n1 > 20
    assert ahead == one_by_one
    eos = one_by_one[0][0][11]
    a, _ = run(False, eos)
    b, n2 = run(True, eos)
    assert a == b and n2 > 0 and a[0][1] == "stop" and len(a[0][0]) <= 12


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_long_decoding(dirs, dtype):
    """One step of 8 tokens, then 400 single tokens across many pages: every position against
    the plain model."""
    from machserve_amd.engine import StepEntry, load_model
    w, sizes = read_for_plain(dirs["A"])
    toks = random_prompt(250, 512, 8)
    ww = w if dtype == torch.float32 else {k: v.to(torch.bfloat16).float() if v.dim() == 2 else v for k, v in w.items()}
    ref = P.forward(ww, sizes, toks)
    lm = load_model(dirs["A"], dtype=dtype, device=DEV, page_size=16, num_pages=16)
    slot = lm.cache.admit()
    out = [lm.step([StepEntry(slot, toks[:8], list(range(8)))])]
    for t in toks[8:]:
        out.append(lm.step([StepEntry(slot, [t], [0])]))
    got = torch.cat(out).float().cpu()
    scale = ref.abs().max().item()
    allowed = 2e-5 + 2e-5 * scale if dtype == torch.float32 else 3e-2 * scale
    assert (got - ref).abs().max().item() <= allowed


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_long_context(tmp_path, dtype):
    """A 5,000-token prompt in portions of 1,500 and then decoded tokens: positions in the
    thousands (rotation angles, dozens of pages, split keys in the decode kernel), checked at
    the ends of the portions and at every decoded position."""
    from machserve_amd.engine import StepEntry, load_model
    from machserve_amd.weights import write_random_model
    from tiny_configs import TINY_A
    raw = dict(TINY_A, max_position_embeddings=8192, rope_theta=1000000.0)
    d = write_random_model(raw, 4, str(tmp_path / "long"))
    w, sizes = read_for_plain(d)
    ww = w if dtype == torch.float32 else {k: v.to(torch.bfloat16).float() if v.dim() == 2 else v for k, v in w.items()}
    toks = random_prompt(5010, 512, 6)
    ref = P.forward(ww, sizes, toks)
    lm = load_model(d, dtype=dtype, device=DEV, page_size=64, num_pages=80)
    slot = lm.cache.admit()
    got, where, i = [], [], 0
    for c in (1500, 1500, 1500, 500):
        want = [0, c // 2, c - 1]
        got.append(lm.step([StepEntry(slot, toks[i:i + c], want)]))
        where += [i + k for k in want]
        i += c
    for j in range(5000, 5010):
        got.append(lm.step([StepEntry(slot, [toks[j]], [0])]))
        where.append(j)
    got = torch.cat(got).float().cpu()
    scale = ref.abs().max().item()
    allowed = 1e-4 + 1e-4 * scale if dtype == torch.float32 else 3e-2 * scale
    # 32-bit: the angle pos * freq itself carries 2^-24 * 5000 of relative error at these positions,
    # five times the bound used at short positions
    err = (got - ref[where]).abs().max().item()
    assert err <= allowed, f"max error {err:.3e}, allowed {allowed:.3e}"


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("which", ["A", "B", "C"])
def test_first_tokens_of_a_sequence(dirs, which, dtype):
    """Positions 0, 1, 2 alone and together: a one-token prompt, and the first rows of a portion."""
    from machserve_amd.engine import StepEntry, load_model
    w, sizes = read_for_plain(dirs[which])
    ww = w if dtype == torch.float32 else {k: v.to(torch.bfloat16).float() if v.dim() == 2 else v for k, v in w.items()}
    lm = load_model(dirs[which], dtype=dtype, device=DEV, page_size=16, num_pages=8)
    toks = random_prompt(3, sizes["vocab"], 2)
    ref = P.forward(ww, sizes, toks)
    allowed = 2e-5 + 2e-5 * ref.abs().max().item() if dtype == torch.float32 else 3e-2 * ref.abs().max().item()
    for cuts in ([1, 1, 1], [3], [1, 2], [2, 1]):
        slot, i, out = lm.cache.admit(), 0, []
        for c in cuts:
            out.append(lm.step([StepEntry(slot, toks[i:i + c], list(range(c)))]))
            i += c
        lm.cache.release(slot)
        assert (torch.cat(out).float().cpu() - ref).abs().max().item() <= allowed, cuts


def test_wanted_places_select_rows(dirs):
    from machserve_amd.engine import StepEntry, load_model
    lm = load_model(dirs["B"], dtype="float32", device=DEV, page_size=32, num_pages=8)
    a, b = lm.cache.admit(), lm.cache.admit()
    ta, tb = random_prompt(10, 1000, 1), random_prompt(6, 1000, 2)
    full = lm.step([StepEntry(a, ta, list(range(10))), StepEntry(b, tb, list(range(6)))])
    lm.cache.release(a), lm.cache.release(b)
    a, b = lm.cache.admit(), lm.cache.admit()
    some = lm.step([StepEntry(a, ta, [9, 0]), StepEntry(b, tb, []), ])
    assert some.shape == (2, 1000)
    assert torch.equal(some[0], full[9]) and torch.equal(some[1], full[0])
    assert lm.step([StepEntry(b, [5], [])]) is None


def test_trace_run_program(dirs, tmp_path):
    """bin/trace_run as a user runs it: JSON lines in, <step>.f32 files and 'done' lines out."""
    w, sizes = read_for_plain(dirs["A"])
    a, b = random_prompt(37, 512, 1), random_prompt(20, 512, 2)
    steps = [
        {"step": 0, "entries": [{"id": "a", "tokens": a[:30], "want": [0, 29]}], "end": []},
        {"step": 1, "entries": [{"id": "a", "tokens": a[30:32], "want": []}, {"id": "b", "tokens": b[:18], "want": [17]}], "end": []},
        {"step": 2, "entries": [{"id": "b", "tokens": b[18:], "want": [0, 1]}], "end": ["b"]},
        {"step": 3, "entries": [{"id": "a", "tokens": a[32:], "want": [4]}], "end": ["a"]},
    ]
    out = tmp_path / "out"
    for dtype in ("float32", "bfloat16"):
        r = subprocess.run([sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model", dirs["A"], "--dtype", dtype,
                            "--out", str(out / dtype), "--max-tokens", "128"],
                           input="\n".join(json.dumps(s) for s in steps) + "\n", capture_output=True, text=True, timeout=600)
        assert r.returncode == 0, r.stderr
        assert r.stdout.split() == ["done", "0", "done", "1", "done", "2", "done", "3"]
        ra, rb = P.forward(w, sizes, a), P.forward(w, sizes, b)
        want = {0: ra[[0, 29]], 1: rb[[17]], 2: rb[[18, 19]], 3: ra[[36]]}
        tolr = 2e-5 if dtype == "float32" else 4e-2
        for s, ref in want.items():
            got = torch.from_numpy(np.fromfile(out / dtype / f"{s}.f32", dtype="<f4").reshape(-1, 512))
            assert got.shape == ref.shape
            assert (got - ref).abs().max() <= tolr * (1 + ref.abs().max())


def test_trace_run_takes_a_step_only_after_the_one_before_is_done(dirs, tmp_path):
    """The sender writes a step, waits for its 'done' line, and only then writes the next; a request is left
    out of a step and goes on later; the input's end ends the program with 0."""
    w, sizes = read_for_plain(dirs["B"])
    a, b = random_prompt(70, 1000, 3), random_prompt(9, 1000, 4)
    steps = [
        {"step": 0, "entries": [{"id": "a", "tokens": a[:40], "want": [39]}], "end": []},
        {"step": 1, "entries": [{"id": "b", "tokens": b, "want": [8]}], "end": ["b"]},
        {"step": 2, "entries": [{"id": "a", "tokens": a[40:68], "want": [0]}], "end": []},
        {"step": 3, "entries": [{"id": "a", "tokens": a[68:], "want": [0, 1]}], "end": ["a"]},
    ]
    out = tmp_path / "out"
    proc = subprocess.Popen([sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model", dirs["B"], "--dtype", "float32",
                             "--out", str(out), "--max-tokens", "128"], stdin=subprocess.PIPE, stdout=subprocess.PIPE,
                            stderr=subprocess.DEVNULL, text=True)
    try:
        for s in steps:
            proc.stdin.write(json.dumps(s) + "\n")
            proc.stdin.flush()
            assert proc.stdout.readline().split() == ["done", str(s["step"])]
            assert (out / f"{s['step']}.f32").exists(), "a step's logits are there when its 'done' line is"
        proc.stdin.close()
        assert proc.wait(timeout=60) == 0
    finally:
        if proc.poll() is None:
            proc.kill()
    ra, rb = P.forward(w, sizes, a), P.forward(w, sizes, b)
    want = {0: ra[[39]], 1: rb[[8]], 2: ra[[40]], 3: ra[[68, 69]]}
    for s, ref in want.items():
        got = torch.from_numpy(np.fromfile(out / f"{s}.f32", dtype="<f4").reshape(-1, 1000))
        assert got.shape == ref.shape
        assert (got - ref).abs().max() <= 2e-5 * (1 + ref.abs().max())


def test_command_line(dirs, tmp_path):
    w, sizes = read_for_plain(dirs["A"])
    p = random_prompt(7, 512, 9)
    r = subprocess.run([sys.executable, "-m", "machserve_amd", "--model", dirs["A"], "--dtype", "f32", "--prompt-ids",
                        ",".join(map(str, p)), "--max-new", "5", "--tpp", "16", "--json"],
                       capture_output=True, text=True, cwd=ROOT, timeout=600)
    assert r.returncode == 0, r.stderr
    rec = json.loads(r.stdout.strip().splitlines()[-1])
    assert rec["generated"] == P.greedy_generate(w, sizes, p, 5) and rec["finish_reason"] == "length"
    cfg = tmp_path / "cfg.json"
    cfg.write_text(json.dumps(CONFIGS["B"]))
    r = subprocess.run([sys.executable, "-m", "machserve_amd", "--random-config", str(cfg), "--weights-seed", "1",
                        "--dtype", "f32", "--prompt-ids", "1,2,3", "--prompt-ids", "4,5", "--max-new", "4", "--tpp", "32",
                        "--temperature", "0.7", "--seed", "3"], capture_output=True, text=True, cwd=ROOT, timeout=600)
    assert r.returncode == 0, r.stderr
    assert [len(l.split()) for l in r.stdout.strip().splitlines()] == [4, 4]


# ---------------------------------------------------------------------------- each part alone

def _runtime(dtype):
    from machserve_amd.kernels import get_ops
    from machserve_amd.parts import Runtime
    return Runtime(torch.device(DEV), dtype, get_ops(dtype, DEV))


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_norm_part_alone(dtype):
    from machserve_amd.config import NormSpec
    from machserve_amd.parts import NORMS
    part = NORMS.build(NormSpec("rmsnorm", 200, 1e-5), _runtime(dtype))
    assert [(d.name, d.shape, d.role) for d in part.tensor_decls()] == [("weight", (200,), "vector")]
    w = 1 + 0.1 * torch.randn(200)
    part.load({"weight": w.to(DEV)})
    from machserve_amd.parts import ResidualStream
    x = torch.randn(9, 200) * 3
    assert_close(part.forward(ResidualStream(x.to(DEV), part.rt.ops)), P.rms_norm(x, w, 1e-5), dtype)


def test_rotary_part_alone():
    """The position-encoding part owns the table of inverse frequencies, made in 32-bit as
    1 / theta^(2j / head_dim) (crates/mach-model/src/ref_model.rs:636-643)."""
    from machserve_amd.config import RotarySpec
    from machserve_amd.parts import POSITION_ENCODINGS
    for hd, theta in ((16, 1e4), (64, 1e6), (48, 5e4)):
        part = POSITION_ENCODINGS.build(RotarySpec("rotary", hd, theta), _runtime(torch.float32))
        assert part.tensor_decls() == []
        want = P.rope_angles(torch.tensor([1]), hd, theta)[0]   # the angles at position 1 are the frequencies
        assert torch.equal(part.rotary_inv_freq().cpu(), want)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_feed_forward_part_alone(dtype):
    from machserve_amd.config import GatedMlpSpec
    from machserve_amd.parts import FEED_FORWARDS
    part = FEED_FORWARDS.build(GatedMlpSpec("gated_mlp", 72, 200), _runtime(dtype))
    t = {"gate.weight": torch.randn(200, 72) * 0.2, "up.weight": torch.randn(200, 72) * 0.2, "down.weight": torch.randn(72, 200) * 0.1}
    t = {k: v.to(dtype) for k, v in t.items()}
    part.load({k: v.to(DEV) for k, v in t.items()})
    from machserve_amd.parts import ResidualStream
    for rows in (11, 100):  # few rows: partial sums for the next reader; many: added in the product's epilogue
        h = torch.randn(rows, 72).to(dtype)
        x = torch.randn(rows, 72)
        stream = ResidualStream(x.to(DEV).clone(), part.rt.ops)
        part.forward(h.to(DEV), stream, None)
        assert stream.deferred is not None, "the product waits for the stream's next reader"
        ref = x + P.swiglu(h.float(), t["gate.weight"].float(), t["up.weight"].float(), t["down.weight"].float())
        assert_close(stream.value(), ref, dtype)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("window,shared", [(None, False), (7, False), (None, True)])
def test_attention_part_alone(dtype, window, shared):
    """The mixer with its own cache manager: a portion, then single tokens, against the plain
    attention block over the whole sequence.  With ``shared`` a second layer reads the first
    layer's cache and writes none."""
    from machserve_amd.cache import CacheManager, DeviceCache
    from machserve_amd.config import AttentionSpec, RotarySpec
    from machserve_amd.engine.step import StepEntry, StepFunction
    from machserve_amd.parts import MIXERS, ResidualStream
    rt = _runtime(dtype)
    H, KV, hd, d, T = 6, 2, 32, 80, 45
    names = {k: k for k in ("q.weight", "k.weight", "v.weight", "o.weight", "q.bias", "k.bias", "v.bias")}
    spec = AttentionSpec("attention", d, H, KV, hd, RotarySpec("rotary", hd, 1e4), window=window, tensors=names)
    part = MIXERS.build(spec, rt)
    g = torch.Generator().manual_seed(5)
    t = {"q.weight": torch.randn(H * hd, d, generator=g) * 0.1, "k.weight": torch.randn(KV * hd, d, generator=g) * 0.1,
         "v.weight": torch.randn(KV * hd, d, generator=g) * 0.1, "o.weight": torch.randn(d, H * hd, generator=g) * 0.1,
         "q.bias": torch.randn(H * hd, generator=g) * 0.1, "k.bias": torch.randn(KV * hd, generator=g) * 0.1,
         "v.bias": None}
    t = {k: (v.to(dtype) if v is not None and v.dim() == 2 else v) for k, v in t.items()}
    part.load({k: (v.to(DEV) if v is not None else None) for k, v in t.items()})
    parts = [part]
    if shared:
        spec2 = AttentionSpec("attention", d, H, KV, hd, RotarySpec("rotary", hd, 1e4), kv_source=0, tensors=names)
        part2 = MIXERS.build(spec2, rt)
        assert [dd.name for dd in part2.tensor_decls()] == ["q.weight", "o.weight", "q.bias"]
        part2.load({k: (v.to(DEV) if v is not None else None) for k, v in t.items()})
        parts.append(part2)
    cache = CacheManager([p.cache_request() for p in parts], 16, 8, 2)
    dc = DeviceCache(cache, dtype, rt.device)
    for i, p in enumerate(parts):
        p.bind_cache(dc.binding(i))

    class OneLayer:  # just enough of a model for the step function's context builder
        vocab = 100
        class spec:
            max_positions = 1000
        def attention_rows_per_token(self):
            return [H // KV]
    sf = StepFunction(OneLayer(), cache, rt)
    h = torch.randn(T, d, generator=g).to(dtype)
    slot = cache.admit()
    outs = [torch.zeros(T, d, device=DEV) for _ in parts]
    i = 0
    for c in [20, 1, 1, 13, 1, 9]:
        cache.extend(slot, c)
        ctx = sf.build_context([StepEntry(slot, [0] * c, [])])
        for p, o in zip(parts, outs):
            stream = ResidualStream(torch.zeros(c, d, device=DEV), rt.ops)
            p.forward(h[i:i + c].to(DEV).contiguous(), stream, ctx)
            o[i:i + c] = stream.value()
        cache.commit(slot, c)
        i += c
    w = {"p.q_proj.weight": t["q.weight"].float(), "p.k_proj.weight": t["k.weight"].float(), "p.v_proj.weight": t["v.weight"].float(),
         "p.o_proj.weight": t["o.weight"].float(), "p.q_proj.bias": t["q.bias"], "p.k_proj.bias": t["k.bias"]}
    sizes = {"heads": H, "kv_heads": KV, "head_dim": hd, "theta": 1e4}
    ref = P.attention_block(h.float(), w, "p.", torch.arange(T), sizes, window)
    for o in outs:
        assert_close(o, ref, dtype)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_block_arrangement_alone(dtype):
    """The pre-norm arrangement around the stream, built from the registries with parts of its own
    sizes: x += mixer(norm(x)); x += feed_forward(norm(x))
    (crates/mach-model/src/batched.rs:3180-3200).  A portion and single tokens against the plain parts."""
    from machserve_amd.cache import CacheManager, DeviceCache
    from machserve_amd.config import AttentionSpec, GatedMlpSpec, LayerSpec, NormSpec, RotarySpec
    from machserve_amd.engine.step import StepEntry, StepFunction
    from machserve_amd.parts import BLOCKS, ResidualStream
    rt = _runtime(dtype)
    H, KV, hd, d, I, T, eps = 3, 1, 48, 112, 136, 40, 1e-5
    names = {k: k for k in ("q.weight", "k.weight", "v.weight", "o.weight", "q.bias", "k.bias", "v.bias")}
    layer = LayerSpec("prenorm", AttentionSpec("attention", d, H, KV, hd, RotarySpec("rotary", hd, 5e4), tensors=names),
                      GatedMlpSpec("gated_mlp", d, I), NormSpec("rmsnorm", d, eps), NormSpec("rmsnorm", d, eps))
    block = BLOCKS.get(layer.block)(layer, rt)   # the arrangement builds its own parts from the layer's spec
    n1, mixer, n2, ff = block.parts()
    assert (mixer, ff, n1, n2) == (block.mixer, block.feed_forward, block.mixer_norm, block.feed_forward_norm)
    g = torch.Generator().manual_seed(11)
    r = lambda *s: torch.randn(*s, generator=g) * 0.1
    t = {"q.weight": r(H * hd, d), "k.weight": r(KV * hd, d), "v.weight": r(KV * hd, d), "o.weight": r(d, H * hd),
         "q.bias": r(H * hd), "k.bias": None, "v.bias": r(KV * hd),
         "gate.weight": r(I, d), "up.weight": r(I, d), "down.weight": r(d, I), "n1": 1 + r(d), "n2": 1 + r(d)}
    t = {k: (v.to(dtype) if v is not None and v.dim() == 2 else v) for k, v in t.items()}
    dev = {k: (v.to(DEV) if v is not None else None) for k, v in t.items()}
    mixer.load(dev), ff.load(dev), n1.load({"weight": dev["n1"]}), n2.load({"weight": dev["n2"]})
    cache = CacheManager([block.cache_request()], 16, 4, 1)
    dc = DeviceCache(cache, dtype, rt.device)
    block.bind_cache(dc.binding(0))

    class OneLayer:
        vocab = 100
        class spec:
            max_positions = 1000
        def attention_rows_per_token(self):
            return [H // KV]
    sf = StepFunction(OneLayer(), cache, rt)
    x = torch.randn(T, d, generator=g)
    slot = cache.admit()
    out = torch.zeros(T, d)
    i = 0
    for c in [17, 1, 2, 1, 19]:
        cache.extend(slot, c)
        ctx = sf.build_context([StepEntry(slot, [0] * c, [])])
        stream = ResidualStream(x[i:i + c].to(DEV).clone(), rt.ops)
        block.forward(stream, ctx)
        out[i:i + c] = stream.value().cpu()
        cache.commit(slot, c)
        i += c
    f = {k: (v.float() if v is not None else None) for k, v in t.items()}
    w = {"p.q_proj.weight": f["q.weight"], "p.k_proj.weight": f["k.weight"], "p.v_proj.weight": f["v.weight"],
         "p.o_proj.weight": f["o.weight"], "p.q_proj.bias": f["q.bias"], "p.v_proj.bias": f["v.bias"]}
    sizes = {"heads": H, "kv_heads": KV, "head_dim": hd, "theta": 5e4}
    y = x + P.attention_block(P.rms_norm(x, f["n1"], eps), w, "p.", torch.arange(T), sizes)
    y = y + P.swiglu(P.rms_norm(y, f["n2"], eps), f["gate.weight"], f["up.weight"], f["down.weight"])
    assert_close(out, y, dtype)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("tied", [True, False, None])
def test_embedding_and_head_parts_alone(dtype, tied):
    """Rows of the table in 32-bit, and logits from the head tensor or, tied, from the table
    (crates/mach-model/src/loader.rs:1025-1033); a vocabulary and a width that are no powers of two."""
    from machserve_amd.config import EmbeddingSpec, HeadSpec
    from machserve_amd.parts.model import Embedding, Head
    rt = _runtime(dtype)
    V, d = 333, 88
    table, head_w = (torch.randn(V, d) * 0.3).to(dtype), (torch.randn(V, d) * 0.3).to(dtype)
    emb = Embedding(EmbeddingSpec(V, d), rt)
    emb.load({"weight": table.to(DEV)})
    head = Head(HeadSpec(V, d, tied), rt, emb)
    assert [dd.name for dd in head.tensor_decls()] == ([] if tied is True else ["weight"])
    head.load({"weight": head_w.to(DEV)} if tied is False else {"weight": None} if tied is None else {})
    toks = torch.tensor([0, 332, 17, 17, 200], dtype=torch.int32)
    x = emb.forward(toks.to(DEV))
    assert x.dtype == torch.float32 and torch.equal(x.cpu(), table.float()[toks.long()])
    h = (torch.randn(5, d)).to(dtype)
    logits = head.forward(h.to(DEV))
    used = head_w if tied is False else table
    assert logits.dtype == torch.float32
    assert_close(logits, P.linear(h.float(), used.float()), dtype)
