"""Schedules at the far ends of what the engine runs: dozens of requests decoding side by side (the buckets of 48 and
64 rows, every product in the tiled kernel, the norm that adds many pending planes, split keys, sampling of all
rows inside the captured step), one request tens of thousands of positions long, and temperature sampling end to
end; every logit and every token against the plain model
(crates/mach-model/tests/continuous.rs:80-97, 393-427: the engine's tokens equal one request's alone)."""
import pytest
import torch

from gpu_util import DEV
from plain import qwen2_plain as P
from tiny_configs import CONFIGS, TINY_A, make_model_dir, random_prompt, read_for_plain, sharpen_attention

pytestmark = pytest.mark.gpu


def _stored(w, dtype):
    return w if dtype == torch.float32 else {k: v.to(dtype).float() if v.dim() == 2 else v for k, v in w.items()}


def _bound(dtype, scale):
    return 2e-5 + 2e-5 * scale if dtype == torch.float32 else (3e-2 if dtype == torch.bfloat16 else 3e-2 / 8) * scale


def _many_decoders(lm, w, sizes, dtype, n, lengths, steps, vocab, captured):
    """``n`` requests with prompts of ``lengths`` (in turn) are fed, a few prompts a step; then all decode side by side
    for ``steps`` steps with given tokens, and once more with the sampler inside the step.  Every logit of the
    prompts' ends and of the decoded positions against the plain model."""
    from machserve_amd.engine import StepEntry
    if captured:
        lm.step.DECODE_CAPTURE_AFTER = 0   # capture at once: the test has only a few steps
    seqs = [random_prompt(lengths[i % len(lengths)] + steps + 1, vocab, 500 + i) for i in range(n)]
    fed = [lengths[i % len(lengths)] for i in range(n)]
    ww = _stored(w, dtype)
    refs = [P.forward(ww, sizes, s) for s in seqs]
    slots = [lm.cache.admit() for _ in range(n)]
    worst = 0.0

    def compare(logits, who):
        nonlocal worst
        got = logits.float().cpu()
        for row, r in enumerate(who):
            ref = refs[r][fed[r] - 1]
            err = (got[row] - ref).abs().max().item()
            assert err <= _bound(dtype, ref.abs().max().item()), f"request {r} at position {fed[r] - 1}: error {err:.3e}"
            worst = max(worst, err)

    for first in range(0, n, 8):   # prompts, eight requests a step
        who = list(range(first, min(first + 8, n)))
        compare(lm.step([StepEntry(slots[r], seqs[r][:fed[r]], [fed[r] - 1]) for r in who]), who)
    everyone = list(range(n))
    for _ in range(steps):
        entries = [StepEntry(slots[r], [seqs[r][fed[r]]], [0]) for r in everyone]
        for r in everyone:
            fed[r] += 1
        compare(lm.step(entries), everyone)
    if captured:
        assert lm.step.use_graphs and any(len(k[0]) >= n and set(k[0]) == {1} for k in lm.step._graphs), \
            "the decode steps must have run from a captured graph"
        # one more step with the sampler inside the captured step: greedy rows and rows at a temperature
        temps = [0.0 if r % 2 == 0 else 0.7 for r in everyone]
        states = [1000 + r for r in everyone]
        entries = [StepEntry(slots[r], [seqs[r][fed[r]]], [0]) for r in everyone]
        for r in everyone:
            fed[r] += 1
        out = lm.step.decode_and_sample(entries, temps, [0] * n, [1.0] * n, states)
        assert out is not None, "a decode step of plain sampling takes the captured path"
        tokens, _ = out
        for r in everyone:
            ref = refs[r][fed[r] - 1]
            if dtype == torch.float32 and temps[r] > 0:
                # The draw is the first token whose cumulated probability exceeds u * total (crates/mach-model/src/
                # sampling.rs:1259-1270).  Over a flat row of 150,000 tokens the 32-bit sums of the kernel's segments and of
                # a walk in index order differ in rounding by more than one token's share, so the token is held to the
                # target in mass: the target lies within 1e-4 of the total of the token's own interval.  (Token for token
                # equality is held at the small vocabularies, where a token's share is far above the rounding.)
                u, _ = P.next_uniform(states[r])
                p = torch.exp((ref.double() - ref.double().max()) / temps[r])
                cum, total = torch.cumsum(p, 0), p.sum().item()
                tok = tokens[r]
                assert cum[tok].item() > u * total - 1e-4 * total and (cum[tok] - p[tok]).item() <= u * total + 1e-4 * total, \
                    f"request {r}: token {tok} covers {((cum[tok] - p[tok]) / total).item():.6f}..{(cum[tok] / total).item():.6f}, u = {u:.6f}"
                if vocab <= 4096:
                    want, _ = P.sample(ref.numpy(), temps[r], 0, 1.0, states[r])
                    assert tok == want, f"request {r}: sampled {tok}, the plain draw is {want}"
            elif temps[r] == 0:
                assert ref[tokens[r]] >= ref.max() - _bound(dtype, ref.abs().max().item()), f"request {r}: greedy token {tokens[r]}"
    else:
        assert not lm.step._graphs
    for s in slots:
        lm.cache.release(s)
    lm.cache.check()
    return worst


@pytest.mark.parametrize("captured", [False, True])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("n", [40, 64])
def test_dozens_of_requests_decode_side_by_side_tiny(tmp_path, n, dtype, captured):
    from machserve_amd.engine import load_model
    d = make_model_dir(tmp_path, "B")
    w, sizes = read_for_plain(d)
    lm = load_model(d, dtype=dtype, device=DEV, page_size=16, num_pages=n * 4 + 8, max_requests=n, use_graphs=captured)
    _many_decoders(lm, w, sizes, dtype, n, (1, 7, 15, 16, 17, 30, 33, 40), 6, sizes["vocab"], captured)


@pytest.mark.parametrize("captured", [False, True])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_dozens_of_requests_decode_side_by_side_at_real_layer_sizes(dtype, captured):
    """The layer sizes of Qwen2.5-0.5B with two layers: the path that the benchmark's 64-request point runs on."""
    from machserve_amd.config import config_from_dict
    from machserve_amd.engine import load_model
    from machserve_amd.weights import random_tensor_dict
    raw = {"architectures": ["Qwen2ForCausalLM"], "model_type": "qwen2", "num_hidden_layers": 2, "max_position_embeddings": 4096,
           "rms_norm_eps": 1e-6, "rope_theta": 1000000.0, "hidden_act": "silu", "hidden_size": 896, "num_attention_heads": 14,
           "num_key_value_heads": 2, "intermediate_size": 4864, "vocab_size": 151936, "tie_word_embeddings": True}
    cfg = config_from_dict(raw)
    tensors = random_tensor_dict(cfg, 3)
    n = 64 if captured else 40
    lm = load_model(config=cfg, tensors=tensors, dtype=dtype, device=DEV, page_size=64, num_pages=n + 4, max_requests=n,
                    use_graphs=captured)
    _many_decoders(lm, tensors, P.sizes_from_config(raw), dtype, n, (1, 2, 3, 5, 8), 6, cfg.vocab_size, captured)


@pytest.mark.parametrize("n", [12, 24])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_a_dozen_or_two_requests_decode_side_by_side_at_real_layer_sizes(dtype, n):
    """9 to 32 requests at the 0.5B layer sizes: the narrow output and down projections and the wide gate/up product
    run in the tiled kernel with K cut over blocks there, and the norms between them add the slices."""
    from machserve_amd.config import config_from_dict
    from machserve_amd.engine import load_model
    from machserve_amd.weights import random_tensor_dict
    raw = {"architectures": ["Qwen2ForCausalLM"], "model_type": "qwen2", "num_hidden_layers": 2, "max_position_embeddings": 4096,
           "rms_norm_eps": 1e-6, "rope_theta": 1000000.0, "hidden_act": "silu", "hidden_size": 896, "num_attention_heads": 14,
           "num_key_value_heads": 2, "intermediate_size": 4864, "vocab_size": 151936, "tie_word_embeddings": True}
    cfg = config_from_dict(raw)
    tensors = random_tensor_dict(cfg, 5)
    from machserve_amd.kernels import get_ops
    ops = get_ops(dtype)
    assert ops._tiled(n, 896, 896) and ops._tiled(n, 896, 4864) and ops._tiled(n, 2 * 4864, 896)
    lm = load_model(config=cfg, tensors=tensors, dtype=dtype, device=DEV, page_size=64, num_pages=n + 4, max_requests=n, use_graphs=True)
    _many_decoders(lm, tensors, P.sizes_from_config(raw), dtype, n, (1, 2, 3, 5, 8), 6, cfg.vocab_size, True)


@pytest.mark.timeout(400)   # the plain model walks 20,000 rows of four heads one by one
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_twenty_thousand_positions(tmp_path, dtype):
    """One request of 20,480 prompt tokens in portions of 4,096 and then eight decoded tokens: block tables 320
    pages wide, dozens of key splits, rotation angles of tens of thousands of radians.  Logits at the portions'
    ends and middles and at every decoded position."""
    from machserve_amd.engine import StepEntry, load_model
    from machserve_amd.weights import write_random_model
    raw = dict(TINY_A, max_position_embeddings=32768, rope_theta=1000000.0)
    d = write_random_model(raw, 4, str(tmp_path / "long"))
    w, sizes = read_for_plain(d)
    toks = random_prompt(20488, 512, 6)
    ref = P.forward(_stored(w, dtype), sizes, toks)
    lm = load_model(d, dtype=dtype, device=DEV, page_size=64, num_pages=324)
    slot = lm.cache.admit()
    got, where, i = [], [], 0
    for c in (4096,) * 5:
        want = [0, c // 2, c - 1]
        got.append(lm.step([StepEntry(slot, toks[i:i + c], want)]))
        where += [i + k for k in want]
        i += c
    for j in range(20480, 20488):
        got.append(lm.step([StepEntry(slot, [toks[j]], [0])]))
        where.append(j)
    got = torch.cat(got).float().cpu()
    scale = ref.abs().max().item()
    # 32-bit: the same bound as at 5,000 positions (sums over thousands of keys in another order)
    allowed = 1e-4 + 1e-4 * scale if dtype == torch.float32 else 3e-2 * scale
    err = (got - ref[where]).abs().max().item()
    assert err <= allowed, f"max error {err:.3e}, allowed {allowed:.3e}"
    if dtype == torch.float32:
        assert torch.equal(got.argmax(-1), ref[where].argmax(-1))


@pytest.mark.parametrize("which", ["A", "B"])
def test_temperature_sampling_through_the_entry_point_equals_the_plain_draws(tmp_path, which):
    """``generate`` with a temperature and top-p in 32-bit: every request's tokens are the CPU mirror's draws
    (crates/mach-model/src/sampling.rs:1169-1274) on the plain model's logits, seed by seed."""
    import machserve_amd
    d = make_model_dir(tmp_path, which)
    w, sizes = read_for_plain(d)
    prompts = [random_prompt(n, sizes["vocab"], 300 + n) for n in (4, 21, 35)]
    got = machserve_amd.generate(d, prompts, max_new=6, dtype="float32", temperature=0.8, top_p=0.9, seed=41, page_size=16,
                                 capacity=3, max_batch_tokens=32)
    for i, (p, g) in enumerate(zip(prompts, got)):
        seq, state = list(p), 41 + i
        for n, tok in enumerate(g):
            want, state = P.sample(P.forward(w, sizes, seq)[-1].numpy(), 0.8, 0, 0.9, state)
            assert tok == want, f"request {i}, token {n}: the engine drew {tok}, the plain model's draw is {want}"
            seq.append(tok)
    greedy = machserve_amd.generate(d, prompts, max_new=6, dtype="float32", page_size=16)
    assert greedy != got, "the test must tell a draw from the most likely token"


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("which", ["A", "B"])
def test_a_step_of_any_mix_that_samples_inside_the_step(tmp_path, which, dtype):
    """``step_and_sample``: portions of prompts beside decoded tokens, some rows greedy and some drawn at a temperature
    with top-k and top-p, a portion that samples nothing in between; captured at its first coming and replayed with other
    tokens.  The same tokens and log-probabilities as the sampler's kernel gives on the logits of ``__call__`` in a second
    model of the same weights, step after step (the sampled tokens are fed to both, so their caches stay alike)."""
    from machserve_amd.engine import StepEntry, load_model
    d = make_model_dir(tmp_path, which)
    sizes = read_for_plain(d)[1]
    a = load_model(d, dtype=dtype, device=DEV, page_size=16, num_pages=40, max_requests=4)
    b = load_model(d, dtype=dtype, device=DEV, page_size=16, num_pages=40, max_requests=4)
    b.step.FILLED_CAPTURE_AFTER = 0   # the same filled sizes, hence the same kernels on the same shapes: the same logits bit by bit
    ops = a.rt.ops
    prompts = [random_prompt(n, sizes["vocab"], 700 + n) for n in (40, 23, 9, 31)]
    sa, sb = [a.cache.admit() for _ in prompts], [b.cache.admit() for _ in prompts]
    fed = [0] * 4
    state = [11, 12, 13, 14]
    # (request, tokens of it in this step, sampled?) per step; request 0 comes in three portions
    plan = [[(0, 17, False), (1, 23, True)],
            [(0, 16, False), (1, 1, True), (2, 9, True)],
            [(0, 7, True), (1, 1, True), (2, 1, True), (3, 31, True)],
            [(0, 17, False), (1, 23, True)]]   # the first step's shape again, replayed: other requests, other tokens
    temp, top_k, top_p = [0.0, 0.9, 0.7, 0.0], [0, 0, 5, 0], [1.0, 0.8, 1.0, 1.0]
    assert a.step.step_and_sample([StepEntry(sa[0], [1], [0]), StepEntry(sa[1], [2], [0])], [0.0, 0.0], [0, 0], [1.0, 1.0], [1, 2]) is None, \
        "plain decoding is not this path's"
    for i, step in enumerate(plan):
        if i == 3:   # new requests in the slots of 0 and 1
            for r in (0, 1):
                a.cache.release(sa[r]), b.cache.release(sb[r])
                sa[r], sb[r], fed[r] = a.cache.admit(), b.cache.admit(), 0
                prompts[r] = random_prompt(len(prompts[r]), sizes["vocab"], 800 + r)
        ea, eb, who = [], [], []
        for r, n, sampled in step:
            toks = prompts[r][fed[r]:fed[r] + n]
            assert len(toks) == n
            ea.append(StepEntry(sa[r], toks, [n - 1] if sampled else []))
            eb.append(StepEntry(sb[r], toks, [n - 1] if sampled else []))
            fed[r] += n
            if sampled:
                who.append(r)
                prompts[r] = prompts[r] + [0]     # room for the token that is sampled now
        got = a.step.step_and_sample(ea, [temp[r] for r in who], [top_k[r] for r in who], [top_p[r] for r in who],
                                     [state[r] for r in who], capture_now=True)
        assert got is not None, f"step {i} must take the path"
        logits = b.step(eb)
        tok, lp = ops.sample(logits, torch.tensor([temp[r] for r in who], device=DEV), torch.tensor([top_k[r] for r in who], dtype=torch.int32, device=DEV),
                             torch.tensor([top_p[r] for r in who], device=DEV), torch.tensor([state[r] for r in who], dtype=torch.int64, device=DEV))
        assert got[0] == tok.cpu().tolist(), f"step {i}: tokens {got[0]} against {tok.cpu().tolist()}"
        assert (torch.tensor(got[1]) - lp.cpu()).abs().max().item() <= 1e-6, f"step {i}: log-probabilities"
        for r, t in zip(who, got[0]):
            prompts[r][fed[r]] = t
            state[r] += 100
        a.cache.check(), b.cache.check()
    filled = [k for k in a.step._graphs if k[0] == "filled, sampled"]
    assert len(filled) == 3, f"{len(filled)} graphs: the fourth step ran from the first one's"


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("which", ["A", "B", "C"])
def test_steps_of_any_mix_run_from_graphs_of_shared_sizes(tmp_path, which, dtype):
    """Prompts of many lengths, alone and beside requests that decode, each step filled up to a size that many steps
    share and run from the captured graph of that size: fewer graphs than steps, and every logit the plain model's.
    The rows that fill a step up belong to nobody; the cache is consistent afterwards."""
    from machserve_amd.engine import StepEntry, load_model
    d = make_model_dir(tmp_path, which)
    w, sizes = read_for_plain(d)
    ww = _stored(w, dtype)
    lm = load_model(d, dtype=dtype, device=DEV, page_size=16, num_pages=40, max_requests=4)
    lm.step.FILLED_CAPTURE_AFTER = 0   # every step that can be filled up runs from a graph, captured at its first coming
    limit = CONFIGS[which]["max_position_embeddings"]
    lengths = [n for n in (3, 17, 18, 30, 33, 47, 64, 65, 100, 127, 130, 200) if n + 12 <= limit]
    seqs = [random_prompt(n + 12, sizes["vocab"], 900 + n) for n in lengths]
    refs = [P.forward(ww, sizes, s) for s in seqs]
    steps = 0

    def compare(logits, rows):
        got = logits.float().cpu()
        assert got.shape[0] == len(rows)
        for k, (r, pos) in enumerate(rows):
            ref = refs[r][pos]
            err = (got[k] - ref).abs().max().item()
            assert err <= _bound(dtype, ref.abs().max().item()), f"request {r} ({lengths[r]} tokens) at position {pos}: error {err:.3e}"

    decoding = {}   # request -> [slot, fed]
    for r, n in enumerate(lengths):
        # the new prompt, whole, beside one token of each request that decodes (at most two of them)
        slot = lm.cache.admit()
        entries, rows = [StepEntry(slot, seqs[r][:n], [0, n - 1])], [(r, 0), (r, n - 1)]
        for q, (s_, fed) in decoding.items():
            entries.append(StepEntry(s_, [seqs[q][fed]], [0]))
            rows.append((q, fed))
            decoding[q][1] += 1
        compare(lm.step(entries), rows)
        steps += 1
        decoding[r] = [slot, n]
        for q in [q for q, (s_, fed) in decoding.items() if fed >= lengths[q] + 10 or len(decoding) > 2][:1]:
            lm.cache.release(decoding.pop(q)[0])
        lm.cache.check()
    filled = [k for k in lm.step._graphs if k[0] == "filled"]
    assert filled and len(filled) < steps, f"{len(filled)} graphs of shared sizes for {steps} steps"
    for s_, _ in decoding.values():
        lm.cache.release(s_)
    assert all(g.pool.available() == g.pool.num_pages for g in lm.cache.groups.values())


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("head_dim,heads,kv", [(64, 6, 2), (128, 32, 2)])
def test_prompts_of_one_size_from_one_graph_at_head_sizes_64_and_128(tmp_path, dtype, head_dim, heads, kv):
    """At head size 64 the q/k/v product of a step of many rows rotates by a table of the rows' angles that the step's
    layers share (at 128 the rotation kernel works the angles out itself).  Prompts of several lengths that are filled up to one size run from one captured graph: the
    table is made inside the graph, from the positions of the step at hand (captured from the first prompt's, every
    later prompt's rows beyond the first one's length would be rotated by the angles of the rows that filled the first
    step up).  Every position's logits against the plain model."""
    from machserve_amd.engine import StepEntry, load_model
    from machserve_amd.weights import write_random_model
    raw = {"architectures": ["Qwen2ForCausalLM"], "model_type": "qwen2", "hidden_size": 200, "num_hidden_layers": 2,
           "num_attention_heads": heads, "num_key_value_heads": kv, "head_dim": head_dim, "intermediate_size": 160, "vocab_size": 512,
           "max_position_embeddings": 512, "rms_norm_eps": 1e-5, "rope_theta": 10000.0, "tie_word_embeddings": False,
           "hidden_act": "silu", "attention_bias": True}
    d = write_random_model(raw, 11, str(tmp_path / "m"))
    sharpen_attention(d, 3.0)                        # so that a wrong angle shows in the logits
    w, sizes = read_for_plain(d)
    ww = _stored(w, dtype)
    lm = load_model(d, dtype=dtype, device=DEV, page_size=64, num_pages=12, max_requests=2)
    assert lm.rt.ops.qkv_rope_takes(320, heads, kv, head_dim, 200) == (head_dim == 64)
    bound = 3e-2 if dtype == torch.bfloat16 else 3e-2 / 8
    lm.step.FILLED_CAPTURE_AFTER = 0
    tables, make_table = [], lm.rt.ops.rope_table
    lm.rt.ops.rope_table = lambda *a: (tables.append(1), make_table(*a))[1]
    for n in (260, 301, 276, 258, 318, 310):         # all of them filled up to 320 rows
        prompt = random_prompt(n, 512, 300 + n)
        ref = P.forward(ww, sizes, prompt)
        slot = lm.cache.admit()
        got = lm.step([StepEntry(slot, prompt, list(range(n)))]).float().cpu()
        lm.cache.release(slot)
        err = (got - ref).abs().max().item()
        assert err <= bound * ref.abs().max().item(), f"a prompt of {n} tokens: error {err:.3e} of {ref.abs().max().item():.3f}"
    filled = [k for k in lm.step._graphs if k[0] == "filled"]
    assert len(filled) == 1, "the prompts shared one captured graph"
    # both layers rotate by one table: one for the run that warms the capture up and one inside the graph, none later
    assert len(tables) == (2 if head_dim == 64 else 0), f"{len(tables)} tables of angles were made"


def test_warm_up_captures_the_sizes_that_prompts_will_come_in(tmp_path):
    """After ``Engine.warm_up`` the first prompt of a length is replayed from a graph captured before any request came,
    and the tokens are the plain model's."""
    from machserve_amd.engine import Engine
    d = make_model_dir(tmp_path, "B")
    w, sizes = read_for_plain(d)
    eng = Engine.from_dir(d, dtype="float32", page_size=16, num_pages=40, capacity=2, max_batch_tokens=256)
    n = eng.warm_up([16, 32, 48, 64, 128, 192, 256])
    assert n >= 12 and not eng.loaded.cache.live_requests()
    known = set(eng.loaded.step._graphs)
    replayed = []
    inner = eng.loaded.step._run_graph

    def counted(key, *a, **kw):
        replayed.append(key in known)
        return inner(key, *a, **kw)
    eng.loaded.step._run_graph = counted
    for length in (100, 37, 150, 64):
        prompt = random_prompt(length, sizes["vocab"], 40 + length)
        assert eng.generate([prompt], max_new=3) == [P.greedy_generate(w, sizes, prompt, 3)]
    assert replayed and replayed[0] and sum(replayed) >= 4, "the prompts' steps must have run from the graphs of the warm-up"


@pytest.mark.timeout(300)
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
def test_long_prompts_at_head_size_64(tmp_path, dtype):
    """A head size of 64 and block tables that allow thousands of keys: in the two-byte libraries the prompt's portions
    run in the attention kernel of 32-row tiles (blocks of 128 flat rows, four key groups, tiles straight into LDS).
    A prompt of 3,000 tokens in portions that end inside tiles and blocks, beside a second request that arrives
    later, then decoded tokens; logits at the portions' first, middle and last rows and at every decoded position."""
    from machserve_amd.engine import StepEntry, load_model
    from machserve_amd.weights import write_random_model
    raw = {"architectures": ["Qwen2ForCausalLM"], "model_type": "qwen2", "hidden_size": 320, "num_hidden_layers": 2,
           "num_attention_heads": 6, "num_key_value_heads": 2, "head_dim": 64, "intermediate_size": 328, "vocab_size": 900,
           "max_position_embeddings": 8192, "rms_norm_eps": 1e-6, "rope_theta": 1000000.0, "tie_word_embeddings": False,
           "hidden_act": "silu", "use_sliding_window": False}
    d = write_random_model(raw, 7, str(tmp_path / "hd64"))
    w, sizes = read_for_plain(d)
    ww = _stored(w, dtype)
    a, b = random_prompt(3008, 900, 11), random_prompt(708, 900, 12)
    ra, rb = P.forward(ww, sizes, a), P.forward(ww, sizes, b)
    lm = load_model(d, dtype=dtype, device=DEV, page_size=32, num_pages=130, max_requests=2)
    assert lm.model.attention_rows_per_block() == (64 if dtype == torch.float32 else 128)
    sa, sb = lm.cache.admit(), lm.cache.admit()
    got_a, got_b, where_a, where_b = [], [], [], []
    ia = ib = 0
    for ca, cb in ((1100, 0), (900, 0), (611, 333), (389, 367)):
        entries = [StepEntry(sa, a[ia:ia + ca], [0, ca // 2, ca - 1])]
        if cb:
            entries.append(StepEntry(sb, b[ib:ib + cb], [0, cb - 1]))
        out = lm.step(entries)
        got_a.append(out[:3]), where_a.extend([ia, ia + ca // 2, ia + ca - 1])
        if cb:
            got_b.append(out[3:]), where_b.extend([ib, ib + cb - 1])
        ia, ib = ia + ca, ib + cb
    for j in range(8):
        out = lm.step([StepEntry(sa, [a[ia + j]], [0]), StepEntry(sb, [b[ib]], [0])] if j == 0 else [StepEntry(sa, [a[ia + j]], [0])])
        got_a.append(out[:1]), where_a.append(ia + j)
        if j == 0:
            got_b.append(out[1:]), where_b.append(ib)
    for got, ref, where in ((torch.cat(got_a), ra, where_a), (torch.cat(got_b), rb, where_b)):
        got = got.float().cpu()
        scale = ref.abs().max().item()
        allowed = {torch.float32: 1e-4 + 1e-4 * scale, torch.bfloat16: 3e-2 * scale, torch.float16: 3e-2 / 8 * scale}[dtype]
        err = (got - ref[where]).abs().max().item()
        assert err <= allowed, f"max error {err:.3e}, allowed {allowed:.3e}"


@pytest.mark.parametrize("head_dim", [None, 64])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_yarn_on_the_gpu(tmp_path, dtype, head_dim):
    """YaRN through the kernels (crates/mach-model/src/ref_model.rs:636-704): the scaled frequencies go to the rotation
    kernels as their table, the factors to the attention kernels as the scores' scale; a prompt in portions, then
    decoded tokens (the fused decode kernel rotates by the same table), positions far beyond the original context."""
    from machserve_amd.engine import StepEntry, load_model
    from machserve_amd.weights import write_random_model
    raw = dict(TINY_A, max_position_embeddings=1024,
               rope_scaling={"type": "yarn", "factor": 8.0, "original_max_position_embeddings": 64, "mscale": 0.8, "mscale_all_dim": 0.707})
    if head_dim:  # a head size at which the q/k/v product of the prompt's portions rotates in its own epilogue (two-byte elements)
        raw["head_dim"] = head_dim
    d = write_random_model(raw, 3, str(tmp_path / "yarn"))
    sharpen_attention(d, 4.0)
    w, sizes = read_for_plain(d)
    toks = random_prompt(620, 512, 5)
    ref = P.forward(_stored(w, dtype), sizes, toks)
    lm = load_model(d, dtype=dtype, device=DEV, page_size=16, num_pages=40, max_requests=1)
    slot = lm.cache.admit()
    got = [lm.step([StepEntry(slot, toks[:400], list(range(400)))]), lm.step([StepEntry(slot, toks[400:600], list(range(200)))])]
    got += [lm.step([StepEntry(slot, toks[i:i + 1], [0])]) for i in range(600, 620)]
    got = torch.cat(got).float().cpu()
    scale = ref.abs().max().item()
    err = (got - ref).abs().max().item()
    assert err <= _bound(dtype, scale), f"max error {err:.3e}"
