"""The plain implementation is pinned by what fixes it beside the reference's text: library
routines it must reduce to, invariants, and the vectors the reference's own tests hold.
Each check is chosen so that a plausible mistake fails it."""
import math

import numpy as np
import pytest
import torch
import torch.nn.functional as F

from plain import qwen2_plain as P
from tiny_configs import make_model_dir, random_prompt, read_for_plain


def rnd(*shape, seed=0, dtype=torch.float64):
    return torch.randn(*shape, generator=torch.Generator().manual_seed(seed), dtype=dtype)


def test_rms_norm_is_the_library_routine():
    x, w = rnd(5, 48, seed=1), 1 + 0.1 * rnd(48, seed=2)
    for eps in (1e-6, 1e-2):
        assert torch.allclose(P.rms_norm(x, w, eps), F.rms_norm(x, (48,), w, eps), atol=1e-12)
    # eps inside the root: with unit weight the mean square of the output is ms / (ms + eps)
    x = 1e-2 * rnd(3, 64, seed=3)
    ms = (x * x).mean(-1)
    y = P.rms_norm(x, torch.ones(64, dtype=torch.float64), 1e-4)
    assert torch.allclose((y * y).mean(-1), ms / (ms + 1e-4), atol=1e-12)
    # (a norm that added eps outside the root, or used 1 + w, fails the two checks above)


def test_linear_is_the_library_routine():
    x, w, b = rnd(4, 10, seed=4), rnd(7, 10, seed=5), rnd(7, seed=6)
    assert torch.allclose(P.linear(x, w, b), F.linear(x, w, b))
    assert torch.allclose(P.linear(x, w, torch.zeros(7, dtype=torch.float64)), P.linear(x, w))


def test_rope_identity_at_zero_and_norms():
    """pos 0 is the identity (crates/mach-model/src/ref_model.rs:1446) and every pair keeps its norm."""
    x = rnd(6, 3, 32, seed=7)
    assert torch.equal(P.rope(x[:1], torch.tensor([0]), 1e4), x[:1])
    y = P.rope(x, torch.arange(6) * 37, 1e4)
    half = 16
    assert torch.allclose(x[..., :half] ** 2 + x[..., half:] ** 2, y[..., :half] ** 2 + y[..., half:] ** 2, atol=1e-10)
    assert not torch.allclose(x[1:], y[1:], atol=1e-3)


def test_rope_is_rotate_half_and_not_interleaved():
    hd, theta = 16, 1e4
    x, pos = rnd(4, 2, hd, seed=8), torch.tensor([0, 3, 17, 200])
    inv = 1.0 / theta ** (torch.arange(0, hd, 2, dtype=torch.float64) / hd)
    ang = pos[:, None].double() * inv[None, :]
    cos, sin = torch.cat([ang.cos(), ang.cos()], -1)[:, None], torch.cat([ang.sin(), ang.sin()], -1)[:, None]
    rot_half = torch.cat([-x[..., hd // 2:], x[..., :hd // 2]], -1)
    assert torch.allclose(P.rope(x, pos, theta), x * cos + rot_half * sin, atol=1e-12)
    # adjacent pairing (2j, 2j+1) agrees at pos 0 only (crates/mach-model/src/ref_model.rs:1413)
    xi = x.reshape(4, 2, hd // 2, 2)
    a, b = xi[..., 0], xi[..., 1]
    inter = torch.stack([a * ang.cos()[:, None] - b * ang.sin()[:, None], a * ang.sin()[:, None] + b * ang.cos()[:, None]], -1).reshape(4, 2, hd)
    assert torch.allclose(inter[0], P.rope(x, pos, theta)[0])
    assert not torch.allclose(inter[1:], P.rope(x, pos, theta)[1:], atol=1e-3)


def test_yarn_frequencies_and_factors_are_the_reference_s_own_vectors():
    """The numbers that the reference's tests hold for YaRN (crates/mach-model/src/ref_model.rs:1330-1560): with head
    size 64, theta 10,000, factor 40 over 4,096 positions, beta 32 / 1 the ramp runs from pair 10 to pair 23 (clamped to
    the head size, not to the number of pairs); pair 0 keeps its own frequency, pair 31 has 1 / factor of it; the
    factor on cosines and sines is mscale(1.0) / mscale(0.707); the scores' scale has mscale(0.707)^2.  And the
    formulas written out once more, in 64-bit, as the library that the checkpoints come from writes them."""
    import math
    yarn = P.yarn_of({"type": "yarn", "factor": 40.0, "original_max_position_embeddings": 4096, "mscale": 1.0, "mscale_all_dim": 0.707})
    assert yarn == (40.0, 4096, 32.0, 1.0, 1.0, 0.707)
    assert P.yarn_of(None) is None and P.yarn_of({"type": "linear", "factor": 2.0}) is None
    f = P.rope_freq(64, 1e4, torch.float64, yarn)
    assert abs(f[0].item() - 1.0) < 1e-12 and abs(f[31].item() - 1.0 / (40.0 * 1e4 ** (62 / 64))) < 1e-15
    dim, base, factor, orig = 64, 1e4, 40.0, 4096.0
    corr = lambda rot: dim * math.log(orig / (rot * 2 * math.pi)) / (2 * math.log(base))
    low, high = max(math.floor(corr(32.0)), 0), min(math.ceil(corr(1.0)), dim - 1)
    assert (low, high) == (10, 23)
    for d in range(32):
        extra = 1.0 / base ** (2 * d / dim)
        mask = 1.0 - min(max((d - low) / (high - low), 0.0), 1.0)
        want = extra / factor * (1 - mask) + extra * mask
        assert abs(f[d].item() - want) <= 1e-12 * want, d
    assert torch.equal(P.rope_freq(64, 1e4, torch.float64, None), 1.0 / torch.pow(torch.tensor(1e4, dtype=torch.float64), torch.arange(0, 64, 2, dtype=torch.float64) / 64))
    ln = math.log(40.0)
    assert abs(P.yarn_attention_factor(yarn) - (0.1 * ln + 1) / (0.1 * 0.707 * ln + 1)) < 1e-12
    assert P.yarn_attention_factor(yarn[:4] + (0.707, 0.707)) == 1.0 and P.yarn_attention_factor(None) == 1.0
    m = 0.1 * 0.707 * ln + 1
    assert abs(P.attn_scale(192, yarn) - m * m / math.sqrt(192)) < 1e-12
    assert P.attn_scale(192, yarn[:5] + (0.0,)) == 1 / math.sqrt(192) and P.attn_scale(64) == 0.125
    # rotation with the factor: every pair's norm grows by it, position 0 is the identity times it
    x = rnd(3, 2, 64, seed=21)
    y = P.rope(x, torch.tensor([0, 5, 9000]), 1e4, yarn)
    af = P.yarn_attention_factor(yarn)
    assert torch.allclose(y[0], x[0] * af) and torch.allclose((y[..., :32] ** 2 + y[..., 32:] ** 2), (x[..., :32] ** 2 + x[..., 32:] ** 2) * af * af)


def test_rope_scores_depend_on_distance_only():
    q, k = rnd(1, 1, 32, seed=9), rnd(1, 1, 32, seed=10)
    def score(p, s, theta=1e6):
        return (P.rope(q, torch.tensor([p]), theta) * P.rope(k, torch.tensor([s]), theta)).sum()
    assert abs(score(50, 47) - score(1003, 1000)) < 1e-9
    assert abs(score(50, 47) - score(47, 50)) > 1e-3   # a wrong sign of the rotation would be symmetric here


def test_attention_is_the_library_routine():
    T, H, KV, hd = 19, 6, 2, 16
    q, k, v = rnd(T, H, hd, seed=11), rnd(T, KV, hd, seed=12), rnd(T, KV, hd, seed=13)
    g = H // KV
    ke, ve = k.repeat_interleave(g, dim=1), v.repeat_interleave(g, dim=1)  # head h reads kv head h // g
    ref = F.scaled_dot_product_attention(q.transpose(0, 1), ke.transpose(0, 1), ve.transpose(0, 1), is_causal=True)
    assert torch.allclose(P.attention(q, k, v), ref.transpose(0, 1), atol=1e-12)
    # KV = H is ordinary multi-head attention; a tiling (h % KV) instead of h // g fails the check above
    # one token attends to itself only
    assert torch.allclose(P.attention(q[:1], k[:1], v[:1]), v[:1].repeat_interleave(g, dim=1))


def test_attention_window():
    T, H, KV, hd = 30, 2, 1, 8
    q, k, v = rnd(T, H, hd, seed=14), rnd(T, KV, hd, seed=15), rnd(T, KV, hd, seed=16)
    assert torch.allclose(P.attention(q, k, v, window=T), P.attention(q, k, v))
    assert torch.allclose(P.attention(q, k, v, window=1), v.repeat_interleave(2, dim=1))
    W = 5
    mask = torch.tril(torch.ones(T, T, dtype=torch.bool)) & ~torch.tril(torch.ones(T, T, dtype=torch.bool), -W)
    ref = F.scaled_dot_product_attention(q.transpose(0, 1), k.repeat_interleave(2, 1).transpose(0, 1),
                                         v.repeat_interleave(2, 1).transpose(0, 1), attn_mask=mask)
    assert torch.allclose(P.attention(q, k, v, window=W), ref.transpose(0, 1), atol=1e-12)


def test_swiglu_activation_is_on_the_gate():
    x, g, u, d = rnd(3, 12, seed=17), rnd(20, 12, seed=18), rnd(20, 12, seed=19), rnd(12, 20, seed=20)
    ref = F.linear(F.silu(F.linear(x, g)) * F.linear(x, u), d)
    assert torch.allclose(P.swiglu(x, g, u, d), ref, atol=1e-12)
    assert not torch.allclose(P.swiglu(x, u, g, d), ref, atol=1e-3)


@pytest.mark.parametrize("which", ["A", "B", "C"])
def test_whole_sequence_equals_token_by_token(tmp_path, which):
    """The whole-sequence form against a loop over positions with growing key and value lists,
    the form of tools/ref_llama.py:89-125 (which adds the q/k/v biases)."""
    d = make_model_dir(tmp_path, which)
    w, sizes = read_for_plain(d)
    w = {k: v.double() for k, v in w.items()}
    toks = random_prompt(50 if which == "C" else 12, sizes["vocab"], 3)
    whole = P.forward(w, sizes, toks, torch.float64)
    H, KV, hd = sizes["heads"], sizes["kv_heads"], sizes["head_dim"]
    windows = P.layer_windows(sizes)
    ks = [[] for _ in range(sizes["layers"])]
    vs = [[] for _ in range(sizes["layers"])]
    head = w["model.embed_tokens.weight"] if sizes["tied"] else w["lm_head.weight"]
    for pos, tok in enumerate(toks):
        x = w["model.embed_tokens.weight"][tok]
        for i in range(sizes["layers"]):
            p = f"model.layers.{i}."
            xn = P.rms_norm(x, w[p + "input_layernorm.weight"], sizes["eps"])
            q = P.linear(xn, w[p + "self_attn.q_proj.weight"], w.get(p + "self_attn.q_proj.bias"))
            k = P.linear(xn, w[p + "self_attn.k_proj.weight"], w.get(p + "self_attn.k_proj.bias"))
            v = P.linear(xn, w[p + "self_attn.v_proj.weight"], w.get(p + "self_attn.v_proj.bias"))
            q = P.rope(q.view(1, H, hd), torch.tensor([pos]), sizes["theta"])[0]
            ks[i].append(P.rope(k.view(1, KV, hd), torch.tensor([pos]), sizes["theta"])[0])
            vs[i].append(v.view(KV, hd))
            lo = 0 if windows[i] is None else max(0, pos - windows[i] + 1)
            kc, vc = torch.stack(ks[i][lo:]), torch.stack(vs[i][lo:])
            o = torch.zeros(H, hd, dtype=torch.float64)
            for h in range(H):
                s = (kc[:, h // (H // KV)] @ q[h]) * hd ** -0.5
                e = torch.exp(s - s.max())
                o[h] = (e[:, None] * vc[:, h // (H // KV)]).sum(0) / e.sum()
            x = x + P.linear(o.reshape(-1), w[p + "self_attn.o_proj.weight"])
            xn = P.rms_norm(x, w[p + "post_attention_layernorm.weight"], sizes["eps"])
            x = x + P.swiglu(xn, w[p + "mlp.gate_proj.weight"], w[p + "mlp.up_proj.weight"], w[p + "mlp.down_proj.weight"])
        logits = P.linear(P.rms_norm(x, w["model.norm.weight"], sizes["eps"]), head)
        assert torch.allclose(logits, whole[pos], atol=1e-10), pos


@pytest.mark.parametrize("which", ["A", "B", "C"])
def test_one_token_reduces_the_whole_model_to_library_routines(tmp_path, which):
    """A sequence of one token at position 0 has no attention to speak of: the softmax over one key is 1,
    the rotation at position 0 is the identity, so a layer's mixer is ``o_proj(v)`` with each value head
    repeated for its group.  What is left is the *composition*, written here with library routines only
    (``F.rms_norm``, ``F.linear``, ``F.silu``): the stream is normalised for each branch's input and never in
    place, the feed-forward reads the stream after the mixer's output was added, ``input_layernorm`` feeds
    the mixer and ``post_attention_layernorm`` the feed-forward, and the final norm comes before the head.
    A post-norm or parallel arrangement, swapped norm weights or a missing final norm fail it."""
    w, sizes = read_for_plain(make_model_dir(tmp_path, which))
    w = {k: v.double() for k, v in w.items()}
    d, g, hd, eps = sizes["hidden"], sizes["heads"] // sizes["kv_heads"], sizes["head_dim"], sizes["eps"]
    head = w["model.embed_tokens.weight"] if sizes["tied"] else w["lm_head.weight"]
    for tok in (0, 7, sizes["vocab"] - 1):
        x = w["model.embed_tokens.weight"][tok]
        for i in range(sizes["layers"]):
            p = f"model.layers.{i}."
            h = F.rms_norm(x, (d,), w[p + "input_layernorm.weight"], eps)
            v = F.linear(h, w[p + "self_attn.v_proj.weight"], w.get(p + "self_attn.v_proj.bias"))
            x = x + F.linear(v.view(-1, hd).repeat_interleave(g, dim=0).reshape(-1), w[p + "self_attn.o_proj.weight"])
            h = F.rms_norm(x, (d,), w[p + "post_attention_layernorm.weight"], eps)
            x = x + F.linear(F.silu(F.linear(h, w[p + "mlp.gate_proj.weight"])) * F.linear(h, w[p + "mlp.up_proj.weight"]),
                             w[p + "mlp.down_proj.weight"])
        want = F.linear(F.rms_norm(x, (d,), w["model.norm.weight"], eps), head)
        got = P.forward(w, sizes, [tok], torch.float64)[0]
        assert torch.allclose(got, want, atol=1e-10)
        wrong = F.linear(x, head)   # the check has teeth: without the final norm the logits are others
        assert not torch.allclose(got, wrong, atol=1e-3)


def test_branches_add_to_a_stream_that_is_never_normalised_in_place(tmp_path):
    """With every output projection (o_proj, down_proj) zero the branches add nothing, and the logits at every
    position are ``head(norm(embedding))``: an arrangement that normalises the stream itself (post-norm)
    does not reduce to this.  And with the embedding scaled up by 10^4 the branches, which read a normalised
    stream and therefore stay as they were, vanish beside it: the logits tend to the same value."""
    w, sizes = read_for_plain(make_model_dir(tmp_path, "B"))
    w = {k: v.double() for k, v in w.items()}
    toks = random_prompt(11, sizes["vocab"], 8)
    d, eps = sizes["hidden"], sizes["eps"]
    bare = F.linear(F.rms_norm(w["model.embed_tokens.weight"][toks], (d,), w["model.norm.weight"], eps), w["lm_head.weight"])
    off = {k: (torch.zeros_like(v) if k.endswith(("o_proj.weight", "down_proj.weight")) else v) for k, v in w.items()}
    assert torch.allclose(P.forward(off, sizes, toks, torch.float64), bare, atol=1e-10)
    full = P.forward(w, sizes, toks, torch.float64)
    assert not torch.allclose(full, bare, atol=1e-3)
    big = dict(w)
    big["model.embed_tokens.weight"] = w["model.embed_tokens.weight"] * 1e4
    bare_big = F.linear(F.rms_norm(big["model.embed_tokens.weight"][toks], (d,), w["model.norm.weight"], eps), w["lm_head.weight"])
    assert (P.forward(big, sizes, toks, torch.float64) - bare_big).abs().max() < 1e-3 * bare_big.abs().max()


def test_shift_of_all_positions_changes_nothing():
    """Only distances count: the same tokens at positions 100.. give the same logits."""
    import tempfile
    with tempfile.TemporaryDirectory() as tmp:
        w, sizes = read_for_plain(make_model_dir(tmp, "B"))
    toks = random_prompt(9, sizes["vocab"], 4)
    a = P.forward(w, sizes, toks, torch.float64)
    b = P.forward(w, sizes, toks, torch.float64, start_pos=100)
    assert torch.allclose(a, b, atol=1e-9)


def test_tied_and_untied_heads(tmp_path):
    wa, sa = read_for_plain(make_model_dir(tmp_path, "A"))
    assert sa["tied"] and "lm_head.weight" not in wa
    wb, sb = read_for_plain(make_model_dir(tmp_path, "B"))
    assert not sb["tied"] and "lm_head.weight" in wb
    toks = random_prompt(5, sb["vocab"], 5)
    tied = dict(sb, tied=True)
    assert not torch.allclose(P.forward(wb, sb, toks), P.forward(wb, tied, toks), atol=1e-3)


def test_splitmix64_vectors():
    """The published first outputs of SplitMix64 seeded with 0 are the finalizer of 1x and 2x
    the golden ratio; the reference applies the finalizer to the state before the increment
    (crates/mach-model/src/sampling.rs:27-44), so seed 0 draws mix64(0) = 0 first."""
    assert P.mix64(0) == 0
    assert P.mix64(P.RNG_GOLDEN) == 0xE220A8397B1DCDAF
    assert P.mix64((2 * P.RNG_GOLDEN) & P.MASK64) == 0x6E789E6AA1B965F4
    u, st = P.next_uniform(0)
    assert u == 0.0 and st == P.RNG_GOLDEN
    u, st = P.next_uniform(st)
    assert u == (0xE220A8397B1DCDAF >> 40) / 2 ** 24 and st == (2 * P.RNG_GOLDEN) & P.MASK64


def test_sampler_mirror():
    logits = np.array([0.1, 2.0, 2.0, -1.0, 0.5], dtype=np.float32)
    tok, st = P.sample(logits, 0.0, 0, 1.0, 123)
    assert tok == 1 and st == (123 + P.RNG_GOLDEN) & P.MASK64     # ties: lowest index; greedy advances too
    # temperature -> 0 is greedy; top_k = 1 is greedy; tiny top_p is greedy
    spread = np.linspace(-3, 3, 50).astype(np.float32)
    for seed in range(1, 20):
        assert P.sample(spread, 1e-3, 0, 1.0, seed)[0] == 49
        assert P.sample(spread, 1.0, 1, 1.0, seed)[0] == 49
        assert P.sample(spread, 1.0, 0, 1e-6, seed)[0] == 49
    # same seed, same token; the draws follow the distribution
    flat = np.zeros(8, dtype=np.float32)
    picks = [P.sample(flat, 1.0, 0, 1.0, s)[0] for s in range(1, 400)]
    assert picks == [P.sample(flat, 1.0, 0, 1.0, s)[0] for s in range(1, 400)]
    counts = np.bincount(picks, minlength=8)
    assert counts.min() > 25
    # top-k keeps exactly the k largest (ties aside)
    for seed in range(1, 50):
        assert P.sample(spread, 5.0, 3, 1.0, seed)[0] >= 47
    # penalties and biases act on the logits first
    tok, _ = P.sample(logits, 0.0, 0, 1.0, 1, presence=5.0, counts=[(1, 1)])
    assert tok == 2
    tok, _ = P.sample(logits, 0.0, 0, 1.0, 1, frequency=0.5, counts=[(1, 3), (2, 4)])
    assert tok == 1
    tok, _ = P.sample(logits, 0.0, 0, 1.0, 1, bias=[(3, 10.0)])
    assert tok == 3


def test_bf16_rounding_vectors():
    """crates/mach-model/src/fp16.rs:84-94, 167-169."""
    assert P.f32_to_bf16_bits(1.0) == 0x3F80
    assert P.f32_to_bf16_bits(1.0 + 2 ** -8) == 0x3F80        # tie to even (down)
    assert P.f32_to_bf16_bits(1.0 + 3 * 2 ** -8) == 0x3F82    # tie to even (up)
    for v in (0.1, -3.7, 1e-20, 65504.0):
        assert P.f32_to_bf16_bits(v) == (torch.tensor(v).to(torch.bfloat16).view(torch.int16).item() & 0xFFFF)
