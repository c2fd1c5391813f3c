"""Configurations drawn at random (seeded): head sizes in steps of 16 up to 256, one to four key/value heads with
one to sixteen heads each, widths and vocabularies that are no power of two, one to three layers, with and without
biases, tied head and sliding window, pages of 16 to 64 tokens.  Each goes through the engine whole, in portions of
changing size, with its last tokens one by one, and as three requests that decode side by side; every logit
against the plain model, with the bounds of ``test_replay_gpu``.  What the three fixed configurations leave out
(a group of 16, a head of 256, a window that a page does not divide) turns up here."""
import os
import random

import pytest
import torch

from gpu_util import DEV
from test_replay_gpu import check, plain_ref
from tiny_configs import random_prompt, read_for_plain

pytestmark = pytest.mark.gpu


def draw(rnd: random.Random) -> dict:
    kv, group, layers = rnd.choice([1, 2, 3, 4]), rnd.choice([1, 2, 3, 4, 5, 7, 8, 12, 16]), rnd.choice([1, 2, 3])
    window = rnd.choice([None, None, 24, 40, 70])
    cfg = {"architectures": ["Qwen2ForCausalLM"], "model_type": "qwen2", "hidden_size": rnd.choice([64, 72, 136, 200, 264, 328]),
           "num_hidden_layers": layers, "num_attention_heads": kv * group, "num_key_value_heads": kv,
           "head_dim": rnd.choice([16, 32, 48, 64, 80, 96, 128, 160, 192, 256]),
           "intermediate_size": rnd.choice([96, 160, 208, 264, 328]), "vocab_size": rnd.choice([300, 512, 777, 1000, 2051]),
           "max_position_embeddings": 512, "rms_norm_eps": rnd.choice([1e-6, 1e-5, 3e-6]), "rope_theta": rnd.choice([1e4, 5e4, 1e6]),
           "tie_word_embeddings": rnd.random() < 0.5, "hidden_act": "silu", "attention_bias": rnd.random() < 0.7,
           "use_sliding_window": window is not None}
    if window is not None:
        cfg["sliding_window"] = window
        cfg["max_window_layers"] = rnd.randrange(0, layers + 1)
    return cfg


def run_cuts(lm, prompt, cuts):
    from machserve_amd.engine import StepEntry
    slot = lm.cache.admit()
    out, i = [], 0
    for c in cuts:
        out.append(lm.step([StepEntry(slot, prompt[i:i + c], list(range(c)))]))
        i += c
    lm.cache.release(slot)
    lm.cache.check()
    return torch.cat(out)


@pytest.mark.parametrize("seed", range(10))
def test_a_configuration_drawn_at_random(seed, tmp_path):
    from machserve_amd.engine import StepEntry, load_model
    from machserve_amd.weights import write_random_model
    rnd = random.Random(1000 + seed)
    cfg = draw(rnd)
    folder = write_random_model(cfg, 200 + seed, os.path.join(str(tmp_path), "model"), torch.float32)
    w, sizes = read_for_plain(folder)
    n, page = rnd.choice([37, 70, 101, 150]), rnd.choice([16, 32, 64])
    prompt = random_prompt(n, cfg["vocab_size"], seed)
    cuts, left = [], n
    while left:
        cuts.append(min(left, rnd.choice([2, 3, 5, 9, 17, 33, 64])))
        left -= cuts[-1]
    side_by_side = [prompt[:n - 25], prompt[5:n - 12], prompt[9:n - 18]]
    what = f"{cfg}, pages of {page}, {n} tokens"
    for dtype in (torch.float32, torch.bfloat16):
        ref = plain_ref(w, sizes, prompt, dtype)
        lm = load_model(folder, dtype=dtype, device=DEV, page_size=page, num_pages=4 * (n // page + 2))
        check(run_cuts(lm, prompt, [n]), ref, dtype, f"whole: {what}")
        check(run_cuts(lm, prompt, cuts), ref, dtype, f"in portions {cuts}: {what}")
        check(run_cuts(lm, prompt, [n - 20] + [1] * 20), ref, dtype, f"the last 20 one by one: {what}")
        slots = [lm.cache.admit() for _ in side_by_side]
        fed = [len(p) - 8 for p in side_by_side]
        outs = [[lm.step([StepEntry(slots[i], p[:fed[i]], list(range(fed[i])))])] for i, p in enumerate(side_by_side)]
        for k in range(8):
            step = lm.step([StepEntry(slots[i], [p[fed[i] + k]], [0]) for i, p in enumerate(side_by_side)])
            for i in range(3):
                outs[i].append(step[i:i + 1])
        for i, p in enumerate(side_by_side):
            check(torch.cat(outs[i]), plain_ref(w, sizes, p, dtype), dtype, f"request {i} of three side by side: {what}")
            lm.cache.release(slots[i])
        lm.cache.check()
        del lm
