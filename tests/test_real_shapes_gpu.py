"""The layer sizes of Qwen2.5-0.5B, 1.5B and 7B (head sizes 64 and 128, 14/12/28 heads over 2/2/4 KV
heads, widths 896/1536/3584, vocabularies of 151,936 and 152,064) with two layers and random
weights: replay in portions, decoded tokens and a mixed batch against the plain model, in
32-bit and in bfloat16."""
import pytest
import torch

from gpu_util import DEV
from plain import qwen2_plain as P
from tiny_configs import random_prompt

pytestmark = pytest.mark.gpu

SHAPES = {
    "0.5B": dict(hidden_size=896, num_attention_heads=14, num_key_value_heads=2, intermediate_size=4864, vocab_size=151936,
                 tie_word_embeddings=True),
    "1.5B": dict(hidden_size=1536, num_attention_heads=12, num_key_value_heads=2, intermediate_size=8960, vocab_size=151936,
                 tie_word_embeddings=True),
    "7B": dict(hidden_size=3584, num_attention_heads=28, num_key_value_heads=4, intermediate_size=18944, vocab_size=152064,
               tie_word_embeddings=False),
}


def config(name):
    raw = {"architectures": ["Qwen2ForCausalLM"], "model_type": "qwen2", "num_hidden_layers": 2,
           "max_position_embeddings": 4096, "rms_norm_eps": 1e-6, "rope_theta": 1000000.0, "hidden_act": "silu"}
    raw.update(SHAPES[name])
    return raw


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("name", ["0.5B", "1.5B", "7B"])
def test_real_layer_sizes(name, dtype):
    from machserve_amd.config import config_from_dict
    from machserve_amd.engine import StepEntry, load_model
    from machserve_amd.weights import random_tensor_dict
    cfg = config_from_dict(config(name))
    tensors = random_tensor_dict(cfg, 3)
    sizes = P.sizes_from_config(config(name))
    ww = tensors if dtype == torch.float32 else {k: v.to(torch.bfloat16).float() if v.dim() == 2 else v for k, v in tensors.items()}
    a, b = random_prompt(150, cfg.vocab_size, 1), random_prompt(70, cfg.vocab_size, 2)
    ra, rb = P.forward(ww, sizes, a), P.forward(ww, sizes, b)
    lm = load_model(config=cfg, tensors=tensors, dtype=dtype, device=DEV, page_size=64, num_pages=5, max_requests=2)
    sa, sb = lm.cache.admit(), lm.cache.admit()
    got_a, got_b = [], []
    # a: a long portion, a short one, then portions beside b's prompt, then both decode side by side
    got_a.append(lm.step([StepEntry(sa, a[:80], list(range(80)))]))
    # twenty rows: few enough for the few-rows kernels, but the large products go to the tiled kernel
    got_a.append(lm.step([StepEntry(sa, a[80:100], list(range(20)))]))
    out = lm.step([StepEntry(sa, a[100:130], list(range(30))), StepEntry(sb, b[:66], list(range(66)))])
    got_a.append(out[:30]), got_b.append(out[30:])
    out = lm.step([StepEntry(sa, a[130:132], [0, 1]), StepEntry(sb, b[66:67], [0])])
    got_a.append(out[:2]), got_b.append(out[2:])
    for i in range(3):
        out = lm.step([StepEntry(sb, b[67 + i:68 + i], [0]), StepEntry(sa, a[132 + i:133 + i], [0])])
        got_b.append(out[:1]), got_a.append(out[1:])
    lm.cache.release(sb)
    for i in range(135, 150):
        got_a.append(lm.step([StepEntry(sa, a[i:i + 1], [0])]))
    lm.cache.release(sa)
    lm.cache.check()
    for got, ref, n in ((torch.cat(got_a), ra, 150), (torch.cat(got_b), rb, 70)):
        got = got.float().cpu()
        assert got.shape[0] == n
        scale = ref.abs().max().item()
        allowed = 2e-5 + 2e-5 * scale if dtype == torch.float32 else 3e-2 * scale
        err = (got - ref[:n]).abs().max().item()
        assert err <= allowed, f"{name} {dtype}: max error {err:.3e}, allowed {allowed:.3e}"
        if dtype == torch.float32:
            assert torch.equal(got.argmax(-1), ref[:n].argmax(-1))


@pytest.mark.timeout(300)
@pytest.mark.parametrize("T,dtype", [(2000, torch.bfloat16), (2048, torch.float16), (8192, torch.bfloat16)])
def test_long_prompts_at_the_0_5b_layer_sizes(T, dtype):
    """A prompt of thousands of tokens in one step at the 0.5B layer sizes (two layers, a small vocabulary), then decoded
    tokens, against the plain model: what only such sizes reach inside the engine: the widest tiles of the products (128x160,
    and 256x256 at 8,192 rows), the down projection cut along K, the q/k/v product that rotates and writes the cache, the
    attention in 32-row tiles over several rounds of blocks, a step filled up and captured."""
    from machserve_amd.config import config_from_dict
    from machserve_amd.engine import StepEntry, load_model
    from machserve_amd.weights import random_tensor_dict
    raw = config("0.5B")
    raw.update(vocab_size=8000, max_position_embeddings=16384)
    cfg = config_from_dict(raw)
    tensors = random_tensor_dict(cfg, 3)
    sizes = P.sizes_from_config(raw)
    ww = {k: v.to(dtype).float() if v.dim() == 2 else v for k, v in tensors.items()}
    toks = random_prompt(T + 6, 8000, T)
    ref = P.forward(ww, sizes, toks)
    lm = load_model(config=cfg, tensors=tensors, dtype=dtype, device=DEV, page_size=64, num_pages=T // 64 + 3, max_requests=1)
    lm.step.FILLED_CAPTURE_AFTER = 0
    rows = [0, 63, 64, T // 2, T - 130, T - 2, T - 1]
    slot = lm.cache.admit()
    got = [lm.step([StepEntry(slot, toks[:T], rows)])]
    got += [lm.step([StepEntry(slot, toks[T + i:T + i + 1], [0])]) for i in range(6)]
    lm.cache.release(slot)
    lm.cache.check()
    got = torch.cat(got).float().cpu()
    want = torch.cat([ref[rows], ref[T:T + 6]])
    scale = want.abs().max().item()
    err = (got - want).abs().max().item()
    allowed = (3e-2 if dtype == torch.bfloat16 else 3e-2 / 8) * scale
    assert err <= allowed, f"{T} tokens, {dtype}: max error {err:.3e}, allowed {allowed:.3e}"
