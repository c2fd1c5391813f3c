"""Small configurations of the architecture that differ in every size and option, and the
helpers that make model folders and plain-model inputs from them."""
from __future__ import annotations

import json
import os

import torch

# 2 layers, 4 heads over 2 KV heads (group 2), head size 16, tied head
TINY_A = {
    "architectures": ["Qwen2ForCausalLM"], "model_type": "qwen2", "hidden_size": 64, "num_hidden_layers": 2,
    "num_attention_heads": 4, "num_key_value_heads": 2, "intermediate_size": 160, "vocab_size": 512,
    "max_position_embeddings": 256, "rms_norm_eps": 1e-6, "rope_theta": 10000.0, "tie_word_embeddings": True,
    "hidden_act": "silu", "use_sliding_window": False,
}
# 3 layers, 6 heads over 1 KV head (group 6), head size 32, untied head, other eps and theta
TINY_B = {
    "architectures": ["Qwen2ForCausalLM"], "model_type": "qwen2", "hidden_size": 192, "num_hidden_layers": 3,
    "num_attention_heads": 6, "num_key_value_heads": 1, "intermediate_size": 320, "vocab_size": 1000,
    "max_position_embeddings": 512, "rms_norm_eps": 1e-5, "rope_theta": 1000000.0, "tie_word_embeddings": False,
    "hidden_act": "silu", "use_sliding_window": False,
}
# 4 layers, 5 heads over 5 KV heads (group 1), explicit head size 48 (heads * head_dim != hidden),
# no biases, sliding window of 40 keys on the upper two layers
TINY_C = {
    "architectures": ["Qwen2ForCausalLM"], "model_type": "qwen2", "hidden_size": 136, "num_hidden_layers": 4,
    "num_attention_heads": 5, "num_key_value_heads": 5, "head_dim": 48, "intermediate_size": 264, "vocab_size": 777,
    "max_position_embeddings": 1024, "rms_norm_eps": 3e-6, "rope_theta": 50000.0, "tie_word_embeddings": False,
    "hidden_act": "silu", "use_sliding_window": True, "sliding_window": 40, "max_window_layers": 2,
    "attention_bias": False,
}
SEEDS = {"A": 0, "B": 1, "C": 2}
CONFIGS = {"A": TINY_A, "B": TINY_B, "C": TINY_C}


def make_model_dir(tmp, which: str, dtype=torch.float32) -> str:
    from machserve_amd.weights import write_random_model
    out = os.path.join(str(tmp), f"tiny_{which}")
    return write_random_model(dict(CONFIGS[which]), SEEDS[which], out, dtype)


def read_for_plain(model_dir: str):
    """(weights by name, sizes) for the plain model, read with the safetensors package."""
    from safetensors.torch import load_file
    from plain.qwen2_plain import sizes_from_config
    with open(os.path.join(model_dir, "config.json")) as f:
        cfg = json.load(f)
    return load_file(os.path.join(model_dir, "model.safetensors")), sizes_from_config(cfg)


def random_prompt(length: int, vocab: int, seed: int):
    g = torch.Generator().manual_seed(seed)
    return torch.randint(0, vocab, (length,), generator=g).tolist()


def sharpen_attention(model_dir: str, by: float) -> None:
    """Multiplies the query and key projections (weights and biases) of a written model by `by`: the scores grow by
    its square, the softmax stops being nearly flat, and what changes a score (a rotation angle, a scale) shows in
    the logits, which it hardly does with small random weights."""
    from safetensors.torch import load_file, save_file
    path = os.path.join(model_dir, "model.safetensors")
    w = load_file(path)
    for name in w:
        if ".q_proj." in name or ".k_proj." in name:
            w[name] = (w[name].float() * by).to(w[name].dtype)
    save_file(w, path)
