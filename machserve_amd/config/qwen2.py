"""Typed configuration of the dense Qwen2 decoder, read from config.json's own keys.

Keys and their meaning follow ``crates/mach-server/src/startup.rs:55-98`` of the
reference (hidden_size, num_hidden_layers, num_attention_heads, num_key_value_heads,
vocab_size, intermediate_size, max_position_embeddings, rms_norm_eps, rope_theta,
head_dim, nested ``text_config``).  The reference falls back to Qwen2.5-0.5B's sizes
and constants when a key is missing; here a missing size, ``max_position_embeddings``,
``rms_norm_eps`` or ``rope_theta`` is an error that names the key, so none of them stands in code.
Keys the reference ignores but that change the result are read and checked:
``tie_word_embeddings``, ``hidden_act``, ``rope_scaling``, and the sliding-window trio
``use_sliding_window`` / ``sliding_window`` / ``max_window_layers``.
"""
from __future__ import annotations

import json
import os
from dataclasses import dataclass, asdict
from typing import Optional

from .specs import (AttentionSpec, ConfigError, EmbeddingSpec, GatedMlpSpec, HeadSpec, LayerSpec, ModelSpec,
                    NormSpec, RotarySpec, YarnSpec)

ARCHITECTURE = "Qwen2ForCausalLM"


def _need_int(d: dict, key: str, minimum: int = 1) -> int:
    if key not in d or d[key] is None:
        raise ConfigError(f"config.json: missing key '{key}'")
    v = d[key]
    if isinstance(v, bool) or not isinstance(v, int) or v < minimum:
        raise ConfigError(f"config.json: '{key}' must be an integer >= {minimum}, got {v!r}")
    return v


def _need_number(d: dict, key: str) -> float:
    v = d.get(key)
    if v is None:
        raise ConfigError(f"config.json: missing key '{key}'")
    if isinstance(v, bool) or not isinstance(v, (int, float)) or v <= 0:
        raise ConfigError(f"config.json: '{key}' must be a positive number, got {v!r}")
    return float(v)


@dataclass(frozen=True)
class Qwen2Config:
    hidden_size: int
    num_hidden_layers: int
    num_attention_heads: int
    num_key_value_heads: int
    head_dim: int
    intermediate_size: int
    vocab_size: int
    max_position_embeddings: int
    rms_norm_eps: float
    rope_theta: float
    tie_word_embeddings: Optional[bool]
    use_sliding_window: bool
    sliding_window: Optional[int]
    max_window_layers: int
    attention_bias: bool
    torch_dtype: Optional[str]
    rope_scaling: Optional[YarnSpec] = None

    @classmethod
    def from_dict(cls, raw: dict) -> "Qwen2Config":
        d = raw.get("text_config") if isinstance(raw.get("text_config"), dict) else raw
        hidden = _need_int(d, "hidden_size")
        layers = _need_int(d, "num_hidden_layers")
        heads = _need_int(d, "num_attention_heads")
        kv = _need_int(d, "num_key_value_heads") if d.get("num_key_value_heads") is not None else heads
        if d.get("head_dim") is not None:
            head_dim = _need_int(d, "head_dim")
        else:
            if hidden % heads:
                raise ConfigError(f"config.json: hidden_size {hidden} is not a multiple of num_attention_heads "
                                  f"{heads} and no head_dim is given")
            head_dim = hidden // heads
        if heads % kv:
            raise ConfigError(f"config.json: num_attention_heads {heads} is not a multiple of "
                              f"num_key_value_heads {kv}")
        if head_dim % 2:
            raise ConfigError(f"config.json: head_dim {head_dim} must be even for rotary pairs")
        act = d.get("hidden_act", "silu")
        if act != "silu":
            raise ConfigError(f"config.json: hidden_act {act!r} is not supported (silu only)")
        yarn = cls._yarn_of(d.get("rope_scaling"))
        theta = d.get("rope_theta")
        if theta is None and isinstance(d.get("rope_parameters"), dict):
            theta = d["rope_parameters"].get("rope_theta")
        if theta is None:
            raise ConfigError("config.json: missing key 'rope_theta' (or 'rope_parameters.rope_theta')")
        if isinstance(theta, bool) or not isinstance(theta, (int, float)) or theta <= 0:
            raise ConfigError(f"config.json: 'rope_theta' must be a positive number, got {theta!r}")
        theta = float(theta)
        use_win = bool(d.get("use_sliding_window", False))
        window = d.get("sliding_window")
        max_win_layers = d.get("max_window_layers")
        if use_win:
            if not isinstance(window, int) or window < 1:
                raise ConfigError(f"config.json: use_sliding_window needs sliding_window >= 1, got {window!r}")
            if max_win_layers is None:
                raise ConfigError("config.json: use_sliding_window needs max_window_layers")
        tie = d.get("tie_word_embeddings", raw.get("tie_word_embeddings"))
        return cls(
            hidden_size=hidden, num_hidden_layers=layers, num_attention_heads=heads, num_key_value_heads=kv,
            head_dim=head_dim, intermediate_size=_need_int(d, "intermediate_size"),
            vocab_size=_need_int(d, "vocab_size"),
            max_position_embeddings=_need_int(d, "max_position_embeddings"),
            rms_norm_eps=_need_number(d, "rms_norm_eps"), rope_theta=theta,
            tie_word_embeddings=None if tie is None else bool(tie),
            use_sliding_window=use_win, sliding_window=window if use_win else None,
            max_window_layers=int(max_win_layers) if max_win_layers is not None else layers,
            attention_bias=bool(d.get("attention_bias", True)),
            torch_dtype=d.get("torch_dtype"), rope_scaling=yarn,
        )

    @staticmethod
    def _yarn_of(rs) -> Optional[YarnSpec]:
        """``rope_scaling``: absent, or YaRN with the keys and defaults of ``crates/mach-server/src/startup.rs:172-199``
        (``type`` or ``rope_type`` "yarn", ``factor`` > 1, ``original_max_position_embeddings`` > 0, ``beta_fast`` 32,
        ``beta_slow`` 1, ``mscale`` 1, ``mscale_all_dim`` 0); any other kind is refused, as the reference refuses it."""
        if rs is None:
            return None
        if not isinstance(rs, dict):
            raise ConfigError(f"config.json: rope_scaling must be an object, got {rs!r}")
        kind = rs.get("type", rs.get("rope_type"))
        if kind in (None, "default"):
            return None
        if kind != "yarn":
            raise ConfigError(f"config.json: rope_scaling of type {kind!r} is not supported (only yarn)")

        def number(key, default):
            v = rs.get(key, default)
            if isinstance(v, bool) or not isinstance(v, (int, float)):
                raise ConfigError(f"config.json: rope_scaling.{key} must be a number, got {v!r}")
            return float(v)
        factor, orig = number("factor", 1.0), rs.get("original_max_position_embeddings", 0)
        if isinstance(orig, bool) or not isinstance(orig, int) or orig <= 0 or factor <= 1.0:
            raise ConfigError("config.json: rope_scaling of type yarn needs factor > 1 and original_max_position_embeddings > 0 "
                              f"(got factor={factor}, original_max_position_embeddings={orig!r})")
        return YarnSpec(factor, orig, number("beta_fast", 32.0), number("beta_slow", 1.0), number("mscale", 1.0),
                        number("mscale_all_dim", 0.0))

    @classmethod
    def from_json_file(cls, path: str) -> "Qwen2Config":
        if os.path.isdir(path):
            path = os.path.join(path, "config.json")
        with open(path, "r", encoding="utf-8") as f:
            return cls.from_dict(json.load(f))

    def to_dict(self) -> dict:
        d = asdict(self)
        if self.rope_scaling is not None:
            y = self.rope_scaling
            d["rope_scaling"] = {"type": "yarn", "factor": y.factor, "original_max_position_embeddings": y.original_max_positions,
                                 "beta_fast": y.beta_fast, "beta_slow": y.beta_slow, "mscale": y.mscale,
                                 "mscale_all_dim": y.mscale_all_dim}
        d["architectures"] = [ARCHITECTURE]
        d["model_type"] = "qwen2"
        d["hidden_act"] = "silu"
        return {k: v for k, v in d.items() if v is not None}

    def layer_window(self, i: int) -> Optional[int]:
        """Layers from ``max_window_layers`` on see only the last ``sliding_window`` keys."""
        if self.use_sliding_window and i >= self.max_window_layers:
            return self.sliding_window
        return None

    def attention_scale(self) -> Optional[float]:
        """What the scores are multiplied by: ``head_dim ** -0.5`` (None: the part's own default), times the square of
        YaRN's ``0.1 mscale_all_dim ln(factor) + 1`` where that applies (``crates/mach-model/src/config.rs:218-234``)."""
        y = self.rope_scaling
        if y is None or y.mscale_all_dim <= 0.0:
            return None
        import math
        m = 0.1 * y.mscale_all_dim * math.log(y.factor) + 1.0
        return m * m / math.sqrt(self.head_dim)

    def to_spec(self) -> ModelSpec:
        """Tensor names: ``crates/mach-model/src/loader.rs:1023-1037, 1189-1231``."""
        layers = []
        for i in range(self.num_hidden_layers):
            p = f"model.layers.{i}."
            rotary = RotarySpec("rotary", self.head_dim, self.rope_theta, yarn=self.rope_scaling)
            mixer = AttentionSpec(
                "attention", self.hidden_size, self.num_attention_heads, self.num_key_value_heads, self.head_dim,
                rotary, window=self.layer_window(i), scale=self.attention_scale(),
                tensors={"q.weight": p + "self_attn.q_proj.weight", "k.weight": p + "self_attn.k_proj.weight",
                         "v.weight": p + "self_attn.v_proj.weight", "o.weight": p + "self_attn.o_proj.weight",
                         "q.bias": p + "self_attn.q_proj.bias", "k.bias": p + "self_attn.k_proj.bias",
                         "v.bias": p + "self_attn.v_proj.bias"})
            ff = GatedMlpSpec("gated_mlp", self.hidden_size, self.intermediate_size, "silu",
                              tensors={"gate.weight": p + "mlp.gate_proj.weight", "up.weight": p + "mlp.up_proj.weight",
                                       "down.weight": p + "mlp.down_proj.weight"})
            n1 = NormSpec("rmsnorm", self.hidden_size, self.rms_norm_eps, {"weight": p + "input_layernorm.weight"})
            n2 = NormSpec("rmsnorm", self.hidden_size, self.rms_norm_eps,
                          {"weight": p + "post_attention_layernorm.weight"})
            layers.append(LayerSpec("prenorm", mixer, ff, n1, n2))
        spec = ModelSpec(
            architecture=ARCHITECTURE,
            embedding=EmbeddingSpec(self.vocab_size, self.hidden_size, {"weight": "model.embed_tokens.weight"}),
            layers=tuple(layers), order=tuple(range(self.num_hidden_layers)),
            final_norm=NormSpec("rmsnorm", self.hidden_size, self.rms_norm_eps, {"weight": "model.norm.weight"}),
            head=HeadSpec(self.vocab_size, self.hidden_size, self.tie_word_embeddings, {"weight": "lm_head.weight"}),
            max_positions=self.max_position_embeddings)
        spec.validate()
        return spec

    def random_tensor_plan(self):
        """(name, shape, law) of every tensor a random checkpoint of this configuration holds;
        law is 'matrix', 'norm' or 'bias'."""
        d, nq, nkv = self.hidden_size, self.num_attention_heads * self.head_dim, self.num_key_value_heads * self.head_dim
        plan = [("model.embed_tokens.weight", (self.vocab_size, d), "matrix")]
        for i in range(self.num_hidden_layers):
            p = f"model.layers.{i}."
            plan += [(p + "input_layernorm.weight", (d,), "norm"),
                     (p + "self_attn.q_proj.weight", (nq, d), "matrix"),
                     (p + "self_attn.k_proj.weight", (nkv, d), "matrix"),
                     (p + "self_attn.v_proj.weight", (nkv, d), "matrix")]
            if self.attention_bias:
                plan += [(p + "self_attn.q_proj.bias", (nq,), "bias"), (p + "self_attn.k_proj.bias", (nkv,), "bias"),
                         (p + "self_attn.v_proj.bias", (nkv,), "bias")]
            plan += [(p + "self_attn.o_proj.weight", (d, nq), "matrix"),
                     (p + "post_attention_layernorm.weight", (d,), "norm"),
                     (p + "mlp.gate_proj.weight", (self.intermediate_size, d), "matrix"),
                     (p + "mlp.up_proj.weight", (self.intermediate_size, d), "matrix"),
                     (p + "mlp.down_proj.weight", (d, self.intermediate_size), "matrix")]
        plan.append(("model.norm.weight", (d,), "norm"))
        if not self.tie_word_embeddings:
            plan.append(("lm_head.weight", (self.vocab_size, d), "matrix"))
        return plan
