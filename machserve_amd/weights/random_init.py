"""Random-weights mode: a model folder (config.json, model.safetensors) from a
configuration and a seed.

Law: matrices ~ N(0, 0.02), norm weights ~ 1 + N(0, 0.02), biases ~ N(0, 0.02), drawn
in float32 from one seeded generator in the order of the configuration's tensor plan,
then stored in ``dtype``.  (The reference's ``Weights::random`` draws
``U(-1,1)/sqrt(d)`` and no biases, ``crates/mach-model/src/weights.rs:230-245,
336-374``; biases are drawn here so that the q/k/v bias path is exercised.)
"""
from __future__ import annotations

import json
import os
from typing import Dict, Iterator, Tuple

import torch

from ..config import config_from_dict
from .safetensors_io import write_safetensors

STD = 0.02


def _draw(shape, law: str, gen: torch.Generator, device) -> torch.Tensor:
    t = torch.randn(shape, generator=gen, dtype=torch.float32, device=device) * STD
    if law == "norm":
        t = t + 1.0
    elif law not in ("matrix", "bias"):
        raise ValueError(f"unknown law {law!r}")
    return t


def random_tensors(config, seed: int, dtype: torch.dtype = torch.float32,
                   device: str = "cpu") -> Iterator[Tuple[str, torch.Tensor]]:
    gen = torch.Generator(device=device)
    gen.manual_seed(int(seed))
    for name, shape, law in config.random_tensor_plan():
        yield name, _draw(shape, law, gen, device).to(dtype)


def random_tensor_dict(config, seed: int, dtype=torch.float32, device="cpu") -> Dict[str, torch.Tensor]:
    return dict(random_tensors(config, seed, dtype, device))


def write_random_model(config, seed: int, out_dir: str, dtype: torch.dtype = torch.float32) -> str:
    """``config`` is a typed configuration or a config.json dict.  Returns ``out_dir``."""
    if isinstance(config, dict):
        config = config_from_dict(config)
    os.makedirs(out_dir, exist_ok=True)
    raw = config.to_dict()
    raw["torch_dtype"] = {torch.float32: "float32", torch.bfloat16: "bfloat16", torch.float16: "float16"}[dtype]
    with open(os.path.join(out_dir, "config.json"), "w", encoding="utf-8") as f:
        json.dump(raw, f, indent=1)
    it = random_tensors(config, seed, dtype)
    plan = [(n, s, dtype) for n, s, _ in config.random_tensor_plan()]

    def produce(name):
        got, t = next(it)
        assert got == name
        return t

    write_safetensors(os.path.join(out_dir, "model.safetensors"), plan, produce)
    return out_dir
