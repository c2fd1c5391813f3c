"""A model folder's tensors by name: every ``*.safetensors`` file of the folder (one
``model.safetensors`` or shards), with the reference's renaming of
``model.language_model.`` to ``model.`` (``crates/mach-model/src/loader.rs:52-57,
113-118, 877-910``).  A name that two files hold, or that appears twice after
renaming, is an error.
"""
from __future__ import annotations

import os
from typing import Dict, Tuple

import torch

from .safetensors_io import SafetensorsError, SafetensorsFile

_RENAMES = (("model.language_model.", "model."),)


def _canonical(name: str) -> str:
    for old, new in _RENAMES:
        if name.startswith(old):
            return new + name[len(old):]
    return name


class Checkpoint:
    def __init__(self, model_dir: str):
        if os.path.isdir(model_dir):
            files = sorted(f for f in os.listdir(model_dir) if f.endswith(".safetensors"))
            paths = [os.path.join(model_dir, f) for f in files]
        else:
            paths = [model_dir]
        if not paths:
            raise SafetensorsError(f"{model_dir}: no .safetensors file")
        self._where: Dict[str, Tuple[SafetensorsFile, str]] = {}
        for p in paths:
            sf = SafetensorsFile(p)
            for raw in sf.entries:
                name = _canonical(raw)
                if name in self._where:
                    raise SafetensorsError(f"tensor {name!r} appears in {self._where[name][0].path} and in {p}")
                self._where[name] = (sf, raw)

    def names(self):
        return list(self._where)

    def __contains__(self, name: str) -> bool:
        return name in self._where

    def meta(self, name: str) -> Tuple[torch.dtype, Tuple[int, ...]]:
        sf, raw = self._where[name]
        dtype, shape, _, _ = sf.entries[raw]
        return dtype, shape

    def tensor(self, name: str) -> torch.Tensor:
        sf, raw = self._where[name]
        return sf.tensor(raw)


class TensorDict:
    """The same interface over tensors already in memory (random weights without a disk)."""

    def __init__(self, tensors: Dict[str, torch.Tensor]):
        self._t = tensors

    def names(self):
        return list(self._t)

    def __contains__(self, name):
        return name in self._t

    def meta(self, name):
        t = self._t[name]
        return t.dtype, tuple(t.shape)

    def tensor(self, name):
        return self._t[name]
