"""A model folder's tensors by name: every ``*.safetensors`` file of the folder (one
``model.safetensors`` or shards), with the reference's renaming of
``model.language_model.`` to ``model.`` (``crates/mach-model/src/loader.rs:52-57,
113-118, 877-910``).  A name that two files hold, or that appears twice after
renaming, is an error.  When the folder holds a ``model.safetensors.index.json`` it is checked
against the files (``crates/mach-model/src/loader.rs:327-502``): shards it names that are missing,
``.safetensors`` files it does not name, tensors it does not list or lists in another shard,
listed tensors that no shard holds, and a ``metadata.total_size`` that differs from the bytes the
headers describe; one error lists every finding.
"""
from __future__ import annotations

import json
import os
from typing import Dict, List, Optional, Tuple

import torch

from .safetensors_io import SafetensorsError, SafetensorsFile

_RENAMES = (("model.language_model.", "model."),)


def _canonical(name: str) -> str:
    for old, new in _RENAMES:
        if name.startswith(old):
            return new + name[len(old):]
    return name


INDEX_FILE = "model.safetensors.index.json"


class CheckpointIndexError(SafetensorsError):
    """The folder's index and its files disagree; the message lists every finding."""

    def __init__(self, path: str, findings: List[str]):
        self.findings = findings
        super().__init__(f"{path} does not fit the folder's files:\n  " + "\n  ".join(findings))


def _read_index(model_dir: str) -> Optional[Tuple[Dict[str, str], Optional[int]]]:
    """``(tensor -> shard file name, metadata.total_size or None)`` of the folder's index, or None
    if it has none.  A shard is named by a plain file name beside the index, never by a path."""
    path = os.path.join(model_dir, INDEX_FILE)
    if not os.path.isfile(path):
        return None
    try:
        with open(path, "r", encoding="utf-8") as f:
            raw = json.load(f)
    except (OSError, ValueError) as e:
        raise SafetensorsError(f"{path}: {e}") from None
    weight_map = raw.get("weight_map") if isinstance(raw, dict) else None
    if not isinstance(weight_map, dict):
        raise SafetensorsError(f"{path}: weight_map is missing or not an object")
    findings, out = [], {}
    for name, shard in weight_map.items():
        if not isinstance(shard, str) or os.path.basename(shard) != shard or not shard.endswith(".safetensors"):
            findings.append(f"weight_map[{name!r}] = {shard!r} does not name a .safetensors file beside the index")
            continue
        canon = _canonical(name)
        if canon in out:
            findings.append(f"tensor {canon!r} is listed twice after renaming")
        out[canon] = shard
    total = raw.get("metadata", {}).get("total_size") if isinstance(raw.get("metadata"), dict) else None
    if total is not None and (isinstance(total, bool) or not isinstance(total, (int, float)) or total < 0 or total != int(total)):
        findings.append(f"metadata.total_size = {total!r} is not a non-negative integer")
        total = None
    if findings:
        raise CheckpointIndexError(path, findings)
    return out, None if total is None else int(total)


class Checkpoint:
    def __init__(self, model_dir: str):
        index = None
        if os.path.isdir(model_dir):
            files = sorted(f for f in os.listdir(model_dir) if f.endswith(".safetensors"))
            index = _read_index(model_dir)
            if index is not None:
                named = set(index[0].values())
                findings = [f"shard {f!r} is named by the index but missing" for f in sorted(named - set(files))]
                findings += [f"file {f!r} is not named by the index" for f in sorted(set(files) - named)]
                if findings:
                    raise CheckpointIndexError(os.path.join(model_dir, INDEX_FILE), findings)
            paths = [os.path.join(model_dir, f) for f in files]
        else:
            paths = [model_dir]  # a single file is read on its own, whatever index lies beside it
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
        if index is not None:
            self._check_index(os.path.join(model_dir, INDEX_FILE), *index)

    def _check_index(self, path: str, listed: Dict[str, str], total_size: Optional[int]) -> None:
        findings = []
        payload = 0
        for name, (sf, raw) in sorted(self._where.items()):
            _, _, start, end = sf.entries[raw]
            payload += end - start
            shard = os.path.basename(sf.path)
            if name not in listed:
                findings.append(f"tensor {name!r} of {shard} is absent from the index")
            elif listed[name] != shard:
                findings.append(f"tensor {name!r} lies in {shard}, the index lists it in {listed[name]}")
        findings += [f"tensor {name!r} is listed in {shard} but no shard holds it"
                     for name, shard in sorted(listed.items()) if name not in self._where]
        if total_size is not None and total_size != payload:
            findings.append(f"metadata.total_size = {total_size}, the shards' headers describe {payload} bytes")
        if findings:
            raise CheckpointIndexError(path, findings)

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
