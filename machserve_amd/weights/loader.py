"""Binding of a checkpoint's tensors to a model's parts, by name.

Every part declares its tensors by its own names; its spec maps them to checkpoint
names.  All declarations are checked against the checkpoint first, and one error lists
every missing tensor, every unexpected one and every wrong shape (full shapes, where the
reference compares element counts only, ``crates/mach-model/src/loader.rs:1016-1033``).
Then each tensor goes to the device in the dtype of its role: a 'matrix' in the element
type of the run, a 'vector' in float32, a 'table' in int32.
"""
from __future__ import annotations

from typing import Dict, List

import torch

_ROLE_DTYPE = {"vector": torch.float32, "table": torch.int32}


class WeightsError(ValueError):
    def __init__(self, missing: List[str], unexpected: List[str], shapes: List[str], other: List[str]):
        self.missing, self.unexpected, self.shapes, self.other = missing, unexpected, shapes, other
        lines = ["the checkpoint does not fit the model:"]
        if missing:
            lines.append(f"  missing tensors ({len(missing)}): " + ", ".join(missing))
        if unexpected:
            lines.append(f"  unexpected tensors ({len(unexpected)}): " + ", ".join(unexpected))
        if shapes:
            lines.append(f"  wrong shapes ({len(shapes)}): " + "; ".join(shapes))
        if other:
            lines.append("  " + "; ".join(other))
        super().__init__("\n".join(lines))


def _checkpoint_name(part, decl) -> str:
    return part.spec.tensors.get(decl.name, decl.name)


def load_weights(model, source, rt) -> None:
    """``source`` has ``names()``, ``meta(name)``, ``tensor(name)`` and ``in``."""
    missing, shapes, other = [], [], []
    used, ignored = set(), set()
    plan = []
    for part in model.parts():
        ignored.update(getattr(part, "ignored_tensors", lambda: [])())
        for decl in part.tensor_decls():
            name = _checkpoint_name(part, decl)
            if name not in source:
                if not decl.optional:
                    missing.append(name)
                plan.append((part, decl, None))
                continue
            used.add(name)
            dtype, shape = source.meta(name)
            if tuple(shape) != tuple(decl.shape):
                shapes.append(f"{name}: checkpoint {list(shape)}, model {list(decl.shape)}")
            if decl.role == "table" and dtype.is_floating_point:
                other.append(f"{name}: an integer table stored as {dtype}")
            if decl.role != "table" and not dtype.is_floating_point:
                other.append(f"{name}: a floating-point tensor stored as {dtype}")
            plan.append((part, decl, name))
    unexpected = sorted(set(source.names()) - used - ignored)
    if missing or unexpected or shapes or other:
        raise WeightsError(sorted(missing), unexpected, shapes, other)
    per_part: Dict[int, Dict[str, torch.Tensor]] = {}
    parts = {}
    for part, decl, name in plan:
        parts[id(part)] = part
        d = per_part.setdefault(id(part), {})
        if name is None:
            d[decl.name] = None
            continue
        want = _ROLE_DTYPE.get(decl.role, rt.dtype)
        t = source.tensor(name)
        d[decl.name] = t.to(device=rt.device, dtype=want).contiguous()
    for part in model.parts():
        part.load(per_part.get(id(part), {}))
