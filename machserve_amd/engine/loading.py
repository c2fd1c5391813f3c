"""From a model folder (or a typed configuration plus tensors) to a model on the device
with its cache and step function."""
from __future__ import annotations

from dataclasses import dataclass
from typing import Optional

import torch

from ..cache import CacheManager, DeviceCache, pages_by_need
from ..config import load_config
from ..kernels import get_ops
from ..parts import DecoderModel, Runtime
from ..weights import Checkpoint, TensorDict, load_weights
from .step import StepFunction

DTYPES = {"bfloat16": torch.bfloat16, "bf16": torch.bfloat16, "float16": torch.float16, "fp16": torch.float16,
          "f16": torch.float16, "half": torch.float16, "float32": torch.float32, "fp32": torch.float32, "f32": torch.float32}


def parse_dtype(name) -> torch.dtype:
    if isinstance(name, torch.dtype):
        if name in (torch.bfloat16, torch.float16, torch.float32):
            return name
    elif name in DTYPES:
        return DTYPES[name]
    raise ValueError(f"dtype {name!r}: choose bfloat16, float16 or float32")


@dataclass
class LoadedModel:
    config: object
    model: DecoderModel
    cache: CacheManager
    device_cache: DeviceCache
    step: StepFunction
    rt: Runtime


def load_model(model_dir: Optional[str] = None, *, dtype="bfloat16", device: str = "cuda:0", page_size: int = 64,
               num_pages=None, max_tokens: Optional[int] = None, max_requests: int = 64,
               config=None, tensors=None, ops=None, use_graphs: bool = True, portion: Optional[int] = None) -> LoadedModel:
    """``model_dir`` holds config.json and model.safetensors; alternatively pass a typed
    ``config`` and a dict of ``tensors``.  Every group's pool has ``num_pages`` pages (a dict
    gives each group its own number), or enough for ``max_tokens`` tokens; with ``portion``
    (the most tokens of one request that a step will bring) a group of layers that see a window
    gets only what ``max_requests`` requests can hold of it at a time."""
    dt = parse_dtype(dtype)
    if config is None:
        config = load_config(model_dir)
    if ops is None:
        ops = get_ops(dt, device)
    rt = Runtime(torch.device(device), dt, ops)
    model = DecoderModel(config.to_spec(), rt)
    source = TensorDict(tensors) if tensors is not None else Checkpoint(model_dir)
    load_weights(model, source, rt)
    if num_pages is None:
        if max_tokens is None:
            max_tokens = 4096
        num_pages = (pages_by_need(max_tokens, max_requests, portion, page_size) if portion
                     else max(1, -(-max_tokens // page_size)))
    cache = CacheManager(model.cache_requests(), page_size, num_pages, max_requests)
    device_cache = DeviceCache(cache, dt, rt.device)
    model.bind_cache(device_cache)
    # the work lists of a step are cut in the unit that the attention kernels themselves report
    step = StepFunction(model, cache, rt, model.attention_rows_per_block() or 64, use_graphs)
    return LoadedModel(config, model, cache, device_cache, step, rt)
