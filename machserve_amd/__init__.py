"""machserve_amd: a one-GPU inference engine for the dense Qwen2 decoder on MI355X (gfx950).

    from machserve_amd import generate
    outputs = generate("path/to/model", [[1, 2, 3]], max_new=16)
"""
from __future__ import annotations

from typing import List, Optional, Sequence

__version__ = "0.1.0"


def generate(model, prompts: Sequence[Sequence[int]], max_new: int, temperature: float = 0.0, seed: int = 0,
             eos: Optional[int] = None, *, dtype="bfloat16", **options) -> List[List[int]]:
    """Token ids generated for each prompt.  ``model`` is a model folder (config.json and
    model.safetensors) or an :class:`machserve_amd.engine.Engine`.  ``temperature <= 0`` is
    greedy; ``seed`` seeds the first prompt's generator, the i-th gets ``seed + i``
    (0: the request's id).  Further ``options``: top_k, top_p, presence_penalty,
    frequency_penalty, stop_seqs for sampling, and page_size, num_pages, max_tokens, capacity,
    max_batch_tokens, chunk_size for a model folder."""
    from .engine import Engine
    sampling = {k: options.pop(k) for k in ("top_k", "top_p", "presence_penalty", "frequency_penalty", "stop_seqs")
                if k in options}
    if isinstance(model, Engine):
        if options:
            raise TypeError(f"options {sorted(options)} apply to a model folder, not to a built engine")
        engine = model
    else:
        if "max_tokens" not in options and "num_pages" not in options:
            page = options.get("page_size", 64)
            options["max_tokens"] = sum((len(p) + max_new + page - 1) // page * page for p in prompts)
        engine = Engine.from_dir(model, dtype=dtype, **options)
    return engine.generate(prompts, max_new, temperature, seed, eos, **sampling)
