"""Typed descriptions of a model: what each part is and how the parts are arranged.

A :class:`ModelSpec` is pure data.  An architecture (see ``registry.py``) turns its
typed configuration into one; ``parts.model.DecoderModel`` builds the parts it names
from the part registries.  A spec of a part carries every size and constant of that
part, and ``tensors`` maps the part's own tensor names to names in the checkpoint, so
no part needs to know which model it belongs to.

Role in the reference: ``crates/mach-model/src/config.rs:15-142`` keeps one flat
struct for all families and dispatches inside one forward function; here the
per-layer choice is data.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Mapping, Optional, Sequence


class ConfigError(ValueError):
    """A configuration that cannot be built; the message names the key and the value."""


@dataclass(frozen=True)
class NormSpec:
    kind: str
    width: int
    eps: float
    tensors: Mapping[str, str] = field(default_factory=dict)


@dataclass(frozen=True)
class YarnSpec:
    """YaRN scaling of a rotation's frequencies (``crates/mach-server/src/startup.rs:172-199``): between the
    pair indices that ``beta_fast`` and ``beta_slow`` rotations over ``original_max_positions`` mark, a frequency
    goes over from its own value to ``1 / factor`` of it; cosines and sines are multiplied by
    ``mscale(factor, mscale) / mscale(factor, mscale_all_dim)`` with ``mscale(f, m) = 0.1 m ln f + 1``."""
    factor: float
    original_max_positions: int
    beta_fast: float = 32.0
    beta_slow: float = 1.0
    mscale: float = 1.0
    mscale_all_dim: float = 0.0


@dataclass(frozen=True)
class RotarySpec:
    """Rotation of pairs ``(j, j + rotary_dim/2)`` with ``freq_j = theta^(-2j/rotary_dim)``, or those frequencies
    scaled as ``yarn`` says."""
    kind: str
    head_dim: int
    theta: float
    tensors: Mapping[str, str] = field(default_factory=dict)
    yarn: Optional[YarnSpec] = None


@dataclass(frozen=True)
class AttentionSpec:
    """Grouped-query attention over a paged cache.

    ``window``: number of most recent keys a row may see (None = all).
    ``kv_source``: index of another layer whose cache this layer reads instead of
    writing its own (None = own cache).
    ``scale``: what the scores are multiplied by before the softmax (None = ``head_dim ** -0.5``,
    ``crates/mach-model/src/config.rs:231-234``).
    """
    kind: str
    hidden: int
    heads: int
    kv_heads: int
    head_dim: int
    position: Optional[RotarySpec]
    window: Optional[int] = None
    kv_source: Optional[int] = None
    tensors: Mapping[str, str] = field(default_factory=dict)
    scale: Optional[float] = None


@dataclass(frozen=True)
class GatedMlpSpec:
    """``down(act(gate(x)) * up(x))``."""
    kind: str
    hidden: int
    intermediate: int
    activation: str = "silu"
    tensors: Mapping[str, str] = field(default_factory=dict)


@dataclass(frozen=True)
class LayerSpec:
    """One pre-norm block: the specs of the four parts it arranges.  ``block`` names the registered arrangement,
    which builds its parts from the fields it reads; another arrangement brings a spec class of its own (any object
    with ``block`` and the fields that arrangement reads)."""
    block: str
    mixer: object
    feed_forward: object
    mixer_norm: object
    feed_forward_norm: object


@dataclass(frozen=True)
class EmbeddingSpec:
    """Token embedding: rows of a table, times ``scale``."""
    vocab: int
    width: int
    tensors: Mapping[str, str] = field(default_factory=dict)
    kind: str = "embedding"
    scale: float = 1.0


@dataclass(frozen=True)
class HeadSpec:
    """Output projection.  ``tied``: use the embedding table; ``tied=None``: use the head
    tensor if the checkpoint has it, else the embedding table."""
    vocab: int
    width: int
    tied: Optional[bool]
    tensors: Mapping[str, str] = field(default_factory=dict)
    kind: str = "linear"
    scale: float = 1.0  # the logits are multiplied by it


@dataclass(frozen=True)
class ModelSpec:
    architecture: str
    embedding: EmbeddingSpec
    layers: Sequence[LayerSpec]
    order: Sequence[int]
    final_norm: object
    head: HeadSpec
    max_positions: int

    def validate(self) -> None:
        n = len(self.layers)
        if not self.order:
            raise ConfigError("order: a model runs at least one layer")
        for i in self.order:
            if not 0 <= i < n:
                raise ConfigError(f"order names layer {i}, but there are {n} layers")
        for i, layer in enumerate(self.layers):
            src = getattr(getattr(layer, "mixer", None), "kv_source", None)
            if src is not None:
                if not 0 <= src < n or src == i:
                    raise ConfigError(f"layer {i}: kv_source {src} is not another layer")
                if getattr(getattr(self.layers[src], "mixer", None), "kv_source", None) is not None:
                    raise ConfigError(f"layer {i}: kv_source {src} itself reads another layer's cache")
                if self.order.index(src) > self.order.index(i):
                    raise ConfigError(f"layer {i} reads the cache of layer {src}, which runs later")
