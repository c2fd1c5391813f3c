"""A decoder built from a :class:`ModelSpec`: embedding, blocks chosen layer by layer from
the registries, final norm, output head.  ``order`` is the list of layers a step runs; it
may name a layer twice.  Only the rows whose logits are wanted reach the head
(the reference computes the head for every row, ``crates/mach-model/src/batched.rs:4594-4626``).
"""
from __future__ import annotations

from typing import List, Optional

import torch

from ..config.specs import ModelSpec
from .base import Block, Part, ResidualStream, Runtime, StepContext, TensorDecl, require_kernel_sizes
from .registry import BLOCKS, EMBEDDINGS, HEADS, NORMS, register_embedding, register_head


@register_embedding("embedding")
class Embedding(Part):
    """Rows of a table, times the spec's ``scale`` (1 for an embedding that is not scaled)."""

    def tensor_decls(self):
        return [TensorDecl("weight", (self.spec.vocab, self.spec.width), "matrix")]

    def load(self, t):
        self.weight = t["weight"]

    def forward(self, tokens: torch.Tensor) -> torch.Tensor:
        return self.rt.ops.embed(tokens, self.weight, getattr(self.spec, "scale", 1.0))


@register_head("linear")
class Head(Part):
    """Output projection, times the spec's ``scale``; tied to the embedding table when the spec says so, or
    when it leaves it open and the checkpoint has no head tensor
    (``crates/mach-model/src/loader.rs:1025-1033``).  A head is built with the model's embedding part as
    its third argument and has ``forward(h) -> float32 logits`` and ``vocab`` in its spec."""

    def __init__(self, spec, rt, embedding):
        super().__init__(spec, rt)
        self.embedding = embedding
        self.weight = None

    def tensor_decls(self):
        if self.spec.tied is True:
            return []
        return [TensorDecl("weight", (self.spec.vocab, self.spec.width), "matrix", optional=self.spec.tied is None)]

    def ignored_tensors(self):
        """Checkpoint names that may be present without being used."""
        return [self.spec.tensors.get("weight", "weight")] if self.spec.tied is True else []

    def load(self, t):
        self.weight = t.get("weight")

    def forward(self, h: torch.Tensor) -> torch.Tensor:
        w = self.weight if self.weight is not None else self.embedding.weight
        logits = self.rt.ops.linear(h, w, None, out_f32=True)
        scale = getattr(self.spec, "scale", 1.0)
        if scale != 1.0:
            logits *= scale
        return logits


class DecoderModel:
    def __init__(self, spec: ModelSpec, rt: Runtime):
        spec.validate()
        self.spec, self.rt = spec, rt
        require_kernel_sizes(rt, "output head", [("width", spec.embedding.width)])
        self.embedding = EMBEDDINGS.build(spec.embedding, rt)
        self.blocks: List[Block] = []
        for layer in spec.layers:  # a block builds its own parts from the fields of its layer's spec
            self.blocks.append(BLOCKS.get(layer.block)(layer, rt))
        self.order = list(spec.order)
        self.final_norm = NORMS.build(spec.final_norm, rt)
        self.head = HEADS.build(spec.head, rt, self.embedding)
        self._bindings, self._rebind = [], False
        # Debugging aid: a callable (name, float32 stream [rows, width]) that sees the residual stream after the
        # embedding and after every run of a layer (crates/mach-model/src/batched.rs:3040-3088 dumps the same
        # points).  While it is set the step function runs every step as it is, from no captured graph.
        self.observer = None

    # ------------------------------------------------------------------ structure
    def parts(self) -> List[Part]:
        out: List[Part] = [self.embedding]
        for b in self.blocks:
            for p in b.parts():
                out.append(p)
                out.extend(getattr(p, "sub_parts", lambda: [])())
        out += [self.final_norm, self.head]
        return out

    def cache_requests(self):
        """One cache request per *position of the order*: a layer that runs twice shares its
        weights between the two runs, but each run keeps a cache (or state) of its own, so
        what a run reads never depends on how the tokens were cut into steps.  A layer that
        reads another layer's cache reads that of the layer's latest earlier run."""
        from .base import SharedKVRequest

        def placed(req, p, i):
            if isinstance(req, SharedKVRequest):
                earlier = [q for q in range(p) if self.order[q] == req.source_layer]
                if not earlier:
                    raise ValueError(f"layer {i} reads the cache of layer {req.source_layer}, which has not run before it")
                return SharedKVRequest(earlier[-1])
            return req

        out = []
        for p, i in enumerate(self.order):
            req = self.blocks[i].cache_request()
            out.append([placed(r, p, i) for r in req] if isinstance(req, (list, tuple)) else placed(req, p, i))
        return out

    def bind_cache(self, device_cache) -> None:
        self._bindings = [device_cache.binding(p) for p in range(len(self.order))]
        for p, i in enumerate(self.order):  # a layer that runs once keeps its binding for good
            if self._bindings[p] is not None:
                self.blocks[i].bind_cache(self._bindings[p])
        self._rebind = len(set(self.order)) != len(self.order)

    def attention_rows_per_token(self) -> List[int]:
        return sorted({g for b in self.blocks for m in b.mixers() for g in [m.attention_rows_per_token()] if g})

    def attention_rows_per_block(self) -> Optional[int]:
        """The unit of the attention work lists, which every mixer's kernel must share (the lists are made
        once per step); None if no mixer wants them."""
        units = {(u, type(m).__name__, getattr(m.spec, "head_dim", None))
                 for b in self.blocks for m in b.mixers() for u in [m.attention_rows_per_block()] if u}
        if len({u for u, _, _ in units}) > 1:
            raise ValueError("the mixers' attention kernels take blocks of different numbers of rows: "
                             + ", ".join(f"{name} (head size {hd}): {u}" for u, name, hd in sorted(units)))
        return next(iter(units))[0] if units else None

    def position_axes(self) -> int:
        """Numbers per position of a step: the most that any position encoding of the model reads."""
        return max([getattr(p, "axes", 1) for p in self.parts()] + [1])

    @property
    def vocab(self) -> int:
        return self.spec.head.vocab

    # ------------------------------------------------------------------ the forward pass
    def forward(self, ctx: StepContext) -> Optional[torch.Tensor]:
        """Run the step's rows through the layers in ``order``; float32 logits ``[W, vocab]`` of
        the wanted rows, or None when none is wanted."""
        # What the layers of one pass share (a table of the rows' rotation angles) is made anew in every pass: a context
        # is run once to load everything and once more under capture, and what the first run left would be missing
        # from the captured graph, which would then rotate every later step by the first step's positions.
        ctx.shared.clear()
        stream = ResidualStream(self.embedding.forward(ctx.tokens), self.rt.ops)
        watch = self.observer
        if watch is not None:
            watch("embedding", stream.value())
        for p, i in enumerate(self.order):
            if self._rebind and self._bindings[p] is not None:
                self.blocks[i].bind_cache(self._bindings[p])
            self.blocks[i].forward(stream, ctx)
            if watch is not None:  # the sums still pending are added first: the value is the whole stream
                watch(f"layer{p:02d}", stream.value())
        if ctx.want_rows.numel() == 0:
            return None
        return self.head.forward(self.final_norm.forward(stream, rows=ctx.want_rows))
