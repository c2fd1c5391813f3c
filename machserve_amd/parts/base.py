"""Interfaces of the parts a decoder is put together from.

A part is built from its spec (``config.specs``) and a :class:`Runtime`; it declares the
tensors it needs by its *own* names, receives them from the loader, and runs on a
:class:`StepContext`.  A part never looks at the model around it: sizes and constants
come from its spec, positions and cache addresses from the context.

Adding a part: subclass the matching base class, give it the methods below, and register
it under a ``kind`` in ``parts.registry``; a spec whose ``kind`` names it is all a model
needs to use it.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Dict, List, Mapping, Optional, Tuple

import torch


@dataclass(frozen=True)
class TensorDecl:
    """A tensor a part wants.  ``role`` decides how it is kept on the device: a 'matrix'
    (operand of a matrix product, or the embedding table) in the element type of the
    run, a 'vector' (norm weight, bias) in float32, a 'table' of integers in int32."""
    name: str
    shape: Tuple[int, ...]
    role: str = "matrix"
    optional: bool = False


@dataclass
class Runtime:
    """What a part gets from its surroundings: the device, the element type and the kernels."""
    device: torch.device
    dtype: torch.dtype
    ops: object


@dataclass(frozen=True)
class PagedKVRequest:
    """A mixer's need of a paged cache: K and V per token, all keys or a window of them.  ``v_head_dim``
    is the width of a value where it differs from a key's ``head_dim`` (a compressed or latent cache)."""
    kv_heads: int
    head_dim: int
    window: Optional[int] = None
    v_head_dim: Optional[int] = None


@dataclass(frozen=True)
class SharedKVRequest:
    """A mixer that reads the cache another layer writes."""
    source_layer: int


@dataclass(frozen=True)
class StateRequest:
    """A mixer's need of per-request state of fixed size: one tensor ``[slots, *shape]``
    per entry, zeroed when a request takes the slot."""
    shapes: Mapping[str, Tuple[int, ...]]
    dtype: torch.dtype = torch.float32


@dataclass
class GroupView:
    """Addresses of one cache group for the rows and requests of a step."""
    page_size: int
    slot_map: torch.Tensor     # int32 [T]: page * page_size + offset where each row's key goes
    block_table: torch.Tensor  # int32 [S, P]: pages of each request of the step, -1 = none


@dataclass
class StepContext:
    """Everything about one step that parts may read.  Device tensors are int32.

    Rows are the tokens of the step; requests are listed in the order of their rows, and a
    request's rows are contiguous and in position order.
    """
    n_rows: int
    n_seqs: int
    tokens: torch.Tensor        # [T]
    positions: torch.Tensor     # [T, axes]: what a position encoding encodes; one axis unless the model asks for more
    seq_q_start: torch.Tensor   # [S] first row of each request
    seq_q_len: torch.Tensor     # [S] number of its rows
    seq_pos0: torch.Tensor      # [S] position of its first row
    seq_slot: torch.Tensor      # [S] state slot of each request
    want_rows: torch.Tensor     # [W] rows whose logits are wanted
    groups: Dict[str, GroupView] = field(default_factory=dict)
    attention_work: Dict[int, torch.Tensor] = field(default_factory=dict)  # rows per token -> [n, 2]
    host: Dict[str, object] = field(default_factory=dict)  # the same lists on the host
    decode_only: bool = False
    # True: every row's position is, on every axis, its index in its request's cache (``seq_pos0`` onwards), so a
    # kernel may take positions from there; False: the caller gave positions of its own for some rows
    positions_sequential: bool = True
    # what parts have worked out from this step's rows and share between layers (a table of the rows' rotation angles)
    shared: Dict[object, object] = field(default_factory=dict)

    def position_axis(self, axis: int = 0) -> torch.Tensor:
        """``[T]`` positions along one axis, contiguous."""
        if self.positions.dim() == 1:
            return self.positions
        if self.positions.shape[1] == 1:
            return self.positions.view(-1)
        return self.positions[:, axis].contiguous()


class ResidualStream:
    """The 32-bit residual stream ``x [T, width]`` and what is still to be added to it.

    ``add_linear`` does not launch its product at once but when the stream is next read.  With
    few rows the product leaves partial sums (``pending``) that a reading norm may add in its
    own kernel, which saves a pass over the stream; with many rows the product adds to the
    stream in its epilogue.  A reader that knows nothing of this calls ``value()``.
    """

    def __init__(self, x: torch.Tensor, ops):
        self.x = x
        self.ops = ops
        self.deferred = None                         # (a, w): x += a @ w.T, not yet launched
        self.pending: Optional[torch.Tensor] = None  # float32 [P, T, width], not yet added

    def add_linear(self, a: torch.Tensor, w: torch.Tensor) -> None:
        """``x += a @ w.T``."""
        self.flush()
        self.deferred = (a, w)

    def add(self, y: torch.Tensor) -> None:
        """``x += y`` for a part that computes its output by other means."""
        self.flush()
        self.x += y.to(self.x.dtype)

    def launch_deferred(self) -> None:
        """Launch the product that ``add_linear`` left, if any; its sum may stay pending as partial sums."""
        if self.deferred is not None:
            a, w = self.deferred
            self.deferred = None
            self.pending = self.ops.linear_residual(a, w, self.x)

    def flush(self) -> None:
        self.launch_deferred()
        if self.pending is not None:
            self.ops.add_partials(self.x, self.pending)
            self.pending = None

    def value(self) -> torch.Tensor:
        self.flush()
        return self.x


class PendingNorm:
    """The normalised stream, not yet computed: a part that starts with a product over it (``takes_pending_norm``)
    gets this instead of a tensor, so that a norm whose kernels can do so is applied inside the product.  This base
    form runs the norm by itself and then the plain product; a norm with fused forms of its own returns a subclass
    from ``Norm.pending``."""

    def __init__(self, norm: "Norm", stream: ResidualStream):
        self.norm, self.stream = norm, stream

    def tensor(self) -> torch.Tensor:
        return self.norm.forward(self.stream)

    def linear_split(self, w: torch.Tensor) -> torch.Tensor:
        """``norm(x) @ w.T`` as float32 ``[P, T, N]`` partial sums."""
        return self.stream.ops.linear_split(self.tensor(), w)

    def linear_swiglu(self, w_gate_up: torch.Tensor, intermediate: int, activation: str = "silu") -> torch.Tensor:
        """``act(h @ gate.T) * (h @ up.T)`` for ``h = norm(x)``."""
        return self.stream.ops.linear_swiglu(self.tensor(), w_gate_up, intermediate, activation)


def require_kernel_sizes(rt: "Runtime", what: str, reductions=(), head_dim: Optional[int] = None,
                         norm_width: Optional[int] = None, rotated_row: Optional[int] = None) -> None:
    """Lets the kernels refuse sizes they do not take while the model is built, with the size's name
    (``reductions``: pairs of name and size that products sum over; ``norm_width``: the width of a row that is
    normalised; ``rotated_row``: the width of a row of q, k and v), rather than at the first step."""
    check = getattr(rt.ops, "require_sizes", None)
    if check is not None:
        check(what, reductions, head_dim, norm_width, rotated_row)


class Part:
    takes_pending_norm = False  # True: forward's normalised input may be a PendingNorm

    def __init__(self, spec, rt: Runtime):
        self.spec = spec
        self.rt = rt

    def tensor_decls(self) -> List[TensorDecl]:
        return []

    def load(self, tensors: Dict[str, Optional[torch.Tensor]]) -> None:
        """Receive the declared tensors (absent optional ones are None), already on the
        device in the dtype of their role."""


class Norm(Part):
    def forward(self, stream: ResidualStream, rows: Optional[torch.Tensor] = None) -> torch.Tensor:
        """Normalised copy of the stream (of its ``rows`` if given), in the element type.  Pending
        sums of the stream are folded in."""
        raise NotImplementedError

    def pending(self, stream: ResidualStream) -> Optional[PendingNorm]:
        """The same, left to the reader's first product, if this norm can be folded into one."""
        return None


class PositionEncoding(Part):
    axes = 1  # numbers per position this encoding reads; the step's positions are [T, max over the model's encodings]

    def rotary_inv_freq(self) -> Optional[torch.Tensor]:
        """``[head_dim / 2]`` inverse frequencies if this is a plain rotation that the fused
        kernel can apply; None otherwise (then :meth:`apply` is called)."""
        return None

    def apply(self, q: torch.Tensor, k: Optional[torch.Tensor], ctx: StepContext) -> None:
        """Encode positions in place into ``q [T, H, hd]`` and ``k [T, KV, hd]`` (float32 views)."""
        raise NotImplementedError

    def score_factor(self) -> float:
        """What the encoding multiplies every score by, beside what it does to q and k (1: nothing)."""
        return 1.0


class Mixer(Part):
    """Mixes information between positions of one request (attention, or a recurrence)."""

    def cache_request(self):
        """PagedKVRequest, SharedKVRequest, StateRequest, None, or a list of these (pages and state together,
        or several caches of different widths)."""
        return None

    def bind_cache(self, binding) -> None:
        """Receive what the cache manager made for :meth:`cache_request`: one binding, or for a list of
        requests the list of their bindings in the same order."""

    def attention_rows_per_token(self) -> Optional[int]:
        """Query heads per KV head if the mixer needs attention work lists, else None."""
        return None

    def attention_rows_per_block(self) -> Optional[int]:
        """Flat rows (token x head of a group) that one block of the mixer's attention kernel takes: the
        unit in which the step's work lists are cut.  None if the mixer needs no work lists."""
        return None

    def forward(self, h: torch.Tensor, stream: ResidualStream, ctx: StepContext) -> None:
        """Add the mixer's output for the normalised input ``h`` into the stream
        (``stream.add_linear`` for a final projection, ``stream.add`` for a finished tensor)."""
        raise NotImplementedError


class FeedForward(Part):
    def forward(self, h: torch.Tensor, stream: ResidualStream, ctx: StepContext) -> None:
        """Add the feed-forward's output for the normalised input ``h`` into the stream."""
        raise NotImplementedError


class Block:
    """An arrangement of parts around the stream.  A block is built from its layer's spec and the runtime and
    **builds its own parts** from the fields of that spec, which belong to it: the model around it asks only for what
    is below, so an arrangement with other parts (a norm after each branch, one norm for parallel branches, no
    feed-forward, two mixers side by side) is a registered class and a spec with the fields it reads, with ``block``
    naming its kind.

    The defaults serve a block with at most one mixer in ``self.mixer``; a block with several overrides
    :meth:`mixers`, and :meth:`cache_request` / :meth:`bind_cache` deal the requests and bindings out in order."""

    mixer: Optional[Mixer] = None

    def __init__(self, spec, rt: Runtime):
        self.spec, self.rt = spec, rt

    def parts(self) -> List[Part]:
        """Every part of the block that declares tensors (sub-parts of parts excepted: they list their own)."""
        raise NotImplementedError

    def mixers(self) -> List[Mixer]:
        return [self.mixer] if self.mixer is not None else []

    def cache_request(self):
        """What the block's mixers ask of the cache manager: one mixer's request as it is, several mixers' requests
        as one flat list (:meth:`bind_cache` deals the bindings back out)."""
        ms = self.mixers()
        if len(ms) <= 1:
            return ms[0].cache_request() if ms else None
        out = []
        for m in ms:
            r = m.cache_request()
            out.extend(r if isinstance(r, (list, tuple)) else [r])
        return out

    def bind_cache(self, binding) -> None:
        ms = self.mixers()
        if len(ms) == 1:
            ms[0].bind_cache(binding)
            return
        at = 0
        for m in ms:
            r = m.cache_request()
            if isinstance(r, (list, tuple)):
                m.bind_cache(binding[at:at + len(r)])
                at += len(r)
            else:
                if binding[at] is not None:
                    m.bind_cache(binding[at])
                at += 1

    @property
    def graph_safe(self) -> bool:
        """Whether every mixer reads nothing but device memory from the step (its steps may then be captured)."""
        return all(getattr(m, "graph_safe", False) for m in self.mixers())

    def forward(self, stream: ResidualStream, ctx: StepContext) -> None:
        raise NotImplementedError
