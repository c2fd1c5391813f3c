"""Grouped-query attention over the paged cache.

Per step (``crates/mach-model/src/batched.rs:3566-3679, 3819-3878, 4022-4031``):
q/k/v projection in one product with the biases in its epilogue, rotation of q and k fused
with the write of k and v into their pages, attention of every row over its request's
cache, output projection accumulated into the 32-bit stream.  Bias tensors are optional
and their presence decides (``crates/mach-model/src/weights.rs:30-31``).
"""
from __future__ import annotations

import torch

from .base import Mixer, PagedKVRequest, PendingNorm, SharedKVRequest, TensorDecl, require_kernel_sizes
from .registry import POSITION_ENCODINGS, register_mixer


@register_mixer("attention")
class Attention(Mixer):
    graph_safe = True  # reads positions and addresses from device memory only
    takes_pending_norm = True  # its first product can apply the norm of the stream itself

    def __init__(self, spec, rt):
        super().__init__(spec, rt)
        s = spec
        if s.heads % s.kv_heads:
            raise ValueError(f"attention: {s.heads} heads are not a multiple of {s.kv_heads} key/value heads")
        self.nq, self.nkv = s.heads * s.head_dim, s.kv_heads * s.head_dim
        require_kernel_sizes(rt, "attention", [("hidden size", s.hidden), ("heads x head size", self.nq)], s.head_dim,
                             rotated_row=self.nq + (2 * self.nkv if s.kv_source is None else 0))
        scale = getattr(s, "scale", None)
        self.scale = float(s.head_dim) ** -0.5 if scale is None else float(scale)
        self.position = POSITION_ENCODINGS.build(s.position, rt) if s.position is not None else None
        if self.position is not None:
            self.scale *= float(self.position.score_factor())
        self.writes_cache = s.kv_source is None
        self.group = None
        self.kpool = self.vpool = None

    def sub_parts(self):
        return [self.position] if self.position is not None else []

    def tensor_decls(self):
        s = self.spec
        decls = [TensorDecl("q.weight", (self.nq, s.hidden)), TensorDecl("o.weight", (s.hidden, self.nq)),
                 TensorDecl("q.bias", (self.nq,), "vector", optional=True)]
        if self.writes_cache:
            decls += [TensorDecl("k.weight", (self.nkv, s.hidden)), TensorDecl("v.weight", (self.nkv, s.hidden)),
                      TensorDecl("k.bias", (self.nkv,), "vector", optional=True),
                      TensorDecl("v.bias", (self.nkv,), "vector", optional=True)]
        return decls

    def load(self, t):
        names = ["q", "k", "v"] if self.writes_cache else ["q"]
        self.w_qkv = torch.cat([t[n + ".weight"] for n in names], dim=0).contiguous()
        if any(t.get(n + ".bias") is not None for n in names):
            dev = self.w_qkv.device
            self.b_qkv = torch.cat([t[n + ".bias"] if t.get(n + ".bias") is not None
                                    else torch.zeros(t[n + ".weight"].shape[0], dtype=torch.float32, device=dev)
                                    for n in names]).contiguous()
        else:
            self.b_qkv = None
        self.w_o = t["o.weight"]

    def cache_request(self):
        s = self.spec
        if not self.writes_cache:
            return SharedKVRequest(s.kv_source)
        return PagedKVRequest(s.kv_heads, s.head_dim, s.window)

    def bind_cache(self, binding):
        self.group, self.kpool, self.vpool = binding.group, binding.kpool, binding.vpool

    def attention_rows_per_token(self):
        return self.spec.heads // self.spec.kv_heads

    def attention_rows_per_block(self):
        return self.rt.ops.attention_rows_per_block(self.spec.head_dim)

    def forward(self, h, stream, ctx):
        s, ops = self.spec, self.rt.ops
        view = ctx.groups[self.group]
        g = self.attention_rows_per_token()
        # A step of many rows: the q/k/v product rotates and writes the cache in its own epilogue, where the kernels have
        # that form (the rows' angles come from a table that the step's layers share).
        takes = getattr(ops, "qkv_rope_takes", None)
        if (takes is not None and self.writes_cache and self.position is not None and not (ctx.decode_only and g <= ops.DECODE_MAX_GROUP)
                and takes(ctx.n_rows, s.heads, s.kv_heads, s.head_dim, self.w_qkv.shape[1])):
            inv_freq = self.position.rotary_inv_freq()
            if inv_freq is not None:
                key = ("rope table", inv_freq.data_ptr())
                if key not in ctx.shared:
                    ctx.shared[key] = ops.rope_table(ctx.position_axis(0), inv_freq)
                q = ops.linear_qkv_rope(h.tensor() if isinstance(h, PendingNorm) else h, self.w_qkv, self.b_qkv, ctx.shared[key],
                                        view.slot_map, self.kpool, self.vpool, s.heads, s.kv_heads, s.head_dim, view.page_size)
                o = ops.paged_attention(q, self.kpool, self.vpool, view.block_table, ctx.seq_q_start, ctx.seq_q_len, ctx.seq_pos0,
                                        ctx.attention_work[g], s.heads, s.kv_heads, s.head_dim, view.page_size, s.window, self.scale)
                stream.add_linear(o, self.w_o)
                return
        # [P, T, nq (+ 2 nkv)] partial sums, bias not yet added
        qkv = h.linear_split(self.w_qkv) if isinstance(h, PendingNorm) else ops.linear_split(h, self.w_qkv)
        inv_freq = self.position.rotary_inv_freq() if self.position is not None else None
        bias = self.b_qkv
        if self.position is not None and inv_freq is None:
            # a position encoding the fused kernel does not know: finish the sums, let the part
            # encode in place, then write without rotation
            qkv = qkv.sum(0, keepdim=True)
            if bias is not None:
                qkv += bias
                bias = None
            q = qkv[0, :, :self.nq].unflatten(1, (s.heads, s.head_dim))
            k = qkv[0, :, self.nq:self.nq + self.nkv].unflatten(1, (s.kv_heads, s.head_dim)) if self.writes_cache else None
            self.position.apply(q, k, ctx)
        decode = ctx.decode_only and g <= ops.DECODE_MAX_GROUP
        # the fused decode kernel rotates by the row's place in the cache: only where that is its position
        if decode and self.writes_cache and (self.position is None or (inv_freq is not None and ctx.positions_sequential)):
            o = ops.decode_attention_fused(qkv, bias, inv_freq, view.slot_map, self.kpool, self.vpool, view.block_table,
                                           ctx.seq_pos0, s.heads, s.kv_heads, s.head_dim, view.page_size, s.window,
                                           self.scale)
            stream.add_linear(o, self.w_o)
            return
        q = ops.rope_kv_write(qkv, bias, ctx.position_axis(0), inv_freq, view.slot_map if self.writes_cache else None,
                              self.kpool if self.writes_cache else None, self.vpool if self.writes_cache else None,
                              s.heads, s.kv_heads, s.head_dim, view.page_size)
        if decode:
            o = ops.decode_attention(q, self.kpool, self.vpool, view.block_table, ctx.seq_pos0, s.heads, s.kv_heads,
                                     s.head_dim, view.page_size, s.window, self.scale)
        else:
            o = ops.paged_attention(q, self.kpool, self.vpool, view.block_table, ctx.seq_q_start, ctx.seq_q_len,
                                    ctx.seq_pos0, ctx.attention_work[g], s.heads, s.kv_heads, s.head_dim, view.page_size,
                                    s.window, self.scale)
        stream.add_linear(o, self.w_o)
