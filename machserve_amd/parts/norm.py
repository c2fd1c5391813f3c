"""RMS norm: ``y = x / sqrt(mean(x^2) + eps) * w`` with 32-bit statistics
(``crates/mach-model/src/kernels.rs:63-80``), and the forms in which it is folded into the product that
reads it: the norm's factor is one number a row, so a product's kernel can apply it to its finished sums."""
from __future__ import annotations

from .base import Norm, PendingNorm, TensorDecl, require_kernel_sizes
from .registry import register_norm


@register_norm("rmsnorm")
class RMSNorm(Norm):
    def __init__(self, spec, rt):
        super().__init__(spec, rt)
        require_kernel_sizes(rt, "rmsnorm", norm_width=spec.width)

    def tensor_decls(self):
        return [TensorDecl("weight", (self.spec.width,), "vector")]

    def load(self, tensors):
        self.weight = tensors["weight"]

    def forward(self, stream, rows=None):
        """``rmsnorm(x) * weight`` of the stream with everything added (of its ``rows`` if given), in the
        element type; partial sums that are pending are added by the norm's own kernel."""
        stream.launch_deferred()
        h = stream.ops.rmsnorm(stream.x, self.weight, self.spec.eps, rows, False, stream.pending)
        if rows is None:
            stream.pending = None  # the kernel wrote the sum back
        return h

    def pending(self, stream):
        return PendingRMSNorm(self, stream)


class PendingRMSNorm(PendingNorm):
    """The RMS norm left to its reader's first product, folded into it where the kernels take the shape."""

    def linear_split(self, w):
        stream, ops, weight, eps = self.stream, self.stream.ops, self.norm.weight, self.norm.spec.eps
        stream.launch_deferred()
        T, K = stream.x.shape
        P = 0 if stream.pending is None else stream.pending.shape[0]
        if ops.norm_folds_into(T, w.shape[0], K, P):
            out, x_new = ops.linear_split_normed(stream.x, stream.pending, weight, eps, w)
            if x_new is not None:
                stream.x, stream.pending = x_new, None
            return out
        return ops.linear_split(self.tensor(), w)

    def linear_swiglu(self, w_gate_up, intermediate, activation="silu"):
        stream, ops, weight, eps = self.stream, self.stream.ops, self.norm.weight, self.norm.spec.eps
        if stream.deferred is not None and stream.pending is None:
            # a product that is still to be added: where the kernels can, it leaves what the norm needs beside its
            # sum, and the gated product applies the norm's factor to its own finished sums
            a, w = stream.deferred
            takes = getattr(ops, "prenorm_swiglu_takes", None)
            if takes is not None and takes(a.shape[0], w.shape[0], w.shape[1], w_gate_up.shape[0]):
                stream.deferred = None
                hn, row_ss = ops.linear_residual_prenorm(a, w, stream.x, weight)
                return ops.linear_swiglu_scaled(hn, row_ss, eps, w_gate_up, intermediate, activation)
        stream.launch_deferred()
        T, K = stream.x.shape
        P = 0 if stream.pending is None else stream.pending.shape[0]
        if ops.norm_folds_into(T, w_gate_up.shape[0], K, P):
            out, x_new = ops.linear_swiglu_normed(stream.x, stream.pending, weight, eps, w_gate_up, intermediate, activation)
            if x_new is not None:
                stream.x, stream.pending = x_new, None
            return out
        return ops.linear_swiglu(self.tensor(), w_gate_up, intermediate, activation)
