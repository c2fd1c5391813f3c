"""RMS norm: ``y = x / sqrt(mean(x^2) + eps) * w`` with 32-bit statistics
(``crates/mach-model/src/kernels.rs:63-80``)."""
from __future__ import annotations

from .base import Norm, PendingNorm, TensorDecl
from .registry import register_norm


@register_norm("rmsnorm")
class RMSNorm(Norm):
    def tensor_decls(self):
        return [TensorDecl("weight", (self.spec.width,), "vector")]

    def load(self, tensors):
        self.weight = tensors["weight"]

    def forward(self, stream, rows=None):
        return stream.normed(self.weight, self.spec.eps, rows)

    def pending(self, stream):
        return PendingNorm(stream, self.weight, self.spec.eps)
