"""Dense gated feed-forward ``down(act(gate(x)) * up(x))``, activation on the gate branch
(``crates/mach-model/src/batched.rs:4424-4453``; SiLU: ``crates/mach-model/src/kernels.rs:131-140``,
the tanh form of GELU: ``crates/mach-model/src/kernels.rs:199-208``).  Which activation is the
specification's to say.  Gate and up are one product whose epilogue applies the activation; down
accumulates into the 32-bit stream."""
from __future__ import annotations

from ..kernels.ops import GATE_ACTIVATIONS, interleave_gate_up
from .base import FeedForward, PendingNorm, TensorDecl, require_kernel_sizes
from .registry import register_feed_forward


@register_feed_forward("gated_mlp")
class GatedMlp(FeedForward):
    takes_pending_norm = True  # its first product can apply the norm of the stream itself

    def __init__(self, spec, rt):
        super().__init__(spec, rt)
        if spec.activation not in GATE_ACTIVATIONS:
            raise ValueError(f"gated_mlp: activation {spec.activation!r} is not built (built: {', '.join(sorted(GATE_ACTIVATIONS))})")
        require_kernel_sizes(rt, "gated_mlp", [("hidden size", spec.hidden), ("intermediate size", spec.intermediate)])

    def tensor_decls(self):
        s = self.spec
        return [TensorDecl("gate.weight", (s.intermediate, s.hidden)), TensorDecl("up.weight", (s.intermediate, s.hidden)),
                TensorDecl("down.weight", (s.hidden, s.intermediate))]

    def load(self, t):
        self.w_gate_up = interleave_gate_up(t["gate.weight"], t["up.weight"])
        self.w_down = t["down.weight"]

    def forward(self, h, stream, ctx):
        if isinstance(h, PendingNorm):
            a = h.linear_swiglu(self.w_gate_up, self.spec.intermediate, self.spec.activation)
        else:
            a = self.rt.ops.linear_swiglu(h, self.w_gate_up, self.spec.intermediate, self.spec.activation)
        stream.add_linear(a, self.w_down)
