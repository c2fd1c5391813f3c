from .ops import HipOps, KernelError, get_ops, interleave_gate_up

__all__ = ["HipOps", "KernelError", "get_ops", "interleave_gate_up"]
