"""Helpers shared by the GPU tests."""
from __future__ import annotations

import torch

DEV = "cuda:0"


def tol(dtype):
    """(relative to the largest reference magnitude, absolute floor) for one kernel's output.
    float32: rounding of sums of a few hundred terms in another order.  bfloat16: one rounding
    of the output to 8 bits of mantissa (2^-9 relative) on top of 32-bit accumulation; float16: the same
    with 11 bits (2^-12 relative)."""
    if dtype == torch.float32:
        return (2e-5, 1e-6)
    return (6e-3, 1e-5) if dtype == torch.bfloat16 else (8e-4, 1e-5)


def assert_close(got, ref, dtype, what=""):
    got, ref = got.float().cpu(), ref.float().cpu()
    rel, floor = tol(dtype)
    scale = ref.abs().max().item()
    err = (got - ref).abs().max().item()
    assert err <= rel * scale + floor, f"{what}: max error {err:.3e} over scale {scale:.3e} (allowed {rel * scale + floor:.3e})"
