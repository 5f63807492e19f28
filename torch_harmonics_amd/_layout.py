"""
NCHW <-> NHWC conversion at the module boundary (torch_harmonics/attention/_layout.py:137-184).

Layout is stated by the caller, never inferred from strides; both functions always return
freshly allocated storage, also when a degenerate shape makes the two layouts byte-identical.
"""

import torch

from . import ops

__all__ = ["to_nhwc", "to_nchw"]


def to_nhwc(x: torch.Tensor) -> torch.Tensor:
    """(B, C, H, W) contiguous -> (B, H, W, C) contiguous, same values."""
    torch._check(x.dim() == 4, lambda: "to_nhwc expects a 4-dimensional (B, C, H, W) tensor")
    return ops.permute_to_nhwc(x.contiguous())


def to_nchw(x: torch.Tensor) -> torch.Tensor:
    """(B, H, W, C) contiguous -> (B, C, H, W) contiguous, same values."""
    torch._check(x.dim() == 4, lambda: "to_nchw expects a 4-dimensional (B, H, W, C) tensor")
    return ops.permute_to_nchw(x.contiguous())
