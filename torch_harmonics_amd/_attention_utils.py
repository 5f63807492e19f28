"""Argument checks and the backward context of the attention op (torch_harmonics/attention/_attention_utils.py:49-100)."""

import torch


def _check_ndim(tensor: torch.Tensor, ndim: int, name: str) -> None:
    """RuntimeError unless tensor has `ndim` dimensions (a plain branch: dynamo folds it to a constant while tracing)."""
    if tensor.dim() != ndim:
        raise RuntimeError(f"Expected {ndim}-dimensional {name} tensor, got {tensor.dim()} dimensions")


def _check_extent(tensor: torch.Tensor, dim: int, expected: int, name: str) -> None:
    """RuntimeError unless tensor.shape[dim] == expected (under tracing the comparison becomes a shape guard)."""
    expected = int(expected)
    if tensor.shape[dim] != expected:
        raise RuntimeError(f"Expected {name} shape[{dim}] == {expected}, got {tensor.shape[dim]}")


def _check_dtypes_match(tensors) -> None:
    """RuntimeError unless all tensors share one dtype: the kernels read every activation as q's element type."""
    first = tensors[0].dtype
    for t in tensors[1:]:
        if t.dtype != first:
            raise RuntimeError("all attention inputs must share a single dtype")


def _setup_context_attention_backward(ctx, inputs, output):
    kw, vw, qw, quad_weights, col_idx, row_off, nh, nlon_in, nlat_out, nlon_out = inputs
    ctx.save_for_backward(col_idx, row_off, quad_weights, kw, vw, qw)
    ctx.nh = nh
    ctx.nlon_in = nlon_in
    ctx.nlat_out = nlat_out
    ctx.nlon_out = nlon_out
