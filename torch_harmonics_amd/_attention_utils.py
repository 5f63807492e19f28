"""Argument checks and the backward context of the attention op (torch_harmonics/attention/_attention_utils.py:49-100)."""

import torch


def _check_ndim(tensor: torch.Tensor, ndim: int, name: str) -> None:
    """RuntimeError unless tensor has `ndim` dimensions; the message closes over plain ints only so dynamo can trace it."""
    actual = tensor.dim()
    torch._check(actual == ndim, lambda: f"Expected {ndim}-dimensional {name} tensor, got {actual} dimensions")


def _check_extent(tensor: torch.Tensor, dim: int, expected: int, name: str) -> None:
    """RuntimeError unless tensor.shape[dim] == expected (the actual extent may be symbolic and stays out of the message)."""
    expected = int(expected)
    torch._check(tensor.shape[dim] == expected, lambda: f"Expected {name} shape[{dim}] == {expected}")


def _dtype_mismatch_message() -> str:
    return "all attention inputs must share a single dtype"


def _check_dtypes_match(tensors) -> None:
    """RuntimeError unless all tensors share one dtype: the kernels read every activation as q's element type."""
    first = tensors[0].dtype
    for t in tensors[1:]:
        torch._check(t.dtype == first, _dtype_mismatch_message)


def _setup_context_attention_backward(ctx, inputs, output):
    kw, vw, qw, quad_weights, col_idx, row_off, nh, nlon_in, nlat_out, nlon_out = inputs
    ctx.save_for_backward(col_idx, row_off, quad_weights, kw, vw, qw)
    ctx.nh = nh
    ctx.nlon_in = nlon_in
    ctx.nlat_out = nlat_out
    ctx.nlon_out = nlon_out
