"""
Neighborhood plans: the run-length form of psi that the kernels consume, built once per
(col_idx, row_off) pair by the C++ builder in libs2attn.so and cached.

The reference re-sorts the CSR rows by length on the device on every call
(attention_cuda_utils.cu:74-113).  Here the conversion happens on the host the first time
a psi is seen (one device-to-host copy of the two index tensors) and later calls reuse the
device-resident plan.  A cache entry keeps its col_idx/row_off tensors alive, so their
addresses cannot be recycled for a different psi while the entry exists, and an in-place
edit of either tensor changes its version counter and misses the cache.
"""

import threading
from collections import OrderedDict

import torch

from . import _lib

_MAX_ENTRIES = 32
_cache = OrderedDict()
_lock = threading.Lock()


def _version(t: torch.Tensor) -> int:
    """Version counter of a tensor for the cache keys; inference tensors have none (reading it raises) and cannot be edited in place while tracked."""
    return 0 if t.is_inference() else t._version


class Plan:
    """Six int32 arrays plus the two interleaved launch orders on one device, and the ctypes view the library takes."""

    def __init__(self, arrays, nruns, ndense, keepalive, mixed):
        self.gather_off, self.gather_runs, self.gather_order, self.scatter_off, self.scatter_runs, self.scatter_order = arrays
        self.gather_order_mixed, self.scatter_order_mixed = mixed
        self.nruns = nruns
        self.gather_ndense, self.scatter_ndense = ndense
        self._keepalive = keepalive
        self.struct = _lib.PlanStruct(
            self.gather_off.data_ptr(),
            self.gather_runs.data_ptr(),
            self.gather_order.data_ptr(),
            self.scatter_off.data_ptr(),
            self.scatter_runs.data_ptr(),
            self.scatter_order.data_ptr(),
            nruns,
            self.gather_ndense,
            self.scatter_ndense,
            self.gather_order_mixed.data_ptr(),
            self.scatter_order_mixed.data_ptr(),
        )


def build_host_plan(col_idx: torch.Tensor, row_off: torch.Tensor, nlat_in: int, nlon_in: int, nlat_out: int, nlon_out: int, with_mixed: bool = False):
    """
    Runs the library's host builder on CPU copies of the CSR.  Returns
    ([gather_off, gather_runs, gather_order, scatter_off, scatter_runs, scatter_order], nruns, (gather_ndense, scatter_ndense))
    as CPU int32 tensors; gather_runs has shape (nruns, 4) = (virtual input latitude, ws, len, real input latitude),
    grouped by virtual output latitude; scatter_runs (virtual output latitude, ws, len, real output latitude), grouped by
    virtual input latitude.  Virtual latitude = real latitude * ratio + column class on the finer of the two grids (see
    include/s2attn.h); the first *_ndense entries of each order are the latitudes with long runs.  with_mixed: a fourth
    element (gather_order_mixed, scatter_order_mixed), the same latitudes with long-run and short-run ones interleaved in
    proportion to their work (the launch order of the kernels that split their work between matrix cores and vector ALU).
    """
    lib = _lib.load()
    ci = col_idx.detach().to(device="cpu", dtype=torch.int64).contiguous()
    ro = row_off.detach().to(device="cpu", dtype=torch.int64).contiguous()
    up = nlon_out % max(nlon_in, 1) == 0 and nlon_out != nlon_in  # scatter direction: the CSR is keyed by input latitude
    nrow = nlat_in if up else nlat_out
    if ro.numel() != nrow + 1:
        raise RuntimeError(f"row_off must have {'nlat_in' if up else 'nlat_out'} + 1 = {nrow + 1} entries, got {ro.numel()}")
    nnz = ci.numel()
    nvin = nlat_in * (1 if up else max(nlon_in // max(nlon_out, 1), 1))
    nvout = nlat_out * (nlon_out // nlon_in if up else 1)
    nruns = lib.s2attn_plan_count(ci.data_ptr(), ro.data_ptr(), nnz, nlat_in, nlon_in, nlat_out, nlon_out)
    _lib.check(nruns, "s2attn_plan_count")
    arrays = [
        torch.zeros(nvout + 1, dtype=torch.int32),
        torch.zeros((max(nruns, 1), 4), dtype=torch.int32),
        torch.zeros(nvout, dtype=torch.int32),
        torch.zeros(nvin + 1, dtype=torch.int32),
        torch.zeros((max(nruns, 1), 4), dtype=torch.int32),
        torch.zeros(nvin, dtype=torch.int32),
    ]
    ndense = torch.zeros(2, dtype=torch.int32)
    mixed = (torch.zeros(nvout, dtype=torch.int32), torch.zeros(nvin, dtype=torch.int32))
    rc = lib.s2attn_plan_build(
        ci.data_ptr(), ro.data_ptr(), nnz, nlat_in, nlon_in, nlat_out, nlon_out, nruns, *[a.data_ptr() for a in arrays], ndense.data_ptr(),
        mixed[0].data_ptr() if with_mixed else None, mixed[1].data_ptr() if with_mixed else None,
    )  # fmt: skip
    _lib.check(rc, "s2attn_plan_build")
    if with_mixed:
        return arrays, int(nruns), (int(ndense[0]), int(ndense[1])), mixed
    return arrays, int(nruns), (int(ndense[0]), int(ndense[1]))


def get_plan(col_idx: torch.Tensor, row_off: torch.Tensor, nlat_in: int, nlon_in: int, nlat_out: int, nlon_out: int) -> Plan:
    """Device plan for this psi, from the cache when the same tensors were seen before."""
    key = (
        col_idx.data_ptr(),
        row_off.data_ptr(),
        col_idx.numel(),
        row_off.numel(),
        _version(col_idx),
        _version(row_off),
        str(col_idx.device),
        nlat_in,
        nlon_in,
        nlat_out,
        nlon_out,
    )
    with _lock:
        plan = _cache.get(key)
        if plan is not None:
            _cache.move_to_end(key)
            return plan
    arrays, nruns, ndense, mixed = build_host_plan(col_idx, row_off, nlat_in, nlon_in, nlat_out, nlon_out, with_mixed=True)
    dev = col_idx.device
    plan = Plan([a.to(dev) for a in arrays], nruns, ndense, (col_idx, row_off), [m.to(dev) for m in mixed])
    with _lock:
        _cache[key] = plan
        while len(_cache) > _MAX_ENTRIES:
            _cache.popitem(last=False)
    return plan


def get_transposed_csr(col_idx: torch.Tensor, row_off: torch.Tensor, modulus: int, key_lo: int, nkeys: int):
    """
    The CSR entries regrouped by key = col // modulus (the latitude named in col), for the ring-step kernels that gather
    over the grid psi is not keyed by: (t_lat int32, t_lon int32, t_off int64 of nkeys + 1 entries, t_order int32) with the
    entries of key key_lo + i at t_off[i] .. t_off[i + 1], in CSR order, as (CSR row of the entry, col mod modulus), and
    t_order the keys by decreasing number of entries; see include/s2attn.h.  Built with device operations only (no host round trip) the first time a psi is seen, then served
    from the same cache as the plans.
    """
    key = ("transposed", col_idx.data_ptr(), row_off.data_ptr(), col_idx.numel(), row_off.numel(), _version(col_idx), _version(row_off),
           str(col_idx.device), modulus, key_lo, nkeys)  # fmt: skip
    with _lock:
        hit = _cache.get(key)
        if hit is not None:
            _cache.move_to_end(key)
            return hit[:4]
    dev, nnz, nrow = col_idx.device, col_idx.numel(), row_off.numel() - 1
    rows = torch.repeat_interleave(torch.arange(nrow, device=dev, dtype=torch.int32), row_off[1:] - row_off[:-1], output_size=nnz)
    lat = torch.div(col_idx, modulus, rounding_mode="floor")
    order = torch.argsort(lat, stable=True)
    t_lat = rows[order].contiguous()
    t_lon = (col_idx - lat * modulus)[order].to(torch.int32).contiguous()
    t_off = torch.searchsorted(lat[order], torch.arange(key_lo, key_lo + nkeys + 1, device=dev, dtype=lat.dtype)).contiguous()
    t_order = torch.argsort(t_off[1:] - t_off[:-1], descending=True, stable=True).to(torch.int32).contiguous()  # launch order: longest rows first
    entry = (t_lat, t_lon, t_off, t_order, (col_idx, row_off))  # the CSR tensors stay alive with the entry: their addresses cannot be recycled
    with _lock:
        _cache[key] = entry
        while len(_cache) > _MAX_ENTRIES:
            _cache.popitem(last=False)
    return entry[:4]


def get_row_order(row_off: torch.Tensor) -> torch.Tensor:
    """CSR rows by decreasing number of entries (int32, on row_off's device), cached per row_off."""
    key = ("order", row_off.data_ptr(), row_off.numel(), _version(row_off), str(row_off.device))
    with _lock:
        hit = _cache.get(key)
        if hit is not None:
            _cache.move_to_end(key)
            return hit[0]
    order = torch.argsort(row_off[1:] - row_off[:-1], descending=True, stable=True).to(torch.int32).contiguous()
    with _lock:
        _cache[key] = (order, row_off)
        while len(_cache) > _MAX_ENTRIES:
            _cache.popitem(last=False)
    return order


def clear_plan_cache() -> None:
    with _lock:
        _cache.clear()
