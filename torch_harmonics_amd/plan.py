"""
Neighborhood plans: the run-length form of psi that the kernels consume, built once per
(col_idx, row_off) pair by the C++ builder in libs2attn.so (one position-independent int32
array, see include/s2attn.h) and cached.

The reference re-sorts the CSR rows by length on the device on every call
(attention_cuda_utils.cu:74-113).  Here the conversion happens on the host the first time
a psi is seen (one device-to-host copy of the two index tensors) and later calls reuse the
device-resident plan.  A cache entry keeps its col_idx/row_off tensors alive, so their
addresses cannot be recycled for a different psi while the entry exists, and an in-place
edit of either tensor changes its version counter and misses the cache.
"""

import hashlib
import os
import tempfile
import threading
from collections import OrderedDict

import numpy as np
import torch

from . import _lib

_MAX_ENTRIES = 32
_cache = OrderedDict()
_lock = threading.Lock()


def _version(t: torch.Tensor) -> int:
    """Version counter of a tensor for the cache keys; inference tensors have none (reading it raises) and cannot be edited in place while tracked."""
    return 0 if t.is_inference() else t._version


class Plan:
    """The plan blob on one device (one int32 tensor), its header on the host, and the ctypes view the library takes."""

    def __init__(self, blob: torch.Tensor, header, keepalive=None):
        self.blob = blob
        self.header = tuple(int(x) for x in header)
        self._keepalive = keepalive
        self.struct = _lib.PlanStruct.make(blob.data_ptr(), self.header)

    def _array(self, off_field: str, n: int, width: int = 1) -> torch.Tensor:
        off = self.header[_lib.PH[off_field]]
        a = self.blob[off : off + n * width]
        return a.view(n, width) if width > 1 else a

    # views into the blob (see include/s2attn.h for their meaning)
    @property
    def nruns(self):
        return self.header[_lib.PH["NRUNS"]]

    def arrays(self):
        """(gather_off, gather_runs, gather_order, scatter_off, scatter_runs, scatter_order) as views of the blob."""
        h, PH = self.header, _lib.PH
        nvout, nvin, nruns = h[PH["NVOUT"]], h[PH["NVIN"]], h[PH["NRUNS"]]
        return [
            self._array("GATHER_OFF", nvout + 1), self._array("GATHER_RUNS", nruns, 4), self._array("GATHER_ORDER", nvout),
            self._array("SCATTER_OFF", nvin + 1), self._array("SCATTER_RUNS", nruns, 4), self._array("SCATTER_ORDER", nvin),
        ]  # fmt: skip

    def mixed_orders(self):
        h, PH = self.header, _lib.PH
        return self._array("GATHER_ORDER_MIXED", h[PH["NVOUT"]]), self._array("SCATTER_ORDER_MIXED", h[PH["NVIN"]])

    def items(self, side: str):
        """Work list of the hybrid kernels for side "GATHER" or "SCATTER": (items [n, 2] = (latitude, pair or -1),
        pair_off [npairs + 1], pair_runs [*, 8] = (lat, ws, len, aux, dA, lenA, dB, lenB))."""
        h, PH = self.header, _lib.PH
        n, npairs = h[PH[side + "_NITEMS"]], h[PH[side + "_NPAIRS"]]
        poff = self._array(side + "_PAIR_OFF", npairs + 1)
        return self._array(side + "_ITEMS", n, 2), poff, self._array(side + "_PAIR_RUNS", int(poff[-1]) if self.blob.device.type == "cpu" else 0, 8)

    def to(self, device) -> "Plan":
        return Plan(self.blob.to(device), self.header, self._keepalive)


def build_host_blob(col_idx: torch.Tensor, row_off: torch.Tensor, nlat_in: int, nlon_in: int, nlat_out: int, nlon_out: int) -> Plan:
    """Runs the library's host builder on CPU copies of the CSR and returns the plan with its blob in host memory."""
    lib = _lib.load()
    ci = col_idx.detach().to(device="cpu", dtype=torch.int64).contiguous()
    ro = row_off.detach().to(device="cpu", dtype=torch.int64).contiguous()
    up = nlon_out % max(nlon_in, 1) == 0 and nlon_out != nlon_in  # scatter direction: the CSR is keyed by input latitude
    nrow = nlat_in if up else nlat_out
    if ro.numel() != nrow + 1:
        raise RuntimeError(f"row_off must have {'nlat_in' if up else 'nlat_out'} + 1 = {nrow + 1} entries, got {ro.numel()}")
    args = (ci.data_ptr(), ro.data_ptr(), ci.numel(), nlat_in, nlon_in, nlat_out, nlon_out)
    n = lib.s2attn_plan_size(*args)
    _lib.check(n, "s2attn_plan_size")
    blob = torch.zeros(n, dtype=torch.int32)
    _lib.check(lib.s2attn_plan_build(*args, blob.data_ptr(), n), "s2attn_plan_build")
    return Plan(blob, blob[: _lib.PLAN_HEADER_INTS].tolist())


def _disk_cache_dir():
    """Directory of the on-disk plan cache: $S2ATTN_CACHE_DIR, else ~/.cache/torch_harmonics_amd; None when the variable is set to
    an empty string or "off" (no caching)."""
    d = os.environ.get("S2ATTN_CACHE_DIR")
    if d is None:
        home = os.path.expanduser("~")
        if not os.path.isabs(home):  # no home directory known: no default cache (never a directory named "~" under the working directory)
            return None
        d = os.path.join(home, ".cache", "torch_harmonics_amd")
    return None if d in ("", "off") else d


def cached_host_blob(key, col_idx: torch.Tensor, row_off: torch.Tensor, nlat_in: int, nlon_in: int, nlat_out: int, nlon_out: int) -> Plan:
    """build_host_blob with the blob kept on disk between processes.  `key` names the psi (a module passes its grids, shapes
    and cutoff); the file name also carries the library's ABI version, the plan format and the psi's size, and a file whose
    header does not describe this problem is ignored and rewritten.  Any I/O failure falls back to building in memory."""
    d = _disk_cache_dir()
    if d is None:
        return build_host_blob(col_idx, row_off, nlat_in, nlon_in, nlat_out, nlon_out)
    ident = repr((key, _lib.ABI_VERSION, _lib.PLAN_MAGIC, int(col_idx.numel()), int(row_off.numel()), nlat_in, nlon_in, nlat_out, nlon_out))
    path = os.path.join(d, "plan_" + hashlib.sha1(ident.encode()).hexdigest() + ".npy")
    PH = _lib.PH
    try:
        blob = torch.from_numpy(np.load(path, allow_pickle=False))
        h = blob[: _lib.PLAN_HEADER_INTS].tolist()
        ok = (
            blob.dtype == torch.int32 and blob.dim() == 1 and len(h) == _lib.PLAN_HEADER_INTS and h[PH["MAGIC"]] == _lib.PLAN_MAGIC and h[PH["TOTAL"]] == blob.numel()
            and (h[PH["NLAT_IN"]], h[PH["NLON_IN"]], h[PH["NLAT_OUT"]], h[PH["NLON_OUT"]]) == (nlat_in, nlon_in, nlat_out, nlon_out)
        )  # fmt: skip
        if ok:
            return Plan(blob.contiguous(), h)
    except (OSError, ValueError):
        pass
    plan = build_host_blob(col_idx, row_off, nlat_in, nlon_in, nlat_out, nlon_out)
    tmp = None
    try:
        os.makedirs(d, exist_ok=True)
        fd, tmp = tempfile.mkstemp(dir=d, suffix=".tmp")
        with os.fdopen(fd, "wb") as f:
            np.save(f, plan.blob.numpy(), allow_pickle=False)
        os.replace(tmp, path)  # atomic: a concurrent reader sees the old file or the whole new one
        tmp = None
    except OSError:
        pass
    finally:
        if tmp is not None:  # a write that failed half way leaves nothing behind
            try:
                os.unlink(tmp)
            except OSError:
                pass
    return plan


def build_host_plan(col_idx: torch.Tensor, row_off: torch.Tensor, nlat_in: int, nlon_in: int, nlat_out: int, nlon_out: int, with_mixed: bool = False):
    """
    The plan's basic arrays as CPU int32 tensors (views of the blob):
    ([gather_off, gather_runs, gather_order, scatter_off, scatter_runs, scatter_order], nruns, (gather_ndense, scatter_ndense));
    gather_runs has shape (nruns, 4) = (virtual input latitude, ws, len, real input latitude),
    grouped by virtual output latitude; scatter_runs (virtual output latitude, ws, len, real output latitude), grouped by
    virtual input latitude.  Virtual latitude = real latitude * ratio + column class on the finer of the two grids (see
    include/s2attn.h); the first *_ndense entries of each order are the latitudes with long runs.  with_mixed: a fourth
    element (gather_order_mixed, scatter_order_mixed), the same latitudes with long-run and short-run ones interleaved in
    proportion to their work.
    """
    plan = build_host_blob(col_idx, row_off, nlat_in, nlon_in, nlat_out, nlon_out)
    h, PH = plan.header, _lib.PH
    out = (plan.arrays(), plan.nruns, (h[PH["GATHER_NDENSE"]], h[PH["SCATTER_NDENSE"]]))
    return out + (plan.mixed_orders(),) if with_mixed else out


def _plan_key(col_idx, row_off, nlat_in, nlon_in, nlat_out, nlon_out):
    return (col_idx.data_ptr(), row_off.data_ptr(), col_idx.numel(), row_off.numel(), _version(col_idx), _version(row_off), str(col_idx.device),
            nlat_in, nlon_in, nlat_out, nlon_out)  # fmt: skip


def get_plan(col_idx: torch.Tensor, row_off: torch.Tensor, nlat_in: int, nlon_in: int, nlat_out: int, nlon_out: int) -> Plan:
    """Device plan for this psi, from the cache when the same tensors were seen before; else built from a host copy of the CSR
    (one device-to-host copy, the first time a psi is seen)."""
    key = _plan_key(col_idx, row_off, nlat_in, nlon_in, nlat_out, nlon_out)
    with _lock:
        plan = _cache.get(key)
        if plan is not None:
            _cache.move_to_end(key)
            return plan
    host = build_host_blob(col_idx, row_off, nlat_in, nlon_in, nlat_out, nlon_out)
    plan = Plan(host.blob.to(col_idx.device), host.header, (col_idx, row_off))
    with _lock:
        _cache[key] = plan
        while len(_cache) > _MAX_ENTRIES:
            _cache.popitem(last=False)
    return plan


def plan_from_blob(blob: torch.Tensor, header, nlat_in: int, nlon_in: int, nlat_out: int, nlon_out: int) -> Plan:
    """Plan around a blob that already lives on the right device (the module builds it in its constructor and keeps it as a
    buffer, so no forward ever copies the CSR back to the host).  Cached per blob storage."""
    key = ("blob", blob.data_ptr(), blob.numel(), _version(blob), str(blob.device))
    with _lock:
        plan = _cache.get(key)
        if plan is not None:
            _cache.move_to_end(key)
            return plan
    PH = _lib.PH
    header = tuple(int(x) for x in header)
    if len(header) != _lib.PLAN_HEADER_INTS or header[PH["MAGIC"]] != _lib.PLAN_MAGIC or header[PH["TOTAL"]] != blob.numel() or blob.dtype != torch.int32:
        raise RuntimeError("plan header does not describe this plan tensor")
    if (header[PH["NLAT_IN"]], header[PH["NLON_IN"]], header[PH["NLAT_OUT"]], header[PH["NLON_OUT"]]) != (nlat_in, nlon_in, nlat_out, nlon_out):
        raise RuntimeError("plan was built for other grid extents than this call's")
    plan = Plan(blob.contiguous(), header, blob)
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
