"""
ctypes binding of libs2attn.so (the C ABI in include/s2attn.h).

The library is built in-tree by torch_harmonics_amd/csrc/Makefile.  Loading never
falls back to anything: if the shared object is missing or a symbol is absent the
first use raises.
"""

import ctypes
import os
import subprocess
import threading

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libs2attn.so")
TORCH_LIB_PATH = os.path.join(_HERE, "_C.so")  # libtorch registration of the operators (csrc/s2attn_torch.cpp)

S2ATTN_F32, S2ATTN_BF16, S2ATTN_F16 = 0, 1, 2
ABI_VERSION = 12
NOALLOC_SCRATCH_BYTES = 64 * 1024 * 1024

_vp = ctypes.c_void_p
_i64 = ctypes.c_int64
_int = ctypes.c_int


PLAN_HEADER_INTS = 32
PLAN_MAGIC = 0x53324133
# index of each field in the plan header (include/s2attn.h, S2ATTN_PH_*)
PH = dict(
    MAGIC=0, TOTAL=1, NVOUT=2, NVIN=3, NRUNS=4, GATHER_NDENSE=5, SCATTER_NDENSE=6,
    GATHER_OFF=8, GATHER_RUNS=9, GATHER_ORDER=10, GATHER_ORDER_MIXED=11,
    SCATTER_OFF=12, SCATTER_RUNS=13, SCATTER_ORDER=14, SCATTER_ORDER_MIXED=15,
    GATHER_NITEMS=16, GATHER_ITEMS=17, GATHER_PAIR_OFF=18, GATHER_PAIR_RUNS=19, GATHER_NPAIRS=20,
    SCATTER_NITEMS=21, SCATTER_ITEMS=22, SCATTER_PAIR_OFF=23, SCATTER_PAIR_RUNS=24, SCATTER_NPAIRS=25, GATHER_SPAN=26,
    NLAT_IN=28, NLON_IN=29, NLAT_OUT=30, NLON_OUT=31,
)  # fmt: skip


class PlanStruct(ctypes.Structure):
    """s2attn_plan: device address of the plan blob and a host copy of its header."""

    _fields_ = [("data", _vp), ("header", ctypes.c_int32 * PLAN_HEADER_INTS)]

    @classmethod
    def make(cls, data_ptr, header):
        return cls(data_ptr, (ctypes.c_int32 * PLAN_HEADER_INTS)(*[int(x) for x in header]))


class ShapeStruct(ctypes.Structure):
    _fields_ = [
        ("batch", _int),
        ("num_heads", _int),
        ("nlat_in", _int),
        ("nlon_in", _int),
        ("nlat_out", _int),
        ("nlon_out", _int),
        ("ck", _int),
        ("cv", _int),
        ("dtype", _int),
        # point strides in elements, 0 = packed (see include/s2attn.h)
        ("ld_k", _int), ("ld_v", _int), ("ld_q", _int), ("ld_y", _int), ("ld_dy", _int), ("ld_dk", _int), ("ld_dv", _int), ("ld_dq", _int),
    ]  # fmt: skip


class RingShapeStruct(ctypes.Structure):
    _fields_ = [
        ("batch", ctypes.c_int32),
        ("nlat_halo", ctypes.c_int32),
        ("nlon_kx", ctypes.c_int32),
        ("nlat_out", ctypes.c_int32),
        ("nlon_out", ctypes.c_int32),
        ("ck", ctypes.c_int32),
        ("cv", ctypes.c_int32),
        ("nlon_in", ctypes.c_int32),
        ("pscale", ctypes.c_int32),
        ("lon_lo_kx", ctypes.c_int32),
        ("lat_halo_start", ctypes.c_int32),
        ("dtype", ctypes.c_int32),
    ]


class RingUpShapeStruct(ctypes.Structure):
    _fields_ = [
        (n, ctypes.c_int32)
        for n in ("batch", "nlat_halo", "nlon_kx", "nlat_out", "nlon_out", "ck", "cv", "nlon_out_global", "pscale_out", "lon_lo_kx", "lat_halo_start", "dtype")
    ]


# every symbol include/s2attn.h declares: name -> (restype, argtypes)
SYMBOLS = {
    "s2attn_last_error": (ctypes.c_char_p, []),
    "s2attn_abi_version": (_int, []),
    "s2attn_plan_count": (_i64, [_vp, _vp, _i64, _int, _int, _int, _int]),
    "s2attn_plan_size": (_i64, [_vp, _vp, _i64, _int, _int, _int, _int]),
    "s2attn_plan_build": (_int, [_vp, _vp, _i64, _int, _int, _int, _int, _vp, _i64]),
    "s2attn_forward": (_int, [_vp, _vp, _vp, _vp, _vp, ctypes.POINTER(PlanStruct), ctypes.POINTER(ShapeStruct), _vp]),
    "s2attn_forward_lse": (_int, [_vp, _vp, _vp, _vp, _vp, _vp, ctypes.POINTER(PlanStruct), ctypes.POINTER(ShapeStruct), _vp]),
    "s2attn_backward_saved": (_int, [_vp] * 11 + [ctypes.POINTER(PlanStruct), ctypes.POINTER(ShapeStruct), _vp]),
    "s2attn_backward_saved_noalloc": (_int, [_vp] * 10 + [ctypes.POINTER(PlanStruct), ctypes.POINTER(ShapeStruct), _vp]),
    "s2attn_backward_dq_saved": (_int, [_vp] * 9 + [ctypes.POINTER(PlanStruct), ctypes.POINTER(ShapeStruct), _vp]),
    "s2attn_backward_workspace_bytes": (_i64, [ctypes.POINTER(ShapeStruct)]),
    "s2attn_backward_saved_workspace_bytes": (_i64, [ctypes.POINTER(ShapeStruct)]),
    "s2attn_backward": (_int, [_vp] * 9 + [ctypes.POINTER(PlanStruct), ctypes.POINTER(ShapeStruct), _vp]),
    "s2attn_backward_dq": (_int, [_vp] * 7 + [ctypes.POINTER(PlanStruct), ctypes.POINTER(ShapeStruct), _vp]),
    "s2attn_backward_dkdv": (_int, [_vp] * 8 + [ctypes.POINTER(PlanStruct), ctypes.POINTER(ShapeStruct), _vp]),
    "s2attn_permute_to_nhwc": (_int, [_vp, _vp, _i64, _i64, _i64, _i64, _int, _vp]),
    "s2attn_permute_to_nchw": (_int, [_vp, _vp, _i64, _i64, _i64, _i64, _int, _vp]),
    "s2attn_ring_forward_step": (_int, [_vp] * 10 + [ctypes.POINTER(RingShapeStruct), _vp]),
    "s2attn_ring_forward_step_plan": (_int, [_vp] * 7 + [ctypes.POINTER(PlanStruct), ctypes.POINTER(RingShapeStruct), _vp]),
    "s2attn_ring_backward_pass1_plan": (_int, [_vp] * 10 + [ctypes.POINTER(PlanStruct), ctypes.POINTER(RingShapeStruct), _vp]),
    "s2attn_ring_backward_pass2_plan": (_int, [_vp] * 10 + [ctypes.POINTER(PlanStruct), ctypes.POINTER(RingShapeStruct), _vp]),
    "s2attn_ring_forward_step_upsample_plan": (_int, [_vp] * 7 + [ctypes.POINTER(PlanStruct), ctypes.POINTER(RingUpShapeStruct), _vp]),
    "s2attn_ring_backward_pass1_upsample_plan": (_int, [_vp] * 9 + [ctypes.POINTER(PlanStruct), ctypes.POINTER(RingUpShapeStruct), _vp]),
    "s2attn_ring_backward_pass2_upsample_plan": (_int, [_vp] * 10 + [ctypes.POINTER(PlanStruct), ctypes.POINTER(RingUpShapeStruct), _vp]),
    "s2attn_ring_backward_pass1": (_int, [_vp] * 13 + [ctypes.POINTER(RingShapeStruct), _vp]),
    "s2attn_ring_backward_pass2": (_int, [_vp] * 13 + [ctypes.POINTER(RingShapeStruct), _vp]),
    "s2attn_ring_regroup_psi": (_i64, [_vp, _vp, _int, _int, _int, _int, _vp, _vp, _vp, _vp]),
    "s2attn_ring_backward_pass2_transposed": (_int, [_vp] * 14 + [ctypes.POINTER(RingShapeStruct), _vp]),
    "s2attn_ring_forward_step_upsample": (_int, [_vp] * 10 + [ctypes.POINTER(RingUpShapeStruct), _vp]),
    "s2attn_ring_backward_pass1_upsample": (_int, [_vp] * 12 + [ctypes.POINTER(RingUpShapeStruct), _vp]),
    "s2attn_ring_backward_pass2_upsample": (_int, [_vp] * 13 + [ctypes.POINTER(RingUpShapeStruct), _vp]),
}

_lib = None
_lock = threading.Lock()


def build(verbose: bool = False) -> str:
    """Compile libs2attn.so for gfx950 with hipcc (always recompiles)."""
    csrc = os.path.join(_HERE, "csrc")
    subprocess.run(["make", "-C", csrc, "clean"], check=True, capture_output=not verbose)
    proc = subprocess.run(["make", "-C", csrc, "-j4"], capture_output=True, text=True)
    if proc.returncode != 0:
        raise RuntimeError(f"building libs2attn.so failed:\n{proc.stdout}\n{proc.stderr}")
    if verbose:
        print(proc.stdout)
    return LIB_PATH


def is_built() -> bool:
    return os.path.exists(LIB_PATH) and os.path.exists(TORCH_LIB_PATH)


def load():
    """Returns the loaded library with typed entry points; raises if it is not built."""
    global _lib
    if _lib is not None:
        return _lib
    with _lock:
        if _lib is not None:
            return _lib
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(
                f"{LIB_PATH} is not built. Run `make -C {os.path.join(_HERE, 'csrc')}` (needs hipcc); " "this package has no fallback implementation."
            )
        lib = ctypes.CDLL(LIB_PATH)
        for name, (restype, argtypes) in SYMBOLS.items():
            fn = getattr(lib, name)  # AttributeError if the export is missing
            fn.restype = restype
            fn.argtypes = argtypes
        got = lib.s2attn_abi_version()
        if got != ABI_VERSION:
            raise RuntimeError(f"libs2attn.so has ABI version {got}, this package expects {ABI_VERSION}; rebuild it")
        _lib = lib
    return _lib


_torch_ops_loaded = False


def load_torch_ops() -> None:
    """Loads _C.so, whose static initialisers register attention_kernels::{forward, backward, permute_to_nhwc, permute_to_nchw}
    and s2attn_kernels::{forward_lse, backward_saved} with the dispatcher; raises if it is not built."""
    global _torch_ops_loaded
    if _torch_ops_loaded:
        return
    load()  # the C ABI library it links against
    with _lock:
        if _torch_ops_loaded:
            return
        if not os.path.exists(TORCH_LIB_PATH):
            raise RuntimeError(f"{TORCH_LIB_PATH} is not built. Run `make -C {os.path.join(_HERE, 'csrc')}`; this package has no fallback implementation.")
        import torch

        torch.ops.load_library(TORCH_LIB_PATH)
        _torch_ops_loaded = True


def check(rc: int, what: str) -> None:
    """Turns a negative return code into a RuntimeError carrying the library's message."""
    if rc < 0:
        msg = load().s2attn_last_error()
        raise RuntimeError(f"{what}: {msg.decode() if msg else f'error {rc}'}")
