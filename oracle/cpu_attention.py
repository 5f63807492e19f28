"""
ctypes front end of the C oracle (oracle/s2attn_oracle.c) plus a dense float64
formulation used to pin it.

TEST INFRASTRUCTURE ONLY: the shipped package must never import this module.

All functions take CPU torch tensors in the op's layout (NHWC, heads packed):
  k [B,Hi,Wi,nh*Ck], v [B,Hi,Wi,nh*Cv], q [B,Ho,Wo,nh*Ck], dy [B,Ho,Wo,nh*Cv],
  quad_weights [Hi] fp32, col_idx [nnz] int64, row_off [Ho+1] int64.
"""

import ctypes
import os
import subprocess

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIBS = {}

_P = ctypes.c_void_p
_I = ctypes.c_int64


def build(force: bool = False) -> None:
    """Compile both oracle libraries with the Makefile next to this file."""
    if force:
        subprocess.run(["make", "-C", _HERE, "clean"], check=True, capture_output=True)
    subprocess.run(["make", "-C", _HERE], check=True, capture_output=True)


def _lib(fast: bool = False):
    name = "liboracle_s2attn_fast.so" if fast else "liboracle_s2attn.so"
    if name not in _LIBS:
        path = os.path.join(_HERE, name)
        if not os.path.exists(path):
            build()
        lib = ctypes.CDLL(path)
        lib.s2o_fwd_f32.argtypes = [_P] * 7 + [_I] * 8
        lib.s2o_fwd_f32.restype = None
        lib.s2o_bwd_f32.argtypes = [_P] * 10 + [_I] * 8
        lib.s2o_bwd_f32.restype = ctypes.c_int
        lib.s2o_fwd_f64.argtypes = [_P] * 7 + [_I] * 10
        lib.s2o_fwd_f64.restype = None
        lib.s2o_bwd_f64.argtypes = [_P] * 10 + [_I] * 10
        lib.s2o_bwd_f64.restype = None
        _LIBS[name] = lib
    return _LIBS[name]


def _f32(t):
    return t.detach().to(device="cpu", dtype=torch.float32).contiguous()


def _i64(t):
    return t.detach().to(device="cpu", dtype=torch.int64).contiguous()


def _dims(k, v, q, nh):
    B, Hi, Wi, CK = k.shape
    _, Ho, Wo, _ = q.shape
    CV = v.shape[3]
    assert CK % nh == 0 and CV % nh == 0 and (Wi % Wo == 0 or Wo % Wi == 0)
    return B, Hi, Wi, Ho, Wo, CK // nh, CV // nh


def forward_f32(k, v, q, quad_weights, col_idx, row_off, nh, fast=False):
    """fp32 restatement of the reference CPU forward (attention_cpu_fwd.h:63-204)."""
    k, v, q, w = _f32(k), _f32(v), _f32(q), _f32(quad_weights)
    ci, ro = _i64(col_idx), _i64(row_off)
    B, Hi, Wi, Ho, Wo, Ck, Cv = _dims(k, v, q, nh)
    y = torch.zeros((B, Ho, Wo, nh * Cv), dtype=torch.float32)
    _lib(fast).s2o_fwd_f32(k.data_ptr(), v.data_ptr(), q.data_ptr(), w.data_ptr(), ci.data_ptr(), ro.data_ptr(), y.data_ptr(), B, nh, Hi, Wi, Ho, Wo, Ck, Cv)
    return y


def backward_f32(k, v, q, dy, quad_weights, col_idx, row_off, nh, fast=False):
    """fp32 restatement of the reference CPU backward (attention_cpu_bwd.h:75-347): returns (dk, dv, dq)."""
    k, v, q, dy, w = _f32(k), _f32(v), _f32(q), _f32(dy), _f32(quad_weights)
    ci, ro = _i64(col_idx), _i64(row_off)
    B, Hi, Wi, Ho, Wo, Ck, Cv = _dims(k, v, q, nh)
    dk, dv, dq = torch.zeros_like(k), torch.zeros_like(v), torch.zeros_like(q)
    rc = _lib(fast).s2o_bwd_f32(
        k.data_ptr(), v.data_ptr(), q.data_ptr(), dy.data_ptr(), w.data_ptr(), ci.data_ptr(), ro.data_ptr(), dk.data_ptr(), dv.data_ptr(), dq.data_ptr(), B, nh, Hi, Wi, Ho, Wo, Ck, Cv
    )
    if rc != 0:
        raise MemoryError("the reference CPU backward needs 2*B*nh*Ho*Wo*max_row_len floats of scratch, which could not be allocated")
    return dk, dv, dq


def forward_f64(k, v, q, quad_weights, col_idx, row_off, nh, ho_range=None):
    """float64 spec forward (attention_torch.py:74-125); rows outside ho_range stay zero."""
    k, v, q, w = _f32(k), _f32(v), _f32(q), _f32(quad_weights)
    ci, ro = _i64(col_idx), _i64(row_off)
    B, Hi, Wi, Ho, Wo, Ck, Cv = _dims(k, v, q, nh)
    lo, hi = (0, Ho) if ho_range is None else ho_range
    y = torch.zeros((B, Ho, Wo, nh * Cv), dtype=torch.float64)
    _lib().s2o_fwd_f64(k.data_ptr(), v.data_ptr(), q.data_ptr(), w.data_ptr(), ci.data_ptr(), ro.data_ptr(), y.data_ptr(), B, nh, Hi, Wi, Ho, Wo, Ck, Cv, lo, hi)
    return y


def backward_f64(k, v, q, dy, quad_weights, col_idx, row_off, nh, ho_range=None):
    """float64 spec backward (attention_torch.py:130-390): (dk, dv, dq) from the queries on rows ho_range."""
    k, v, q, dy, w = _f32(k), _f32(v), _f32(q), _f32(dy), _f32(quad_weights)
    ci, ro = _i64(col_idx), _i64(row_off)
    B, Hi, Wi, Ho, Wo, Ck, Cv = _dims(k, v, q, nh)
    lo, hi = (0, Ho) if ho_range is None else ho_range
    dk = torch.zeros(k.shape, dtype=torch.float64)
    dv = torch.zeros(v.shape, dtype=torch.float64)
    dq = torch.zeros(q.shape, dtype=torch.float64)
    _lib().s2o_bwd_f64(
        k.data_ptr(), v.data_ptr(), q.data_ptr(), dy.data_ptr(), w.data_ptr(), ci.data_ptr(), ro.data_ptr(), dk.data_ptr(), dv.data_ptr(), dq.data_ptr(), B, nh, Hi, Wi, Ho, Wo, Ck, Cv, lo, hi
    )
    return dk, dv, dq


def dense_mask(col_idx, row_off, Hi, Wi, Ho, Wo):
    """Boolean [Ho*Wo, Hi*Wi] mask: psi row ho shifted by pscale*wo in longitude (attention_torch.py:97-104)."""
    pscale = Wi // Wo
    M = torch.zeros((Ho, Wo, Hi, Wi), dtype=torch.bool)
    ci, ro = _i64(col_idx), _i64(row_off)
    for ho in range(Ho):
        cols = ci[ro[ho] : ro[ho + 1]]
        hi = cols // Wi
        wi = cols % Wi
        for wo in range(Wo):
            M[ho, wo, hi, (wi + pscale * wo) % Wi] = True
    return M.reshape(Ho * Wo, Hi * Wi)


def dense_mask_upsample(col_idx, row_off, Hi, Wi, Ho, Wo):
    """Boolean [Ho*Wo, Hi*Wi] mask of the up-sampling (scatter) direction: psi row hi lists output points (ho, wo) seen from
    input column 0; input column wi sees them shifted by (Wo / Wi) * wi in longitude (attention_torch.py:613-621)."""
    ps = Wo // Wi
    M = torch.zeros((Ho, Wo, Hi, Wi), dtype=torch.bool)
    ci, ro = _i64(col_idx), _i64(row_off)
    for hi in range(Hi):
        cols = ci[ro[hi] : ro[hi + 1]]
        ho = cols // Wo
        wo = cols % Wo
        for wi in range(Wi):
            M[ho, (wo + ps * wi) % Wo, hi, wi] = True
    return M.reshape(Ho * Wo, Hi * Wi)


def is_upsample(Wi, Wo):
    """Direction rule of the reference (attention.py:337): scatter iff nlon_out is a proper multiple of nlon_in."""
    return Wo % Wi == 0 and Wi % Wo != 0


def dense_attention_f64(k, v, q, quad_weights, col_idx, row_off, nh, dtype=torch.float64):
    """
    Textbook formulation, differentiable: softmax over the masked neighborhood of
    q.k + log(quad weight), times v, in float64.  Small grids only (dense mask).  Serves both
    directions: the mask is the only thing that differs (attention_torch.py:74-125 and 582-650).
    dtype=torch.float32 evaluates the same expression in single precision (what plain fp32 arithmetic
    makes of the inputs: the yardstick for shapes where 1e-5 is below fp32's own reach).
    """
    B, Hi, Wi, Ho, Wo, Ck, Cv = _dims(k, v, q, nh)
    M = (dense_mask_upsample if is_upsample(Wi, Wo) else dense_mask)(col_idx, row_off, Hi, Wi, Ho, Wo)
    kd = k.to(dtype).reshape(B, Hi * Wi, nh, Ck).permute(0, 2, 1, 3)
    vd = v.to(dtype).reshape(B, Hi * Wi, nh, Cv).permute(0, 2, 1, 3)
    qd = q.to(dtype).reshape(B, Ho * Wo, nh, Ck).permute(0, 2, 1, 3)
    logw = torch.log(quad_weights.to(torch.float64)).to(dtype).reshape(Hi, 1).expand(Hi, Wi).reshape(1, 1, 1, Hi * Wi)
    scores = qd @ kd.transpose(-1, -2) + logw
    scores = scores.masked_fill(~M.reshape(1, 1, Ho * Wo, Hi * Wi), float("-inf"))
    y = torch.softmax(scores, dim=-1) @ vd
    return y.permute(0, 2, 1, 3).reshape(B, Ho, Wo, nh * Cv)
