"""
torch.library operators over the C ABI of libs2attn.so.

Operator set and signatures follow the reference:
  attention_kernels::forward / backward         the reference's own operator names and schemas (attention_interface.cpp:
  attention_kernels::permute_to_nhwc / _nchw    85-119), registered for the CUDA dispatch key by the C++ binding
                                                csrc/s2attn_torch.cpp; fake and autograd rules here, as in
                                                attention_optimized.py:230-322 and attention/_layout.py:76-103
  attention_kernels::_neighborhood_s2_attention_optimized
                                                the autograd-carrying op, a Python fragment of the namespace the C++
                                                binding defines, as in the reference (attention_optimized.py:230-322)
  attention_kernels::forward_ring_step ...      the six ring-step operators and split_csr_rows under the reference's names
                                                and argument lists (attention_interface.cpp:136-189)
  s2attn::_neighborhood_s2_attention_saved      the same attention with y and the normaliser handed to the backward
Argument order is (k, v, q, ...), outputs of backward are (dk, dv, dq), as there.

Both directions are served: nlon_in a multiple of nlon_out (self-attention, down-sampling; psi keyed by output latitude) and
nlon_out a multiple of nlon_in (up-sampling; psi keyed by input latitude, attention_torch.py:582-592), told apart by the two
longitude counts as in the reference.  Tensors must live on a ROCm device: there is no CPU implementation behind these operators.
"""

import ctypes
from typing import List, Optional, Tuple

import torch

from . import _lib
from ._attention_utils import _setup_context_attention_backward
from . import plan as _plan
from .plan import get_row_order, get_transposed_csr

_DTYPE_CODE = {torch.float32: _lib.S2ATTN_F32, torch.bfloat16: _lib.S2ATTN_BF16, torch.float16: _lib.S2ATTN_F16}


def _stream_ptr(device: torch.device) -> ctypes.c_void_p:
    return ctypes.c_void_p(torch.cuda.current_stream(device).cuda_stream)


def _require_gpu(t: torch.Tensor, name: str, device: torch.device = None) -> None:
    if t.device.type != "cuda":
        raise RuntimeError(f"{name} is on {t.device}; the s2attn operators only run on a ROCm GPU (no CPU implementation is shipped)")
    if device is not None and t.device != device:
        raise RuntimeError(f"{name} is on {t.device} but the other operands are on {device}")


# ---- raw operators: registered by the C++ binding (csrc/s2attn_torch.cpp) under the reference's names -------------------------
#   attention_kernels::forward / backward / permute_to_nhwc / permute_to_nchw      (attention_interface.cpp:85-119)
#   s2attn_kernels::forward_lse / backward_saved   the same pair with y and the softmax normaliser handed to the backward
# Argument checks, output allocation, the plan cache and the launch live there; what Python adds, as in the reference
# (attention_optimized.py:230-322, _layout.py:76-103), are the fake kernels and the autograd rules.
_lib.load_torch_ops()

forward = torch.ops.attention_kernels.forward
backward = torch.ops.attention_kernels.backward
permute_to_nhwc = torch.ops.attention_kernels.permute_to_nhwc
permute_to_nchw = torch.ops.attention_kernels.permute_to_nchw
forward_lse = torch.ops.s2attn_kernels.forward_lse
backward_saved = torch.ops.s2attn_kernels.backward_saved


@torch.library.register_fake("attention_kernels::forward")
def _(kx, vx, qy, quad_weights, col_idx, row_off, num_heads, nlon_in, nlat_out, nlon_out):
    return torch.empty((kx.shape[0], nlat_out, nlon_out, vx.shape[3]), dtype=kx.dtype, device=kx.device)


@torch.library.register_fake("s2attn_kernels::forward_lse")
def _(kx, vx, qy, quad_weights, col_idx, row_off, num_heads, nlon_in, nlat_out, nlon_out, plan=None, plan_header=None):
    y = torch.empty((kx.shape[0], nlat_out, nlon_out, vx.shape[3]), dtype=kx.dtype, device=kx.device)
    return y, torch.empty((kx.shape[0], num_heads, nlat_out, nlon_out), dtype=torch.float32, device=kx.device)


def _point_stride(t: torch.Tensor) -> int:
    """Elements between two grid points when t is a column block of a wider buffer, 0 when it is packed (the binding's point_stride)."""
    return 0 if t.is_contiguous() else t.stride(2)


def _same_buffer(a: torch.Tensor, b: torch.Tensor) -> bool:
    return a.untyped_storage().data_ptr() == b.untyped_storage().data_ptr() if not isinstance(a, torch._subclasses.FakeTensor) else torch._C._is_alias_of(a, b)


def _fake_gradients(kx, vx, qy):
    """Metadata of (dk, dv, dq) as the binding's backward returns them (csrc/s2attn_torch.cpp, backward_impl): packed tensors, except
    that k | v (| q) given as DISJOINT column blocks of one buffer get their gradients as the same column blocks of one new
    buffer."""
    ldk, ldv, ldq = _point_stride(kx), _point_stride(vx), _point_stride(qy)

    def cols(t, ld):
        first = t.storage_offset() % ld
        return first, first + t.shape[3]

    def disjoint(a, b):
        return a[1] <= b[0] or b[1] <= a[0]

    kv_fused = ldk > 0 and ldk == ldv and _same_buffer(kx, vx) and kx.storage_offset() // ldk == vx.storage_offset() // ldk
    if kv_fused:
        ck_, cv_ = cols(kx, ldk), cols(vx, ldk)
        kv_fused = ck_[1] <= ldk and cv_[1] <= ldk and disjoint(ck_, cv_)
    if not kv_fused:
        return kx.new_empty(kx.shape), vx.new_empty(vx.shape), qy.new_empty(qy.shape)
    all_fused = ldq == ldk and _same_buffer(qy, kx) and tuple(qy.shape[:3]) == tuple(kx.shape[:3]) and qy.storage_offset() // ldk == kx.storage_offset() // ldk
    if all_fused:
        cq_ = cols(qy, ldk)
        all_fused = cq_[1] <= ldk and disjoint(cq_, ck_) and disjoint(cq_, cv_)
    buf = kx.new_empty((kx.shape[0], kx.shape[1], kx.shape[2], ldk))
    dk = buf.narrow(3, ck_[0], kx.shape[3])
    dv = buf.narrow(3, cv_[0], vx.shape[3])
    dq = buf.narrow(3, cq_[0], qy.shape[3]) if all_fused else qy.new_empty(qy.shape)
    return dk, dv, dq


@torch.library.register_fake("attention_kernels::backward")
def _(kx, vx, qy, dy, quad_weights, col_idx, row_off, num_heads, nlon_in, nlat_out, nlon_out):
    return _fake_gradients(kx, vx, qy)


@torch.library.register_fake("s2attn_kernels::backward_saved")
def _(kx, vx, qy, dy, y, lse, quad_weights, col_idx, row_off, num_heads, nlon_in, nlat_out, nlon_out, plan=None, plan_header=None):
    return _fake_gradients(kx, vx, qy)


# ---- layout ops ------------------------------------------------------------------------


@torch.library.register_fake("attention_kernels::permute_to_nhwc")
def _(x):
    B, C, H, W = x.shape
    return x.new_empty((B, H, W, C))


@torch.library.register_fake("attention_kernels::permute_to_nchw")
def _(x):
    B, H, W, C = x.shape
    return x.new_empty((B, C, H, W))


def _no_context(ctx, inputs, output):
    pass


# the two conversions are inverses of each other, so each one's gradient is the other one
torch.library.register_autograd("attention_kernels::permute_to_nhwc", lambda ctx, g: permute_to_nchw(g.contiguous()), setup_context=_no_context)
torch.library.register_autograd("attention_kernels::permute_to_nchw", lambda ctx, g: permute_to_nhwc(g.contiguous()), setup_context=_no_context)


# ---- the autograd-carrying attention op ---------------------------------------------------


@torch.library.custom_op("attention_kernels::_neighborhood_s2_attention_optimized", mutates_args=())
def _neighborhood_s2_attention_optimized(
    kw: torch.Tensor,
    vw: torch.Tensor,
    qw: torch.Tensor,
    quad_weights: torch.Tensor,
    col_idx: torch.Tensor,
    row_off: torch.Tensor,
    nh: int,
    nlon_in: int,
    nlat_out: int,
    nlon_out: int,
) -> torch.Tensor:
    return forward(kw.contiguous(), vw.contiguous(), qw.contiguous(), quad_weights, col_idx, row_off, nh, nlon_in, nlat_out, nlon_out)


@_neighborhood_s2_attention_optimized.register_fake
def _(kw, vw, qw, quad_weights, col_idx, row_off, nh, nlon_in, nlat_out, nlon_out):
    return torch.empty((kw.shape[0], nlat_out, nlon_out, vw.shape[3]), dtype=kw.dtype, device=kw.device)


def _neighborhood_s2_attention_bwd_optimized(ctx, grad_output):
    col_idx, row_off, quad_weights, kw, vw, qw = ctx.saved_tensors
    dkw, dvw, dqw = backward(
        kw.contiguous(), vw.contiguous(), qw.contiguous(), grad_output.contiguous(), quad_weights, col_idx, row_off, ctx.nh, ctx.nlon_in, ctx.nlat_out, ctx.nlon_out
    )
    return dkw, dvw, dqw, None, None, None, None, None, None, None


_neighborhood_s2_attention_optimized.register_autograd(_neighborhood_s2_attention_bwd_optimized, setup_context=_setup_context_attention_backward)


def takes_column_blocks(dtype: torch.dtype, ck: int, cv: int, nlon_in: int, nlon_out: int) -> bool:
    """True for the shapes whose kernels read q, k, v in place out of a wider buffer and write dq, dk, dv into one
    (fp32 heads of 32 channels on at least 64 longitudes per virtual latitude: the hybrid kernels)."""
    return dtype == torch.float32 and ck == 32 and cv == 32 and min(nlon_in, nlon_out) >= 64


def _is_column_block(t: torch.Tensor) -> bool:
    """t is a column block of a contiguous (B, nlat, nlon, width) buffer: unit channel stride, one point stride of at least
    its own width (an expanded tensor has stride 0), both offset and stride multiples of four elements."""
    if t.dim() != 4 or t.stride(3) != 1:
        return False
    ld = t.stride(2)
    return ld >= t.shape[3] and ld % 4 == 0 and t.stride(1) == t.shape[2] * ld and t.stride(0) == t.shape[1] * t.stride(1) and t.storage_offset() % 4 == 0


def _packed_or_block(t: torch.Tensor, blocks_ok: bool) -> torch.Tensor:
    """t itself when it is contiguous, or when it is a column block of a wider buffer (a slice of a fused q | k | v
    projection) AND the shape is one whose kernels read such blocks in place (blocks_ok, see takes_column_blocks); a
    contiguous copy otherwise."""
    if t.is_contiguous():
        return t
    if blocks_ok and _is_column_block(t):
        return t
    return t.contiguous()


def _blocks_ok(kw: torch.Tensor, vw: torch.Tensor, nh: int, nlon_in: int, nlon_out: int) -> bool:
    return nh > 0 and takes_column_blocks(kw.dtype, kw.shape[3] // nh, vw.shape[3] // nh, nlon_in, nlon_out)


# Same op, but the forward also hands its output and softmax normaliser to the backward (the reference recomputes both,
# attention_cuda_bwd.cu:856-956).  Two outputs, so it cannot carry the reference's one-tensor signature; the module
# calls it through neighborhood_s2_attention below.
@torch.library.custom_op("s2attn::_neighborhood_s2_attention_saved", mutates_args=())
def _neighborhood_s2_attention_saved(
    kw: torch.Tensor,
    vw: torch.Tensor,
    qw: torch.Tensor,
    quad_weights: torch.Tensor,
    col_idx: torch.Tensor,
    row_off: torch.Tensor,
    nh: int,
    nlon_in: int,
    nlat_out: int,
    nlon_out: int,
    plan: Optional[torch.Tensor] = None,
    plan_header: Optional[List[int]] = None,
) -> Tuple[torch.Tensor, torch.Tensor]:
    ok = _blocks_ok(kw, vw, nh, nlon_in, nlon_out)
    return forward_lse(_packed_or_block(kw, ok), _packed_or_block(vw, ok), _packed_or_block(qw, ok), quad_weights, col_idx, row_off, nh, nlon_in, nlat_out, nlon_out, plan, plan_header)


@_neighborhood_s2_attention_saved.register_fake
def _(kw, vw, qw, quad_weights, col_idx, row_off, nh, nlon_in, nlat_out, nlon_out, plan=None, plan_header=None):
    y = torch.empty((kw.shape[0], nlat_out, nlon_out, vw.shape[3]), dtype=kw.dtype, device=kw.device)
    return y, torch.empty((kw.shape[0], nh, nlat_out, nlon_out), dtype=torch.float32, device=kw.device)


def _setup_context_saved(ctx, inputs, output):
    _setup_context_attention_backward(ctx, inputs[:10], output)
    ctx.y, ctx.lse = output[0].detach(), output[1].detach()
    ctx.plan, ctx.plan_header = inputs[10], inputs[11]
    ctx.mark_non_differentiable(output[1])


def _neighborhood_s2_attention_bwd_saved(ctx, grad_output, grad_lse):
    col_idx, row_off, quad_weights, kw, vw, qw = ctx.saved_tensors
    ok = _blocks_ok(kw, vw, ctx.nh, ctx.nlon_in, ctx.nlon_out)
    dkw, dvw, dqw = backward_saved(
        _packed_or_block(kw, ok), _packed_or_block(vw, ok), _packed_or_block(qw, ok), grad_output.contiguous(), ctx.y, ctx.lse, quad_weights, col_idx, row_off, ctx.nh, ctx.nlon_in,
        ctx.nlat_out, ctx.nlon_out, ctx.plan, ctx.plan_header,
    )  # fmt: skip
    return dkw, dvw, dqw, None, None, None, None, None, None, None, None, None


_neighborhood_s2_attention_saved.register_autograd(_neighborhood_s2_attention_bwd_saved, setup_context=_setup_context_saved)


def neighborhood_s2_attention(kw, vw, qw, quad_weights, col_idx, row_off, nh, nlon_in, nlat_out, nlon_out, plan=None, plan_header=None):
    """Differentiable attention on NHWC heads-packed tensors; what NeighborhoodAttentionS2.forward calls.  plan, plan_header:
    the psi's plan built ahead of time (the module builds it in its constructor), so that no call copies psi to the host."""
    return _neighborhood_s2_attention_saved(kw, vw, qw, quad_weights, col_idx, row_off, nh, nlon_in, nlat_out, nlon_out, plan, plan_header)[0]


# Autocast: k, v, q are brought to the active autocast dtype and the op re-entered with autocast off;
# quad_weights and the index tensors pass through (attention_optimized.py:310-322).
def _make_autocast_impl(device_type: str):
    @torch.library.impl("attention_kernels::_neighborhood_s2_attention_optimized", f"Autocast{device_type.upper()}")
    def _(kw, vw, qw, quad_weights, col_idx, row_off, nh, nlon_in, nlat_out, nlon_out):
        cast_dtype = torch.get_autocast_dtype(device_type)
        with torch.amp.autocast(device_type, enabled=False):
            return _neighborhood_s2_attention_optimized(kw.to(cast_dtype), vw.to(cast_dtype), qw.to(cast_dtype), quad_weights, col_idx, row_off, nh, nlon_in, nlat_out, nlon_out)

    return _


def _make_autocast_impl_saved(device_type: str):
    @torch.library.impl("s2attn::_neighborhood_s2_attention_saved", f"Autocast{device_type.upper()}")
    def _(kw, vw, qw, quad_weights, col_idx, row_off, nh, nlon_in, nlat_out, nlon_out, plan=None, plan_header=None):
        cast_dtype = torch.get_autocast_dtype(device_type)
        with torch.amp.autocast(device_type, enabled=False):
            return _neighborhood_s2_attention_saved(
                kw.to(cast_dtype), vw.to(cast_dtype), qw.to(cast_dtype), quad_weights, col_idx, row_off, nh, nlon_in, nlat_out, nlon_out, plan, plan_header
            )

    return _


for _device_type in ("cuda", "cpu"):
    _make_autocast_impl(_device_type)
    _make_autocast_impl_saved(_device_type)


# ---------------------------------------------------------------------------------------------------------------------
# Ring-step operators of the gather direction (attention_interface.cpp:137-156, fake kernels attention_optimized.py:82-160):
# one longitude chunk of K/V per call, the softmax state lives in caller-owned fp32 buffers that the operators update in
# place.  Same argument lists as the reference's; the three trailing row-split hints are accepted and not needed.
# ---------------------------------------------------------------------------------------------------------------------
def split_csr_rows(row_idx: torch.Tensor, row_off: torch.Tensor, nlat_out: int):
    """(n_long_rows, max_row_len, mid_row_len) of a CSR whose rows are listed in row_idx by decreasing length: the long rows
    are the leading ones of at least max(1024, 0.1 * longest) entries; max_row_len is the longest row if there is a long
    one, else 0; mid_row_len the length of the first short row, else 0 (attention_cuda_utils.cu:286-384).  Host scalar
    computation on either device's tensors; never traced."""
    idx = row_idx.detach().to("cpu", torch.int64)
    off = row_off.detach().to("cpu", torch.int64)
    if nlat_out == 0:
        return 0, 0, 0
    lens = (off[1:] - off[:-1])[idx[:nlat_out]]
    max_rlen = int(lens[0])
    min_long = max(1024, int(float(torch.tensor(max_rlen, dtype=torch.float32) * torch.tensor(0.1, dtype=torch.float32))))
    short = (lens < min_long).nonzero()
    n_long = int(short[0]) if short.numel() else int(nlat_out)
    return n_long, (max_rlen if n_long else 0), (int(lens[n_long]) if n_long < nlat_out else 0)


# the reference's operator of the same name and schema (attention_interface.cpp:136): a set-up-time host computation, not
# pt2-compliant and without a fake kernel there either
_ring_fragment = torch.library.Library("attention_kernels", "FRAGMENT")
_ring_fragment.define("split_csr_rows(Tensor row_idx, Tensor row_off, int nlat_out) -> (int, int, int)")
_ring_fragment.impl("split_csr_rows", split_csr_rows, "CompositeExplicitAutograd")


def _ring_shape(kx, vx, qy, nlon_in, pscale, lon_lo_kx, lat_halo_start, nlat_out, nlon_out) -> _lib.RingShapeStruct:
    B, nlat_halo, nlon_kx, ck = kx.shape
    return _lib.RingShapeStruct(B, nlat_halo, nlon_kx, nlat_out, nlon_out, ck, vx.shape[3], nlon_in, pscale, lon_lo_kx, lat_halo_start, _DTYPE_CODE[qy.dtype])


def _ring_takes_plan(kx, vx, qy, nlon_in, pscale, max_ck=128) -> bool:
    """Shapes of the band-staged ring steps (s2attn_ring_forward_step_plan, s2attn_ring_backward_pass1_plan / pass2_plan in include/s2attn.h).
    Decided by the shape alone, so that the forward step and pass 1 of one problem always run the same formulation (their
    alpha_sum are then bit-identical; the state buffers are fresh torch allocations, 16-byte aligned like every tensor).
    The up-sampling direction stops at 64 channels (max_ck): its pass 1 works from the forward's FINAL maximum, so its sums and
    the forward's alpha_sum are rounded differently whatever the kernels, and the dq formula that combines them amplifies that
    by |alpha_kvw| / alpha_sum, which grows with the head width (3.5e-5 on values of magnitude 1 at 128 channels).
    Any storage dtype: 16-bit rows are widened as they are staged, tiles, matrix instructions and state are fp32."""
    ck, cv = kx.shape[3], vx.shape[3]
    if qy.dtype not in _DTYPE_CODE or ck != cv or ck % 4 or not 16 <= ck <= max_ck or nlon_in // pscale < 32:
        return False
    return True


def _ring_validate(kx, vx, qy, dy, state, quad_weights, col_idx, row_off, row_idx, nlat_out, nlon_out, nrows=None):
    """state: (name, tensor, trailing channel count or None) fp32 buffers shaped like the local output grid; nrows: rows of
    the CSR (output latitudes in the gather direction, the chunk's input latitudes in the scatter direction); row_idx only
    exists in the gather direction."""
    for name, t in (("kx", kx), ("vx", vx), ("qy", qy)) + ((("dy", dy),) if dy is not None else ()):
        if t.dim() != 4 or not t.is_contiguous():
            raise RuntimeError(f"{name} must be a contiguous 4-dimensional (batch*heads, nlat, nlon, channels) tensor")
        _require_gpu(t, name, kx.device)
        if t.dtype != qy.dtype or t.dtype not in _DTYPE_CODE:
            raise RuntimeError(f"{name} has dtype {t.dtype}; k, v, q and dy must share one of fp32, bf16, fp16")
    if kx.shape[:3] != vx.shape[:3] or kx.shape[0] != qy.shape[0] or kx.shape[3] != qy.shape[3]:
        raise RuntimeError("kx and vx must share (batch, nlat_halo, nlon_kx); qy must share batch and channels with kx")
    if tuple(qy.shape[1:3]) != (nlat_out, nlon_out):
        raise RuntimeError(f"qy must be (batch, nlat_out={nlat_out}, nlon_out={nlon_out}, channels)")
    if dy is not None and (dy.shape[:3] != qy.shape[:3] or dy.shape[3] != vx.shape[3]):
        raise RuntimeError("dy must be (batch, nlat_out, nlon_out, v channels)")
    for name, t, c in state:
        want = (qy.shape[0], nlat_out, nlon_out) + (() if c is None else (c,))
        if tuple(t.shape) != want or t.dtype != torch.float32 or not t.is_contiguous():
            raise RuntimeError(f"{name} must be a contiguous fp32 tensor of shape {want}")
        _require_gpu(t, name, kx.device)
    index = (("quad_weights", quad_weights, torch.float32), ("col_idx", col_idx, torch.int64), ("row_off", row_off, torch.int64))
    for name, t, dt in index + ((("row_idx", row_idx, torch.int32),) if row_idx is not None else ()):
        if t.dtype != dt or not t.is_contiguous():
            raise RuntimeError(f"{name} must be a contiguous {dt} tensor")
        _require_gpu(t, name, kx.device)
    nrows = nlat_out if nrows is None else nrows
    if row_off.numel() != nrows + 1 or (row_idx is not None and row_idx.numel() != nrows):
        raise RuntimeError(f"row_off must have {nrows + 1} entries" + ("" if row_idx is None else f" and row_idx {nrows}"))


@torch.library.custom_op("attention_kernels::forward_ring_step", mutates_args=("y_acc", "alpha_sum_buf", "qdotk_max_buf"))
def forward_ring_step(
    kx: torch.Tensor,
    vx: torch.Tensor,
    qy: torch.Tensor,
    y_acc: torch.Tensor,
    alpha_sum_buf: torch.Tensor,
    qdotk_max_buf: torch.Tensor,
    quad_weights: torch.Tensor,
    col_idx: torch.Tensor,
    row_off: torch.Tensor,
    row_idx: torch.Tensor,
    nlon_in: int,
    pscale: int,
    lon_lo_kx: int,
    lat_halo_start: int,
    nlat_out: int,
    nlon_out: int,
    n_long_rows: int,
    max_row_len: int,
    mid_row_len: int,
) -> None:
    state = (("y_acc", y_acc, vx.shape[3]), ("alpha_sum_buf", alpha_sum_buf, None), ("qdotk_max_buf", qdotk_max_buf, None))
    _ring_validate(kx, vx, qy, None, state, quad_weights, col_idx, row_off, row_idx, nlat_out, nlon_out)
    if qy.numel() == 0 or kx.numel() == 0 or col_idx.numel() == 0:  # nothing to fold in
        return
    shape = _ring_shape(kx, vx, qy, nlon_in, pscale, lon_lo_kx, lat_halo_start, nlat_out, nlon_out)
    if _ring_takes_plan(kx, vx, qy, nlon_in, pscale) and all(t.data_ptr() % 16 == 0 for t in (kx, vx, qy, y_acc)):
        # band-staged matrix-core step on the run-length plan of the local psi (built on the host once per psi, cached)
        p = _plan.get_plan(col_idx, row_off, quad_weights.numel(), nlon_in, nlat_out, nlon_in // pscale)
        with torch.cuda.device(kx.device):
            rc = _lib.load().s2attn_ring_forward_step_plan(
                kx.data_ptr(), vx.data_ptr(), qy.data_ptr(), y_acc.data_ptr(), alpha_sum_buf.data_ptr(), qdotk_max_buf.data_ptr(),
                quad_weights.data_ptr(), ctypes.byref(p.struct), ctypes.byref(shape), _stream_ptr(kx.device),
            )  # fmt: skip
        _lib.check(rc, "s2attn_ring_forward_step_plan")
        return
    with torch.cuda.device(kx.device):
        rc = _lib.load().s2attn_ring_forward_step(
            kx.data_ptr(), vx.data_ptr(), qy.data_ptr(), y_acc.data_ptr(), alpha_sum_buf.data_ptr(), qdotk_max_buf.data_ptr(),
            quad_weights.data_ptr(), col_idx.data_ptr(), row_off.data_ptr(), row_idx.data_ptr(), ctypes.byref(shape), _stream_ptr(kx.device),
        )  # fmt: skip
    _lib.check(rc, "s2attn_ring_forward_step")


@forward_ring_step.register_fake
def _(kx, vx, qy, y_acc, alpha_sum_buf, qdotk_max_buf, quad_weights, col_idx, row_off, row_idx, nlon_in, pscale, lon_lo_kx, lat_halo_start, nlat_out, nlon_out, n_long_rows, max_row_len, mid_row_len):
    return None


@torch.library.custom_op(
    "attention_kernels::backward_ring_step_pass1", mutates_args=("alpha_sum_buf", "qdotk_max_buf", "integral_buf", "alpha_k_buf", "alpha_kvw_buf")
)
def backward_ring_step_pass1(
    kx: torch.Tensor,
    vx: torch.Tensor,
    qy: torch.Tensor,
    dy: torch.Tensor,
    alpha_sum_buf: torch.Tensor,
    qdotk_max_buf: torch.Tensor,
    integral_buf: torch.Tensor,
    alpha_k_buf: torch.Tensor,
    alpha_kvw_buf: torch.Tensor,
    quad_weights: torch.Tensor,
    col_idx: torch.Tensor,
    row_off: torch.Tensor,
    row_idx: torch.Tensor,
    nlon_in: int,
    pscale: int,
    lon_lo_kx: int,
    lat_halo_start: int,
    nlat_out: int,
    nlon_out: int,
    n_long_rows: int,
    max_row_len: int,
    mid_row_len: int,
) -> None:
    ck = kx.shape[3]
    state = (("alpha_sum_buf", alpha_sum_buf, None), ("qdotk_max_buf", qdotk_max_buf, None), ("integral_buf", integral_buf, None),
             ("alpha_k_buf", alpha_k_buf, ck), ("alpha_kvw_buf", alpha_kvw_buf, ck))  # fmt: skip
    _ring_validate(kx, vx, qy, dy, state, quad_weights, col_idx, row_off, row_idx, nlat_out, nlon_out)
    if qy.numel() == 0 or kx.numel() == 0 or col_idx.numel() == 0:  # nothing to fold in
        return
    shape = _ring_shape(kx, vx, qy, nlon_in, pscale, lon_lo_kx, lat_halo_start, nlat_out, nlon_out)
    if _ring_takes_plan(kx, vx, qy, nlon_in, pscale) and all(t.data_ptr() % 16 == 0 for t in (kx, vx, qy, dy, alpha_k_buf, alpha_kvw_buf)):
        p = _plan.get_plan(col_idx, row_off, quad_weights.numel(), nlon_in, nlat_out, nlon_in // pscale)
        with torch.cuda.device(kx.device):
            rc = _lib.load().s2attn_ring_backward_pass1_plan(
                kx.data_ptr(), vx.data_ptr(), qy.data_ptr(), dy.data_ptr(), alpha_sum_buf.data_ptr(), qdotk_max_buf.data_ptr(),
                integral_buf.data_ptr(), alpha_k_buf.data_ptr(), alpha_kvw_buf.data_ptr(), quad_weights.data_ptr(),
                ctypes.byref(p.struct), ctypes.byref(shape), _stream_ptr(kx.device),
            )  # fmt: skip
        _lib.check(rc, "s2attn_ring_backward_pass1_plan")
        return
    with torch.cuda.device(kx.device):
        rc = _lib.load().s2attn_ring_backward_pass1(
            kx.data_ptr(), vx.data_ptr(), qy.data_ptr(), dy.data_ptr(), alpha_sum_buf.data_ptr(), qdotk_max_buf.data_ptr(),
            integral_buf.data_ptr(), alpha_k_buf.data_ptr(), alpha_kvw_buf.data_ptr(), quad_weights.data_ptr(), col_idx.data_ptr(),
            row_off.data_ptr(), row_idx.data_ptr(), ctypes.byref(shape), _stream_ptr(kx.device),
        )  # fmt: skip
    _lib.check(rc, "s2attn_ring_backward_pass1")


@backward_ring_step_pass1.register_fake
def _(kx, vx, qy, dy, alpha_sum_buf, qdotk_max_buf, integral_buf, alpha_k_buf, alpha_kvw_buf, quad_weights, col_idx, row_off, row_idx, nlon_in, pscale, lon_lo_kx, lat_halo_start, nlat_out, nlon_out, n_long_rows, max_row_len, mid_row_len):
    return None


# Pass 2 runs on the transposed neighborhood (sums in registers, fixed order); True selects the library's other entry point,
# which walks the CSR as given and adds with fp32 atomics (the reference's formulation), for comparison and tests.
_RING_PASS2_FROM_CSR = False


@torch.library.custom_op("attention_kernels::backward_ring_step_pass2", mutates_args=("dkx", "dvx"))
def backward_ring_step_pass2(
    kx: torch.Tensor,
    vx: torch.Tensor,
    qy: torch.Tensor,
    dy: torch.Tensor,
    alpha_sum_buf: torch.Tensor,
    qdotk_max_buf: torch.Tensor,
    integral_norm_buf: torch.Tensor,
    dkx: torch.Tensor,
    dvx: torch.Tensor,
    quad_weights: torch.Tensor,
    col_idx: torch.Tensor,
    row_off: torch.Tensor,
    row_idx: torch.Tensor,
    nlon_in: int,
    pscale: int,
    lon_lo_kx: int,
    lat_halo_start: int,
    nlat_out: int,
    nlon_out: int,
    n_long_rows: int,
    max_row_len: int,
    mid_row_len: int,
) -> None:
    state = (("alpha_sum_buf", alpha_sum_buf, None), ("qdotk_max_buf", qdotk_max_buf, None), ("integral_norm_buf", integral_norm_buf, None))
    _ring_validate(kx, vx, qy, dy, state, quad_weights, col_idx, row_off, row_idx, nlat_out, nlon_out)
    for name, t, like in (("dkx", dkx, kx), ("dvx", dvx, vx)):
        if t.shape != like.shape or t.dtype != torch.float32 or not t.is_contiguous():
            raise RuntimeError(f"{name} must be a contiguous fp32 tensor shaped like its input, {tuple(like.shape)}")
        _require_gpu(t, name, kx.device)
    if qy.numel() == 0 or kx.numel() == 0 or col_idx.numel() == 0:
        return
    shape = _ring_shape(kx, vx, qy, nlon_in, pscale, lon_lo_kx, lat_halo_start, nlat_out, nlon_out)
    head = (kx.data_ptr(), vx.data_ptr(), qy.data_ptr(), dy.data_ptr(), alpha_sum_buf.data_ptr(), qdotk_max_buf.data_ptr(),
            integral_norm_buf.data_ptr(), dkx.data_ptr(), dvx.data_ptr(), quad_weights.data_ptr())  # fmt: skip
    if not _RING_PASS2_FROM_CSR and _ring_takes_plan(kx, vx, qy, nlon_in, pscale) and all(t.data_ptr() % 16 == 0 for t in (kx, vx, qy, dy, dkx, dvx)):
        p = _plan.get_plan(col_idx, row_off, quad_weights.numel(), nlon_in, nlat_out, nlon_in // pscale)
        with torch.cuda.device(kx.device):
            rc = _lib.load().s2attn_ring_backward_pass2_plan(*head, ctypes.byref(p.struct), ctypes.byref(shape), _stream_ptr(kx.device))
        _lib.check(rc, "s2attn_ring_backward_pass2_plan")
        return
    with torch.cuda.device(kx.device):
        if _RING_PASS2_FROM_CSR:
            rc = _lib.load().s2attn_ring_backward_pass2(*head, col_idx.data_ptr(), row_off.data_ptr(), row_idx.data_ptr(), ctypes.byref(shape), _stream_ptr(kx.device))
        else:
            t_lat, t_lon, t_off, t_order = get_transposed_csr(col_idx, row_off, nlon_in, lat_halo_start, kx.shape[1])  # psi regrouped by input latitude
            rc = _lib.load().s2attn_ring_backward_pass2_transposed(*head, t_lat.data_ptr(), t_lon.data_ptr(), t_off.data_ptr(), t_order.data_ptr(), ctypes.byref(shape), _stream_ptr(kx.device))
    _lib.check(rc, "s2attn_ring_backward_pass2")


@backward_ring_step_pass2.register_fake
def _(kx, vx, qy, dy, alpha_sum_buf, qdotk_max_buf, integral_norm_buf, dkx, dvx, quad_weights, col_idx, row_off, row_idx, nlon_in, pscale, lon_lo_kx, lat_halo_start, nlat_out, nlon_out, n_long_rows, max_row_len, mid_row_len):
    return None


# ---- up-sampling direction (attention_interface.cpp:158-189, fake kernels attention_optimized.py:163-227) ------------
def _ring_up_shape(kx, vx, qy, nlon_out_global, pscale_out, lon_lo_kx, lat_halo_start, nlat_out, nlon_out) -> _lib.RingUpShapeStruct:
    B, nlat_halo, nlon_kx, ck = kx.shape
    return _lib.RingUpShapeStruct(B, nlat_halo, nlon_kx, nlat_out, nlon_out, ck, vx.shape[3], nlon_out_global, pscale_out, lon_lo_kx, lat_halo_start, _DTYPE_CODE[qy.dtype])


def _ring_up_validate(kx, vx, qy, dy, state, quad_weights, col_idx, row_off, nlat_out, nlon_out):
    _ring_validate(kx, vx, qy, dy, state, quad_weights, col_idx, row_off, None, nlat_out, nlon_out, nrows=kx.shape[1])


@torch.library.custom_op("attention_kernels::forward_ring_step_upsample", mutates_args=("y_acc", "alpha_sum_buf", "qdotk_max_buf"))
def forward_ring_step_upsample(
    kx: torch.Tensor,
    vx: torch.Tensor,
    qy: torch.Tensor,
    y_acc: torch.Tensor,
    alpha_sum_buf: torch.Tensor,
    qdotk_max_buf: torch.Tensor,
    quad_weights: torch.Tensor,
    col_idx: torch.Tensor,
    row_off: torch.Tensor,
    nlon_in: int,
    nlon_out_global: int,
    pscale_out: int,
    lon_lo_kx: int,
    lat_halo_start: int,
    nlat_out: int,
    nlon_out: int,
) -> None:
    state = (("y_acc", y_acc, vx.shape[3]), ("alpha_sum_buf", alpha_sum_buf, None), ("qdotk_max_buf", qdotk_max_buf, None))
    _ring_up_validate(kx, vx, qy, None, state, quad_weights, col_idx, row_off, nlat_out, nlon_out)
    if qy.numel() == 0 or kx.numel() == 0 or col_idx.numel() == 0:
        return
    shape = _ring_up_shape(kx, vx, qy, nlon_out_global, pscale_out, lon_lo_kx, lat_halo_start, nlat_out, nlon_out)
    if _ring_takes_plan(kx, vx, qy, nlon_in, 1, 64) and all(t.data_ptr() % 16 == 0 for t in (kx, vx, qy, y_acc)):
        # band-staged matrix-core step on the run-length plan of the local psi (rows = the chunk's latitudes)
        p = _plan.get_plan(col_idx, row_off, kx.shape[1], nlon_in, nlat_out, nlon_out_global)
        with torch.cuda.device(kx.device):
            rc = _lib.load().s2attn_ring_forward_step_upsample_plan(
                kx.data_ptr(), vx.data_ptr(), qy.data_ptr(), y_acc.data_ptr(), alpha_sum_buf.data_ptr(), qdotk_max_buf.data_ptr(),
                quad_weights.data_ptr(), ctypes.byref(p.struct), ctypes.byref(shape), _stream_ptr(kx.device),
            )  # fmt: skip
        _lib.check(rc, "s2attn_ring_forward_step_upsample_plan")
        return
    with torch.cuda.device(kx.device):
        t_lat, t_lon, t_off, _ = get_transposed_csr(col_idx, row_off, nlon_out_global, 0, nlat_out)  # psi regrouped by output latitude
        rc = _lib.load().s2attn_ring_forward_step_upsample(
            kx.data_ptr(), vx.data_ptr(), qy.data_ptr(), y_acc.data_ptr(), alpha_sum_buf.data_ptr(), qdotk_max_buf.data_ptr(),
            quad_weights.data_ptr(), t_lat.data_ptr(), t_lon.data_ptr(), t_off.data_ptr(), ctypes.byref(shape), _stream_ptr(kx.device),
        )  # fmt: skip
    _lib.check(rc, "s2attn_ring_forward_step_upsample")


@forward_ring_step_upsample.register_fake
def _(kx, vx, qy, y_acc, alpha_sum_buf, qdotk_max_buf, quad_weights, col_idx, row_off, nlon_in, nlon_out_global, pscale_out, lon_lo_kx, lat_halo_start, nlat_out, nlon_out):
    return None


@torch.library.custom_op("attention_kernels::backward_ring_step_upsample_pass1", mutates_args=("integral_buf", "alpha_k_buf", "alpha_kvw_buf"))
def backward_ring_step_upsample_pass1(
    kx: torch.Tensor,
    vx: torch.Tensor,
    qy: torch.Tensor,
    dy: torch.Tensor,
    qdotk_max_buf: torch.Tensor,
    integral_buf: torch.Tensor,
    alpha_k_buf: torch.Tensor,
    alpha_kvw_buf: torch.Tensor,
    quad_weights: torch.Tensor,
    col_idx: torch.Tensor,
    row_off: torch.Tensor,
    nlon_in: int,
    nlon_out_global: int,
    pscale_out: int,
    lon_lo_kx: int,
    lat_halo_start: int,
    nlat_out: int,
    nlon_out: int,
) -> None:
    ck = kx.shape[3]
    state = (("qdotk_max_buf", qdotk_max_buf, None), ("integral_buf", integral_buf, None), ("alpha_k_buf", alpha_k_buf, ck), ("alpha_kvw_buf", alpha_kvw_buf, ck))
    _ring_up_validate(kx, vx, qy, dy, state, quad_weights, col_idx, row_off, nlat_out, nlon_out)
    if qy.numel() == 0 or kx.numel() == 0 or col_idx.numel() == 0:
        return
    shape = _ring_up_shape(kx, vx, qy, nlon_out_global, pscale_out, lon_lo_kx, lat_halo_start, nlat_out, nlon_out)
    if _ring_takes_plan(kx, vx, qy, nlon_in, 1, 64) and all(t.data_ptr() % 16 == 0 for t in (kx, vx, qy, dy, alpha_k_buf, alpha_kvw_buf)):
        p = _plan.get_plan(col_idx, row_off, kx.shape[1], nlon_in, nlat_out, nlon_out_global)
        with torch.cuda.device(kx.device):
            rc = _lib.load().s2attn_ring_backward_pass1_upsample_plan(
                kx.data_ptr(), vx.data_ptr(), qy.data_ptr(), dy.data_ptr(), qdotk_max_buf.data_ptr(), integral_buf.data_ptr(), alpha_k_buf.data_ptr(),
                alpha_kvw_buf.data_ptr(), quad_weights.data_ptr(), ctypes.byref(p.struct), ctypes.byref(shape), _stream_ptr(kx.device),
            )  # fmt: skip
        _lib.check(rc, "s2attn_ring_backward_pass1_upsample_plan")
        return
    with torch.cuda.device(kx.device):
        t_lat, t_lon, t_off, _ = get_transposed_csr(col_idx, row_off, nlon_out_global, 0, nlat_out)
        rc = _lib.load().s2attn_ring_backward_pass1_upsample(
            kx.data_ptr(), vx.data_ptr(), qy.data_ptr(), dy.data_ptr(), qdotk_max_buf.data_ptr(), integral_buf.data_ptr(), alpha_k_buf.data_ptr(),
            alpha_kvw_buf.data_ptr(), quad_weights.data_ptr(), t_lat.data_ptr(), t_lon.data_ptr(), t_off.data_ptr(), ctypes.byref(shape), _stream_ptr(kx.device),
        )  # fmt: skip
    _lib.check(rc, "s2attn_ring_backward_pass1_upsample")


@backward_ring_step_upsample_pass1.register_fake
def _(kx, vx, qy, dy, qdotk_max_buf, integral_buf, alpha_k_buf, alpha_kvw_buf, quad_weights, col_idx, row_off, nlon_in, nlon_out_global, pscale_out, lon_lo_kx, lat_halo_start, nlat_out, nlon_out):
    return None


@torch.library.custom_op("attention_kernels::backward_ring_step_upsample_pass2", mutates_args=("dkx", "dvx"))
def backward_ring_step_upsample_pass2(
    kx: torch.Tensor,
    vx: torch.Tensor,
    qy: torch.Tensor,
    dy: torch.Tensor,
    alpha_sum_buf: torch.Tensor,
    qdotk_max_buf: torch.Tensor,
    integral_norm_buf: torch.Tensor,
    dkx: torch.Tensor,
    dvx: torch.Tensor,
    quad_weights: torch.Tensor,
    col_idx: torch.Tensor,
    row_off: torch.Tensor,
    nlon_in: int,
    nlon_out_global: int,
    pscale_out: int,
    lon_lo_kx: int,
    lat_halo_start: int,
    nlat_out: int,
    nlon_out: int,
) -> None:
    state = (("alpha_sum_buf", alpha_sum_buf, None), ("qdotk_max_buf", qdotk_max_buf, None), ("integral_norm_buf", integral_norm_buf, None))
    _ring_up_validate(kx, vx, qy, dy, state, quad_weights, col_idx, row_off, nlat_out, nlon_out)
    for name, t, like in (("dkx", dkx, kx), ("dvx", dvx, vx)):
        if t.shape != like.shape or t.dtype != torch.float32 or not t.is_contiguous():
            raise RuntimeError(f"{name} must be a contiguous fp32 tensor shaped like its input, {tuple(like.shape)}")
        _require_gpu(t, name, kx.device)
    if kx.numel() == 0:
        return
    if qy.numel() == 0 or col_idx.numel() == 0:  # no output cell sees the chunk: the step still writes every element
        dkx.zero_()
        dvx.zero_()
        return
    shape = _ring_up_shape(kx, vx, qy, nlon_out_global, pscale_out, lon_lo_kx, lat_halo_start, nlat_out, nlon_out)
    if _ring_takes_plan(kx, vx, qy, nlon_in, 1, 64) and all(t.data_ptr() % 16 == 0 for t in (kx, vx, qy, dy, dkx, dvx)):
        p = _plan.get_plan(col_idx, row_off, kx.shape[1], nlon_in, nlat_out, nlon_out_global)
        with torch.cuda.device(kx.device):
            rc = _lib.load().s2attn_ring_backward_pass2_upsample_plan(
                kx.data_ptr(), vx.data_ptr(), qy.data_ptr(), dy.data_ptr(), alpha_sum_buf.data_ptr(), qdotk_max_buf.data_ptr(), integral_norm_buf.data_ptr(),
                dkx.data_ptr(), dvx.data_ptr(), quad_weights.data_ptr(), ctypes.byref(p.struct), ctypes.byref(shape), _stream_ptr(kx.device),
            )  # fmt: skip
        _lib.check(rc, "s2attn_ring_backward_pass2_upsample_plan")
        return
    with torch.cuda.device(kx.device):
        rc = _lib.load().s2attn_ring_backward_pass2_upsample(
            kx.data_ptr(), vx.data_ptr(), qy.data_ptr(), dy.data_ptr(), alpha_sum_buf.data_ptr(), qdotk_max_buf.data_ptr(), integral_norm_buf.data_ptr(),
            dkx.data_ptr(), dvx.data_ptr(), quad_weights.data_ptr(), col_idx.data_ptr(), row_off.data_ptr(), get_row_order(row_off).data_ptr(),
            ctypes.byref(shape), _stream_ptr(kx.device),
        )  # fmt: skip
    _lib.check(rc, "s2attn_ring_backward_pass2_upsample")


@backward_ring_step_upsample_pass2.register_fake
def _(kx, vx, qy, dy, alpha_sum_buf, qdotk_max_buf, integral_norm_buf, dkx, dvx, quad_weights, col_idx, row_off, nlon_in, nlon_out_global, pscale_out, lon_lo_kx, lat_halo_start, nlat_out, nlon_out):
    return None
