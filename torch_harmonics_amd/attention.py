"""
NeighborhoodAttentionS2: attention restricted to a geodesic disk around every output point of
a spherical grid, weighted by the grid's quadrature.

Constructor arguments, parameter names and shapes, buffers and forward semantics follow
torch_harmonics/attention/attention.py:253-571 so that a state_dict moves between the two
implementations unchanged.  The attention itself runs in the HIP kernels of libs2attn.so.
"""

import math
from typing import Optional, Tuple, Union

import torch
import torch.nn as nn
import torch.nn.functional as F

from ._attention_utils import _check_dtypes_match, _check_extent, _check_ndim
from ._layout import to_nchw, to_nhwc
from .neighborhood import precompute_neighborhood_s2
from .ops import neighborhood_s2_attention, takes_column_blocks
from .plan import cached_host_blob
from .quadrature import precompute_latitudes

__all__ = ["NeighborhoodAttentionS2"]


def _weight_grad(g: torch.Tensor, x: torch.Tensor) -> torch.Tensor:
    """g^T @ x for g (N, Cout), x (N, Cin) with N in the hundreds of thousands and a few hundred channels: the reduction
    over N is split into S slices that run as one batched GEMM and are then added up.  The single tall GEMM leaves most
    of the GPU idle (2.2 ms at N = 1M, C = 256 against 1.1 ms split; 0.5 ms against 0.04 ms at N = 260K, C = 64)."""
    n = g.shape[0]
    slices = max(1, min(64, n // 8192))
    if slices == 1:
        return g.t() @ x
    for s in range(slices, slices // 2, -1):  # a slice count that divides n leaves no remainder GEMM and no extra add
        if n % s == 0:
            slices = s
            break
    rows = n // slices
    main = slices * rows
    out = torch.bmm(g[:main].view(slices, rows, -1).transpose(1, 2), x[:main].view(slices, rows, -1)).sum(0)
    if main < n:
        out = out + g[main:].t() @ x[main:]
    return out


class _Linear1x1(torch.autograd.Function):
    """F.linear on (..., Cin) with its weight gradient computed by _weight_grad; forward and input gradient as F.linear's."""

    @staticmethod
    def forward(ctx, x, weight, bias):
        y = F.linear(x, weight, bias)
        ctx.save_for_backward(x, weight)
        ctx.bias_dtype = None if bias is None else bias.dtype
        return y

    @staticmethod
    def backward(ctx, g):
        x, weight = ctx.saved_tensors
        g2 = g.reshape(-1, g.shape[-1])
        gx = gw = gb = None
        if ctx.needs_input_grad[0]:
            gx = (g2 @ weight.to(g2.dtype)).reshape(x.shape).to(x.dtype)
        if ctx.needs_input_grad[1]:
            gw = _weight_grad(g2, x.reshape(-1, x.shape[-1]).to(g2.dtype)).to(weight.dtype)
        if ctx.bias_dtype is not None and ctx.needs_input_grad[2]:
            gb = g2.sum(0).to(ctx.bias_dtype)
        return gx, gw, gb


class _SharedInputLinear1x1(torch.autograd.Function):
    """Several _Linear1x1 projections of ONE input (self-attention: q, k, v; cross-attention with key is value: k, v).  Forward
    is one F.linear per projection; the backward accumulates the input gradient inside the GEMMs (beta = 1) instead of
    leaving autograd to add up one full-size tensor per projection with elementwise kernels (two 2 GB adds at 721 x 1440,
    256 channels)."""

    @staticmethod
    def forward(ctx, x, *params):  # params = (w0, b0, w1, b1, ...), biases may be None
        weights, biases = params[0::2], params[1::2]
        ctx.save_for_backward(x, *weights)
        ctx.bias_dtypes = [None if b is None else b.dtype for b in biases]
        return tuple(F.linear(x, w, b) for w, b in zip(weights, biases))

    @staticmethod
    def backward(ctx, *grads):
        x, *weights = ctx.saved_tensors
        x2 = x.reshape(-1, x.shape[-1])
        gx = None
        out = []
        for i, (g, w) in enumerate(zip(grads, weights)):
            gw = gb = None
            if g is not None:
                g2 = g.reshape(-1, g.shape[-1])
                if ctx.needs_input_grad[0]:
                    if gx is None:
                        gx = g2 @ w.to(g2.dtype)
                    elif gx.dtype == g2.dtype:
                        gx.addmm_(g2, w.to(g2.dtype))
                    else:  # gradients of different dtypes (not produced by this module): plain accumulation
                        gx = gx + (g2 @ w.to(g2.dtype)).to(gx.dtype)
                if ctx.needs_input_grad[1 + 2 * i]:
                    gw = _weight_grad(g2, x2.to(g2.dtype)).to(w.dtype)
                if ctx.bias_dtypes[i] is not None and ctx.needs_input_grad[2 + 2 * i]:
                    gb = g2.sum(0).to(ctx.bias_dtypes[i])
            out += [gw, gb]
        if gx is not None:
            gx = gx.reshape(x.shape).to(x.dtype)
        return (gx, *out)


def _column_blocks_of_one_buffer(grads, widths):
    """The 2-D (N, sum(widths)) buffer whose consecutive column blocks the given gradients are, or None."""
    g0 = grads[0]
    total = sum(widths)
    if g0 is None or g0.dim() != 4 or g0.stride(3) != 1 or g0.stride(2) != total:
        return None
    off = g0.storage_offset()
    for g, w in zip(grads, widths):
        if g is None or g.shape[3] != w or g.shape[:3] != g0.shape[:3] or g.stride() != g0.stride() or g.dtype != g0.dtype:
            return None
        if g.untyped_storage().data_ptr() != g0.untyped_storage().data_ptr() or g.storage_offset() != off:
            return None
        off += w
    n = g0.shape[0] * g0.shape[1] * g0.shape[2]
    if g0.stride(1) != g0.shape[2] * total or g0.stride(0) != g0.shape[1] * g0.shape[2] * total:
        return None
    return torch.as_strided(g0, (n, total), (total, 1), g0.storage_offset())


class _FusedLinear1x1(torch.autograd.Function):
    """Several projections of ONE input as ONE GEMM with the concatenated weight: the outputs are the column blocks of one
    (..., sum of widths) buffer, which the attention kernels read in place.  When the gradients come back as column blocks
    of one buffer as well (the attention backward writes them that way), the input gradient, the weight gradients and the
    bias gradients are one GEMM, one split-K GEMM and one reduction over that buffer; otherwise they are concatenated first.
    (The reference runs three F.linear, attention.py:530-532.)"""

    @staticmethod
    def forward(ctx, x, *params):  # params = (w0, b0, w1, b1, ...), biases all present or all None
        weights, biases = params[0::2], params[1::2]
        wcat = torch.cat(weights, 0)
        bcat = None if biases[0] is None else torch.cat(biases, 0)
        ctx.save_for_backward(x, wcat)
        ctx.widths = [w.shape[0] for w in weights]
        ctx.has_bias = bcat is not None
        buf = F.linear(x, wcat, bcat)
        return tuple(buf.split(ctx.widths, dim=-1))

    @staticmethod
    def backward(ctx, *grads):
        x, wcat = ctx.saved_tensors
        x2 = x.reshape(-1, x.shape[-1])
        if any(g is None for g in grads):
            like = next(g for g in grads if g is not None)
            grads = tuple(g if g is not None else like.new_zeros(like.shape[:-1] + (w,)) for g, w in zip(grads, ctx.widths))
        g2 = _column_blocks_of_one_buffer(grads, ctx.widths)
        if g2 is None:
            g2 = torch.cat([g.reshape(-1, g.shape[-1]) for g in grads], 1)
        gx = gwcat = gbcat = None
        if ctx.needs_input_grad[0]:
            gx = (g2 @ wcat.to(g2.dtype)).reshape(x.shape).to(x.dtype)
        if any(ctx.needs_input_grad[1::2]):
            gwcat = _weight_grad(g2, x2.to(g2.dtype)).to(wcat.dtype)
        if ctx.has_bias and any(ctx.needs_input_grad[2::2]):
            gbcat = g2.sum(0)
        out = []
        ofs = 0
        for i, w in enumerate(ctx.widths):
            gw = gwcat[ofs : ofs + w] if gwcat is not None and ctx.needs_input_grad[1 + 2 * i] else None
            gb = gbcat[ofs : ofs + w] if gbcat is not None and ctx.needs_input_grad[2 + 2 * i] else None
            out += [gw, gb]
            ofs += w
        return (gx, *out)


_MAX_NCHW_BATCH = 8  # the projections fed straight from / to NCHW run one GEMM per batch element


def _weight_grad_nchw(g: torch.Tensor, x: torch.Tensor) -> torch.Tensor:
    """g^T @ x^T for g (N, Cout) and x (Cin, N), i.e. _weight_grad with the second operand given channel-major (one batch
    element of an NCHW tensor): the same split of the reduction over N, the slices of x read in place as transposed operands."""
    n = g.shape[0]
    slices = max(1, min(64, n // 8192))
    if slices == 1:
        return g.t() @ x.t()
    for s in range(slices, slices // 2, -1):
        if n % s == 0:
            slices = s
            break
    rows = n // slices
    main = slices * rows
    out = torch.bmm(g[:main].view(slices, rows, -1).transpose(1, 2), x[:, :main].view(x.shape[0], slices, rows).permute(1, 2, 0)).sum(0)
    if main < n:
        out = out + g[main:].t() @ x[:, main:].t()
    return out


class _FusedLinear1x1NCHW(torch.autograd.Function):
    """_FusedLinear1x1 fed straight from the module's NCHW input: x[b] viewed as (Cin, H*W) is the transposed operand of the
    GEMM, so the channels-last copy of the input (0.5 ms at 721 x 1440 x 256) is never made, and the input gradient is
    produced as W^T (Cin, total) times the transposed gradient buffer, i.e. directly in NCHW.  Outputs as _FusedLinear1x1:
    NHWC column blocks of one buffer.  One GEMM per batch element (the batch of such grids is small)."""

    @staticmethod
    def forward(ctx, x, *params):  # x (B, Cin, H, W) contiguous; params = (w0, b0, w1, b1, ...), biases all present or all None
        weights, biases = params[0::2], params[1::2]
        wcat = torch.cat(weights, 0) if len(weights) > 1 else weights[0]
        bcat = None if biases[0] is None else (torch.cat(biases, 0) if len(biases) > 1 else biases[0])
        ctx.save_for_backward(x, wcat)
        ctx.widths = [w.shape[0] for w in weights]
        ctx.has_bias = bcat is not None
        B, C, H, W = x.shape
        total = wcat.shape[0]
        buf = x.new_empty(B, H, W, total)
        for b in range(B):
            xt, ob = x[b].view(C, H * W).t(), buf[b].view(H * W, total)
            if bcat is None:
                torch.mm(xt, wcat.t(), out=ob)
            else:
                torch.addmm(bcat, xt, wcat.t(), out=ob)
        return tuple(buf.split(ctx.widths, dim=-1))

    @staticmethod
    def backward(ctx, *grads):
        x, wcat = ctx.saved_tensors
        B, C, H, W = x.shape
        if any(g is None for g in grads):
            like = next(g for g in grads if g is not None)
            grads = tuple(g if g is not None else like.new_zeros(like.shape[:-1] + (w,)) for g, w in zip(grads, ctx.widths))
        g2 = _column_blocks_of_one_buffer(grads, ctx.widths)
        if g2 is None:
            g2 = torch.cat([g.reshape(-1, g.shape[-1]) for g in grads], 1)
        g3 = g2.view(B, H * W, -1)
        gx = gwcat = gbcat = None
        if ctx.needs_input_grad[0]:
            gx = torch.empty_like(x)
            for b in range(B):
                torch.mm(wcat.t(), g3[b].t(), out=gx[b].view(C, H * W))
        if any(ctx.needs_input_grad[1::2]):
            for b in range(B):
                gwb = _weight_grad_nchw(g3[b], x[b].view(C, H * W))
                gwcat = gwb if gwcat is None else gwcat + gwb
        if ctx.has_bias and any(ctx.needs_input_grad[2::2]):
            gbcat = g2.sum(0)
        out = []
        ofs = 0
        for i, w in enumerate(ctx.widths):
            gw = gwcat[ofs : ofs + w] if gwcat is not None and ctx.needs_input_grad[1 + 2 * i] else None
            gb = gbcat[ofs : ofs + w] if gbcat is not None and ctx.needs_input_grad[2 + 2 * i] else None
            out += [gw, gb]
            ofs += w
        return (gx, *out)


class _Linear1x1ToNCHW(torch.autograd.Function):
    """The output projection from the NHWC attention output straight to the module's NCHW output: out[b] (Cout, H*W) =
    W y[b]^T (+ bias per row), and in the backward the NCHW gradient is the transposed operand of both GEMMs - neither the
    channels-first copy of the output nor the channels-last copy of its gradient is made."""

    @staticmethod
    def forward(ctx, y, weight, bias):  # y (B, H, W, Cin) contiguous
        ctx.save_for_backward(y, weight)
        ctx.has_bias = bias is not None
        B, H, W, C = y.shape
        out = y.new_empty(B, weight.shape[0], H, W)
        for b in range(B):
            yt, ob = y[b].view(H * W, C).t(), out[b].view(weight.shape[0], H * W)
            if bias is None:
                torch.mm(weight, yt, out=ob)
            else:
                torch.addmm(bias.unsqueeze(1), weight, yt, out=ob)
        return out

    @staticmethod
    def backward(ctx, g):
        y, weight = ctx.saved_tensors
        B, H, W, C = y.shape
        g = g.contiguous()
        g3 = g.view(B, weight.shape[0], H * W)
        gy = gw = gb = None
        if ctx.needs_input_grad[0]:
            gy = torch.empty_like(y)
            for b in range(B):
                torch.mm(g3[b].t(), weight, out=gy[b].view(H * W, C))
        if ctx.needs_input_grad[1]:
            for b in range(B):
                gwb = _weight_grad_nchw(y[b].view(H * W, C), g3[b]).t()
                gw = gwb if gw is None else gw + gwb
        if ctx.has_bias and ctx.needs_input_grad[2]:
            gb = g3.sum((0, 2))
        return gy, gw, gb


def _xavier_uniform(c_out: int, c_in: int, bound: float) -> nn.Parameter:
    return nn.Parameter(bound * (2 * torch.rand(c_out, c_in, 1, 1) - 1))


class NeighborhoodAttentionS2(nn.Module):
    r"""
    Neighborhood attention on the 2-sphere.

    Each output point :math:`x` attends to the input points inside the disk
    :math:`\{x' : d(x, x') \le \theta_\mathrm{cutoff}\}` (great-circle distance); the softmax is
    a quadrature of the continuous attention integral, i.e. every neighbor's weight is multiplied
    by the quadrature weight of its latitude ring.

    Parameters
    ----------
    in_channels : int
        channels of the input signal
    in_shape, out_shape : (nlat, nlon)
        input (key/value) and output (query) grids; ``nlon_in`` must be a multiple of ``nlon_out`` (self-attention,
        down-sampling) or ``nlon_out`` a multiple of ``nlon_in`` (up-sampling)
    grid_in, grid_out : str
        ``"equiangular"``, ``"legendre-gauss"``, ``"lobatto"`` or ``"equiangular-trapezoidal"``
    num_heads : int
        attention heads; must divide ``k_channels`` and ``out_channels``
    scale : float or Tensor, optional
        multiplies the query; default ``1 / sqrt(k_channels // num_heads)``
    use_qknorm : bool
        per-head RMS normalisation of q and k with learnable gain ``1 + w``
    bias : bool
        bias on the four 1x1 projections
    theta_cutoff : float, optional
        disk radius in radians; default one latitude spacing of the output grid, ``pi / (nlat_out - 1)``
    k_channels, out_channels : int, optional
        width of the q/k projection and of the v/output projection; default ``in_channels``
    optimized_kernel : bool
        must stay True: the HIP kernels are the only implementation in this package
    """

    def __init__(
        self,
        in_channels: int,
        in_shape: Tuple[int],
        out_shape: Tuple[int],
        grid_in: Optional[str] = "equiangular",
        grid_out: Optional[str] = "equiangular",
        num_heads: Optional[int] = 1,
        scale: Optional[Union[torch.Tensor, float]] = None,
        use_qknorm: Optional[bool] = False,
        bias: Optional[bool] = True,
        theta_cutoff: Optional[float] = None,
        k_channels: Optional[int] = None,
        out_channels: Optional[int] = None,
        optimized_kernel: Optional[bool] = True,
    ):
        super().__init__()

        self.nlat_in, self.nlon_in = in_shape
        self.nlat_out, self.nlon_out = out_shape

        self.upsample = (self.nlon_out % self.nlon_in == 0) and (self.nlon_in % self.nlon_out != 0)
        if not (self.nlon_in % self.nlon_out == 0 or self.upsample):
            raise ValueError(f"either nlon_in ({self.nlon_in}) must be an integer multiple of nlon_out ({self.nlon_out}), or vice versa, for the attention p-shift to be exact")
        if not optimized_kernel:
            raise NotImplementedError("optimized_kernel=False selects a pure-PyTorch loop in the reference; this package ships the HIP kernels only")
        self.optimized_kernel = True

        self.in_channels = in_channels
        self.num_heads = num_heads
        self.k_channels = in_channels if k_channels is None else k_channels
        self.out_channels = in_channels if out_channels is None else out_channels

        # default radius: one latitude spacing of the coarser grid (the input grid when up-sampling, attention.py:352-356)
        if theta_cutoff is None:
            self.theta_cutoff = torch.pi / float((self.nlat_in if self.upsample else self.nlat_out) - 1)
        else:
            self.theta_cutoff = theta_cutoff
        if self.theta_cutoff <= 0.0:
            raise ValueError("Error, theta_cutoff has to be positive.")

        if self.k_channels % self.num_heads != 0:
            raise ValueError(f"Please make sure that number of heads {self.num_heads} divides k_channels {self.k_channels} evenly.")
        if self.out_channels % self.num_heads != 0:
            raise ValueError(f"Please make sure that number of heads {self.num_heads} divides out_channels {self.out_channels} evenly.")

        # quadrature weight of every input latitude ring, normalised so that the rings sum to 4 pi
        _, wgl = precompute_latitudes(self.nlat_in, grid=grid_in)
        self.register_buffer("quad_weights", 2.0 * torch.pi * wgl.to(dtype=torch.float32) / self.nlon_in, persistent=False)

        # Up-sampling keys psi by the (coarser) input latitude: rows hi, columns ho * nlon_out + wo of the output points inside
        # the disk around input point (hi, 0) -- the same construction with the two grids swapped (attention.py:372-387).
        if self.upsample:
            col_idx, row_off, row_idx = precompute_neighborhood_s2(out_shape, in_shape, grid_in=grid_out, grid_out=grid_in, theta_cutoff=self.theta_cutoff)
        else:
            col_idx, row_off, row_idx = precompute_neighborhood_s2(in_shape, out_shape, grid_in=grid_in, grid_out=grid_out, theta_cutoff=self.theta_cutoff)
        self.register_buffer("psi_row_idx", row_idx, persistent=False)
        self.register_buffer("psi_col_idx", col_idx, persistent=False)
        self.register_buffer("psi_roff_idx", row_off, persistent=False)
        # The kernels consume psi as a run-length plan (include/s2attn.h).  It is built here, on the host, from the CSR that was
        # just computed, and travels with the module as one more buffer, so no forward ever copies psi back from the device
        # (the reference re-sorts the CSR rows on the device in every call, attention_cuda_utils.cu:74-113).
        # The blob is also kept on disk, keyed by what determines psi (see plan.cached_host_blob), so later processes skip the build.
        psi_key = ("NeighborhoodAttentionS2", tuple(in_shape), tuple(out_shape), grid_in, grid_out, float(self.theta_cutoff).hex(), bool(self.upsample))
        plan = cached_host_blob(psi_key, col_idx, row_off, self.nlat_in, self.nlon_in, self.nlat_out, self.nlon_out)
        self.register_buffer("psi_plan", plan.blob, persistent=False)
        self._psi_plan_header = list(plan.header)

        # projections are 1x1; stored in convolution shape, drawn in the order q, k, v, proj
        bound_qk = math.sqrt(6.0 / (self.in_channels + self.k_channels))
        bound_v = math.sqrt(6.0 / (self.in_channels + self.out_channels))
        bound_proj = math.sqrt(3.0 / self.out_channels)
        self.q_weights = _xavier_uniform(self.k_channels, self.in_channels, bound_qk)
        self.k_weights = _xavier_uniform(self.k_channels, self.in_channels, bound_qk)
        self.v_weights = _xavier_uniform(self.out_channels, self.in_channels, bound_v)
        self.proj_weights = _xavier_uniform(self.out_channels, self.out_channels, bound_proj)

        self.scale = scale if scale is not None else 1 / math.sqrt(self.k_channels // self.num_heads)

        if bias:
            self.q_bias = nn.Parameter(torch.zeros(self.k_channels))
            self.k_bias = nn.Parameter(torch.zeros(self.k_channels))
            self.v_bias = nn.Parameter(torch.zeros(self.out_channels))
            self.proj_bias = nn.Parameter(torch.zeros(self.out_channels))
        else:
            self.q_bias = self.k_bias = self.v_bias = self.proj_bias = None

        if use_qknorm:
            self.q_norm_weights = nn.Parameter(torch.zeros(self.k_channels // self.num_heads))
            self.k_norm_weights = nn.Parameter(torch.zeros(self.k_channels // self.num_heads))
        else:
            self.q_norm_weights = self.k_norm_weights = None

        self.attention_handle = neighborhood_s2_attention

    def extra_repr(self):
        return (
            f"in_shape={(self.nlat_in, self.nlon_in)}, out_shape={(self.nlat_out, self.nlon_out)}, in_channels={self.in_channels}, "
            f"out_channels={self.out_channels}, k_channels={self.k_channels}, theta_cutoff={self.theta_cutoff}"
        )

    def _head_rms_norm(self, x: torch.Tensor, gain: torch.Tensor, scale=None) -> torch.Tensor:
        B, H, W, C = x.shape
        x = x.reshape(B, H, W, self.num_heads, -1)
        x = F.rms_norm(x, normalized_shape=gain.shape, weight=1 + gain if scale is None else (1 + gain) * scale)
        return x.reshape(B, H, W, C)

    def forward(self, query: torch.Tensor, key: Optional[torch.Tensor] = None, value: Optional[torch.Tensor] = None) -> torch.Tensor:
        """
        query : (B, in_channels, nlat_out, nlon_out); key, value : (B, in_channels, nlat_in, nlon_in), both
        default to ``query`` (self-attention).  Returns (B, out_channels, nlat_out, nlon_out).
        """
        if key is None:
            key = query
        if value is None:
            value = query

        _check_ndim(query, 4, "query")
        _check_ndim(key, 4, "key")
        _check_ndim(value, 4, "value")
        _check_dtypes_match((query, key, value))
        _check_extent(query, -2, self.nlat_out, "query latitudes")
        _check_extent(query, -1, self.nlon_out, "query longitudes")
        _check_extent(key, -2, self.nlat_in, "key latitudes")
        _check_extent(key, -1, self.nlon_in, "key longitudes")
        _check_extent(value, -2, self.nlat_in, "value latitudes")
        _check_extent(value, -1, self.nlon_in, "value longitudes")

        key_is_query, value_is_query, value_is_key = key is query, value is query, value is key
        # the softmax scale rides on the q projection (or on the q gain when the q/k RMS norm is on): no pass of its own
        normed = self.q_norm_weights is not None
        wq = self.q_weights.view(self.q_weights.shape[0], -1)
        bq = self.q_bias
        if not normed:
            wq, bq = wq * self.scale, None if bq is None else bq * self.scale
        wk, wv = self.k_weights.view(self.k_weights.shape[0], -1), self.v_weights.view(self.v_weights.shape[0], -1)
        # Projections that share their input: one fused GEMM whose output the attention kernels read in place (q | k | v as
        # column blocks of one buffer) where the kernels of this shape take such tensors; else one F.linear each with a shared
        # backward that accumulates the input gradient inside the GEMMs.
        fused = (
            not normed
            and not torch.is_autocast_enabled()
            and takes_column_blocks(query.dtype, self.k_channels // self.num_heads, self.out_channels // self.num_heads, self.nlon_in, self.nlon_out)
            and self.k_channels % 4 == 0
            and self.out_channels % 4 == 0
        )
        # The fused projection, and the output projection, read / write the module's NCHW tensors as transposed GEMM operands
        # (no channels-last copy of the input, no channels-first copy of the output) for fp32 tensors outside autocast.
        direct = not torch.is_autocast_enabled() and query.dtype == torch.float32 and query.shape[0] <= _MAX_NCHW_BATCH
        if fused and direct and all(t.is_contiguous() for t in (query, key, value)):
            if key_is_query and value_is_query:
                query, key, value = _FusedLinear1x1NCHW.apply(query, wq, bq, wk, self.k_bias, wv, self.v_bias)
            else:
                (query,) = _FusedLinear1x1NCHW.apply(query, wq, bq)
                if value_is_key:
                    key, value = _FusedLinear1x1NCHW.apply(key, wk, self.k_bias, wv, self.v_bias)
                else:
                    (key,) = _FusedLinear1x1NCHW.apply(key, wk, self.k_bias)
                    (value,) = _FusedLinear1x1NCHW.apply(value, wv, self.v_bias)
            return self._attend_and_project(query, key, value, normed, direct)

        # one channels-last conversion per distinct input tensor; everything after is NHWC
        query = to_nhwc(query)
        key = query if key_is_query else to_nhwc(key)
        value = query if value_is_query else (key if value_is_key else to_nhwc(value))
        shared = _FusedLinear1x1 if fused else _SharedInputLinear1x1
        if key_is_query and value_is_query:
            query, key, value = shared.apply(query, wq, bq, wk, self.k_bias, wv, self.v_bias)
        else:
            query = _Linear1x1.apply(query, wq, bq)
            if value_is_key:
                key, value = shared.apply(key, wk, self.k_bias, wv, self.v_bias)
            else:
                key = _Linear1x1.apply(key, wk, self.k_bias)
                value = _Linear1x1.apply(value, wv, self.v_bias)

        return self._attend_and_project(query, key, value, normed, direct)

    def _attend_and_project(self, query, key, value, normed: bool, direct: bool) -> torch.Tensor:
        """NHWC q, k, v -> the module's NCHW output."""
        if normed:
            query = self._head_rms_norm(query, self.q_norm_weights, self.scale)
            key = self._head_rms_norm(key, self.k_norm_weights)

        out = self.attention_handle(
            key, value, query, self.quad_weights, self.psi_col_idx, self.psi_roff_idx, self.num_heads, self.nlon_in, self.nlat_out, self.nlon_out,
            self.psi_plan, self._psi_plan_header,
        )  # fmt: skip

        wp = self.proj_weights.view(self.proj_weights.shape[0], -1)
        if direct and out.dtype == torch.float32 and out.is_contiguous():
            return _Linear1x1ToNCHW.apply(out, wp, self.proj_bias)
        return to_nchw(_Linear1x1.apply(out, wp, self.proj_bias))
