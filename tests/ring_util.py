"""Shared by the CPU and GPU ring-step tests: a rank's local view of a global problem, the way a longitude/latitude-sharded
layer builds it (torch_harmonics/distributed/distributed_attention.py:963-1006), and the chunk loop around the operators."""

import torch

from oracle import geometry as ogeo

# (in_shape, out_shape, grid_in, grid_out, theta_cutoff, local output window (lat_lo, nlat, lon_lo, nlon), chunk boundaries)
RING_CASES = [
    ((7, 16), (7, 16), "equiangular", "equiangular", 0.9, (0, 7, 0, 16), [0, 16]),  # one chunk, whole grid
    ((7, 16), (7, 16), "equiangular", "equiangular", 0.9, (2, 4, 5, 7), [0, 3, 9, 16]),  # self-attention, unequal chunks
    ((8, 24), (6, 12), "equiangular", "legendre-gauss", 0.8, (1, 4, 4, 6), [0, 5, 16, 24]),  # longitude ratio 2
    ((9, 24), (5, 8), "legendre-gauss", "equiangular", 0.7, (0, 5, 2, 5), [0, 12, 13, 24]),  # ratio 3, a one-column chunk
    ((6, 12), (6, 12), "equiangular", "equiangular", 7.0, (1, 3, 10, 2), [0, 6, 12]),  # every point sees every point
]


def local_problem(case, batch=2, ck=5, cv=3, seed=0, tight_halo=True):
    """Global tensors plus the local CSR / window / halo of one rank.  Returns a dict."""
    ins, outs, gi, go, tc, (lat_lo, nlat_loc, lon_lo, nlon_loc), bounds = case
    (Hi, Wi), (Ho, Wo) = ins, outs
    col, roff = ogeo.neighborhood_csr(ins, outs, gi, go, tc)
    quad = ogeo.attention_quad_weights(Hi, Wi, gi)
    pscale = Wi // Wo
    gen = torch.Generator().manual_seed(1000 + seed)
    k = torch.randn(batch, Hi, Wi, ck, generator=gen)
    v = torch.randn(batch, Hi, Wi, cv, generator=gen)
    q = torch.randn(batch, Ho, Wo, ck, generator=gen) / ck**0.5
    dy = torch.randn(batch, Ho, Wo, cv, generator=gen)
    # local CSR: rows lat_lo .. lat_lo + nlat_loc, wi shifted by pscale * lon_lo
    start, end = int(roff[lat_lo]), int(roff[lat_lo + nlat_loc])
    roff_l = (roff[lat_lo : lat_lo + nlat_loc + 1] - roff[lat_lo]).contiguous()
    col_l = col[start:end].clone()
    hi = col_l // Wi
    col_l = hi * Wi + (col_l - hi * Wi + pscale * lon_lo) % Wi
    nnz_row = roff_l[1:] - roff_l[:-1]
    row_idx = torch.argsort(nnz_row, descending=True, stable=True).to(torch.int32)
    # latitude halo: exactly the input latitudes the local rows touch (or the whole grid)
    if tight_halo and hi.numel():
        h0, h1 = int(hi.min()), int(hi.max()) + 1
    else:
        h0, h1 = 0, Hi
    return dict(
        ins=ins, outs=outs, pscale=pscale, quad=quad, col=col, roff=roff, k=k, v=v, q=q, dy=dy,
        col_l=col_l, roff_l=roff_l, row_idx=row_idx, lat_lo=lat_lo, nlat_loc=nlat_loc, lon_lo=lon_lo, nlon_loc=nlon_loc,
        halo=(h0, h1), chunks=[(bounds[i], bounds[i + 1]) for i in range(len(bounds) - 1)],
        q_l=q[:, lat_lo : lat_lo + nlat_loc, lon_lo : lon_lo + nlon_loc].contiguous(),
        dy_l=dy[:, lat_lo : lat_lo + nlat_loc, lon_lo : lon_lo + nlon_loc].contiguous(),
    )  # fmt: skip


def chunk_of(p, tensor, c):
    """The (halo latitudes, chunk longitudes) block of a global input-grid tensor."""
    (h0, h1), (lo, hi) = p["halo"], p["chunks"][c]
    return tensor[:, h0:h1, lo:hi].contiguous()


def fresh_state(batch, nlat, nlon, ck, cv, dtype, device="cpu"):
    z = lambda *s: torch.zeros(*s, dtype=dtype, device=device)  # noqa: E731
    return dict(
        y_acc=z(batch, nlat, nlon, cv), alpha_sum=z(batch, nlat, nlon), qdotk_max=torch.full((batch, nlat, nlon), float("-inf"), dtype=dtype, device=device),
        integral=z(batch, nlat, nlon), alpha_k=z(batch, nlat, nlon, ck), alpha_kvw=z(batch, nlat, nlon, ck),
    )  # fmt: skip
