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


# gather direction on grids with at least 32 global output longitudes: with fp32 storage and ck == cv a multiple of 4 from 16 to
# 128 the forward step runs on the band-staged matrix-core kernel (s2attn_ring_forward_step_plan)
RING_BAND_CASES = [
    ((9, 48), (9, 48), "equiangular", "equiangular", 0.5, (0, 9, 7, 30), [0, 10, 11, 37, 48]),  # self-attention, a one-column chunk, pole rows see whole circles
    ((8, 96), (6, 48), "equiangular", "legendre-gauss", 0.6, (1, 4, 9, 33), [0, 40, 96]),  # longitude ratio 2, ragged last tile
    ((7, 120), (5, 40), "legendre-gauss", "equiangular", 0.7, (0, 5, 0, 40), [0, 31, 32, 90, 120]),  # ratio 3, the whole output grid is local
    ((6, 40), (6, 40), "equiangular", "equiangular", 7.0, (1, 3, 35, 5), [0, 20, 40]),  # every point sees every point, a window of five columns
    ((12, 80), (12, 80), "legendre-gauss", "legendre-gauss", 0.2, (0, 12, 16, 64), [0, 20, 40, 60, 80]),  # short runs only: most tiles touch one chunk
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


# up-sampling direction: (in_shape, out_shape, grid_in, grid_out, theta_cutoff, local output window, chunk boundaries, halo pad)
RING_UP_CASES = [
    ((6, 8), (6, 16), "equiangular", "equiangular", 0.9, (0, 6, 0, 16), [0, 8], 0),  # one chunk, whole grid
    ((6, 8), (11, 16), "equiangular", "equiangular", 0.8, (2, 6, 5, 7), [0, 3, 8], 0),  # ratio 2, unequal chunks
    ((5, 6), (9, 18), "legendre-gauss", "equiangular", 0.9, (0, 9, 12, 6), [0, 1, 4, 6], 1),  # ratio 3, halo padded past the poles
    ((6, 12), (12, 24), "equiangular", "legendre-gauss", 7.0, (3, 5, 20, 4), [0, 6, 12], 0),  # every point sees every point
]


# up-sampling direction on grids with at least 32 input longitudes: with ck == cv a multiple of 4 from 16 to 128
# the three steps run on the band-staged matrix-core kernels
RING_UP_BAND_CASES = [
    ((6, 40), (11, 80), "equiangular", "equiangular", 0.6, (2, 6, 9, 50), [0, 13, 14, 40], 0),  # ratio 2, a one-column chunk, odd window
    ((5, 32), (9, 96), "legendre-gauss", "equiangular", 0.7, (0, 9, 80, 16), [0, 16, 32], 1),  # ratio 3, halo padded past the poles
    ((7, 48), (13, 96), "equiangular", "legendre-gauss", 0.25, (0, 13, 0, 96), [0, 12, 24, 36, 48], 0),  # short runs, the whole output grid local
    ((6, 36), (6, 72), "equiangular", "equiangular", 7.0, (1, 4, 60, 7), [0, 18, 36], 0),  # every point sees every point, a seven-column window
]


def local_problem_upsample(case, batch=2, ck=5, cv=3, seed=0):
    """Global tensors plus one rank's local view in the scatter direction (psi keyed by input latitude): rows = the halo's input
    latitudes (pad rows past the poles are empty), entries restricted to the local output latitudes and re-based, output
    longitude shifted by the window's first longitude (torch_harmonics/distributed/distributed_attention.py, _build_local_psi_upsample)."""
    ins, outs, gi, go, tc, (lat_lo, nlat_loc, lon_lo, nlon_loc), bounds, pad = case
    (Hi, Wi), (Ho, Wo) = ins, outs
    col, roff = ogeo.neighborhood_csr(outs, ins, go, gi, tc)  # grids swapped: rows index the input grid
    quad = ogeo.attention_quad_weights(Hi, Wi, gi)
    pscale_out = Wo // Wi
    gen = torch.Generator().manual_seed(2000 + seed)
    k = torch.randn(batch, Hi, Wi, ck, generator=gen)
    v = torch.randn(batch, Hi, Wi, cv, generator=gen)
    q = torch.randn(batch, Ho, Wo, ck, generator=gen) / ck**0.5
    dy = torch.randn(batch, Ho, Wo, cv, generator=gen)
    # input latitudes that reach the local output rows, padded by `pad` rows on both sides (possibly past the poles)
    ho_all = col // Wo
    row_of = torch.repeat_interleave(torch.arange(Hi), roff[1:] - roff[:-1])
    keep = (ho_all >= lat_lo) & (ho_all < lat_lo + nlat_loc)
    used = row_of[keep]
    h0, h1 = (int(used.min()) - pad, int(used.max()) + 1 + pad) if used.numel() else (0, 1)
    rows, offs = [], [0]
    for hg in range(h0, h1):
        if 0 <= hg < Hi:
            e = col[int(roff[hg]) : int(roff[hg + 1])]
            ho = e // Wo
            sel = (ho >= lat_lo) & (ho < lat_lo + nlat_loc)
            e, ho = e[sel], ho[sel]
            rows.append((ho - lat_lo) * Wo + (e - ho * Wo - lon_lo) % Wo)
        offs.append(offs[-1] + (rows[-1].numel() if 0 <= hg < Hi else 0))
    col_l = torch.cat(rows) if rows else torch.zeros(0, dtype=torch.int64)
    roff_l = torch.tensor(offs, dtype=torch.int64)

    def halo_block(t, lo, hi):  # rows h0..h1 of the chunk's longitudes, zeros where the halo leaves the grid
        out = torch.zeros(t.shape[0], h1 - h0, hi - lo, t.shape[3], dtype=t.dtype)
        a, b = max(h0, 0), min(h1, Hi)
        out[:, a - h0 : b - h0] = t[:, a:b, lo:hi]
        return out

    return dict(
        ins=ins, outs=outs, pscale_out=pscale_out, quad=quad, col=col, roff=roff, k=k, v=v, q=q, dy=dy, col_l=col_l, roff_l=roff_l,
        lat_lo=lat_lo, nlat_loc=nlat_loc, lon_lo=lon_lo, nlon_loc=nlon_loc, halo=(h0, h1), halo_block=halo_block,
        chunks=[(bounds[i], bounds[i + 1]) for i in range(len(bounds) - 1)],
        q_l=q[:, lat_lo : lat_lo + nlat_loc, lon_lo : lon_lo + nlon_loc].contiguous(),
        dy_l=dy[:, lat_lo : lat_lo + nlat_loc, lon_lo : lon_lo + nlon_loc].contiguous(),
    )  # fmt: skip
