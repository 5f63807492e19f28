"""
CPU restatement of the reference's ring-step kernels (generic variants, gather direction first, the up-sampling direction at
the end of the file): one longitude chunk of K/V per call, softmax state in caller-owned buffers that are updated in place.

TEST INFRASTRUCTURE ONLY: the shipped package must never import this module.

The reference has no CPU implementation of these operators (its distributed layer is CUDA-only,
tests/test_distributed_attention.py:84-92), so this file restates the CUDA kernels' arithmetic entry by entry.
Parity pins (tests/test_oracle_ring.py): folding every chunk of a partition of the input grid into fresh state reproduces the
dense float64 softmax attention and its autograd gradients, for any partition, halo and local output window -- a dropped
rescaling, a wrong chunk test or a wrong index shift breaks that identity.

Layout (heads folded into the batch, NHWC): kx, vx [B, nlat_halo, nlon_kx, C]; qy, dy [B, nlat_out, nlon_out, C];
state y_acc [B, nlat_out, nlon_out, Cv], alpha_sum / qdotk_max / integral [B, nlat_out, nlon_out], alpha_k / alpha_kvw
[B, nlat_out, nlon_out, Ck].  col_idx = hi_global * nlon_in + wi, wi already shifted by pscale * (first local output
longitude).  Everything is computed in the dtype of the state tensors (float64 in the tests).
"""

import torch


def _entries(col_idx, row_off, ho, nlon_in, pscale, lon_lo_kx, nlon_kx, lat_halo_start, nlat_halo, nlon_out):
    """For output latitude ho: yields (hi_global, hi_local, sel, wl) per CSR entry that touches the chunk; sel is the mask of
    local output longitudes whose neighbor (hi, (wi + pscale * wo) mod nlon_in) lies in the chunk, wl its chunk-local
    longitudes (attention_cuda_fwd_ring.cu:132-148)."""
    wo = torch.arange(nlon_out)
    for z in range(int(row_off[ho]), int(row_off[ho + 1])):
        col = int(col_idx[z])
        hi = col // nlon_in
        wi = col - hi * nlon_in
        hl = hi - lat_halo_start
        if hl < 0 or hl >= nlat_halo:
            continue
        wip = (wi + pscale * wo) % nlon_in
        sel = (wip >= lon_lo_kx) & (wip < lon_lo_kx + nlon_kx)
        if bool(sel.any()):
            yield hi, hl, sel, (wip - lon_lo_kx)[sel]


def forward_step(kx, vx, qy, y_acc, alpha_sum, qdotk_max, quad_weights, col_idx, row_off, nlon_in, pscale, lon_lo_kx, lat_halo_start):
    """attention_cuda_fwd_ring.cu:66-175: online softmax update of (y_acc, alpha_sum, qdotk_max) with the chunk's neighbors."""
    _, nlat_halo, nlon_kx, _ = kx.shape
    _, nlat_out, nlon_out, _ = qy.shape
    dt = y_acc.dtype
    for ho in range(nlat_out):
        for hi, hl, sel, wl in _entries(col_idx, row_off, ho, nlon_in, pscale, lon_lo_kx, nlon_kx, lat_halo_start, nlat_halo, nlon_out):
            k, v, q = kx[:, hl, wl, :].to(dt), vx[:, hl, wl, :].to(dt), qy[:, ho, sel, :].to(dt)
            s = (q * k).sum(-1)
            m_old = qdotk_max[:, ho, sel]
            m_new = torch.maximum(m_old, s)
            alpha = torch.exp(s - m_new) * float(quad_weights[hi])
            corr = torch.exp(m_old - m_new)
            alpha_sum[:, ho, sel] = alpha + alpha_sum[:, ho, sel] * corr
            y_acc[:, ho, sel, :] = y_acc[:, ho, sel, :] * corr[..., None] + alpha[..., None] * v
            qdotk_max[:, ho, sel] = m_new


def backward_pass1(kx, vx, qy, dy, alpha_sum, qdotk_max, integral, alpha_k, alpha_kvw, quad_weights, col_idx, row_off, nlon_in, pscale, lon_lo_kx, lat_halo_start):
    """attention_cuda_bwd_ring.cu:78-205: the same online update for alpha_sum, integral = sum alpha <dy, v>,
    alpha_k = sum alpha k, alpha_kvw = sum alpha <dy, v> k."""
    _, nlat_halo, nlon_kx, _ = kx.shape
    _, nlat_out, nlon_out, _ = qy.shape
    dt = alpha_sum.dtype
    for ho in range(nlat_out):
        for hi, hl, sel, wl in _entries(col_idx, row_off, ho, nlon_in, pscale, lon_lo_kx, nlon_kx, lat_halo_start, nlat_halo, nlon_out):
            k, v, q, g = kx[:, hl, wl, :].to(dt), vx[:, hl, wl, :].to(dt), qy[:, ho, sel, :].to(dt), dy[:, ho, sel, :].to(dt)
            s = (q * k).sum(-1)
            gv = (g * v).sum(-1)
            m_old = qdotk_max[:, ho, sel]
            m_new = torch.maximum(m_old, s)
            alpha = torch.exp(s - m_new) * float(quad_weights[hi])
            corr = torch.exp(m_old - m_new)
            alpha_sum[:, ho, sel] = alpha_sum[:, ho, sel] * corr + alpha
            integral[:, ho, sel] = integral[:, ho, sel] * corr + alpha * gv
            alpha_k[:, ho, sel, :] = alpha_k[:, ho, sel, :] * corr[..., None] + alpha[..., None] * k
            alpha_kvw[:, ho, sel, :] = alpha_kvw[:, ho, sel, :] * corr[..., None] + (alpha * gv)[..., None] * k
            qdotk_max[:, ho, sel] = m_new


def backward_pass2(kx, vx, qy, dy, alpha_sum, qdotk_max, integral_norm, dkx, dvx, quad_weights, col_idx, row_off, nlon_in, pscale, lon_lo_kx, lat_halo_start):
    """attention_cuda_bwd_ring.cu:1312-1440: with the final statistics, dkx += p (<dy, v> - integral_norm) q and
    dvx += p dy for the chunk's points, p = exp(q.k - qdotk_max) w / alpha_sum."""
    _, nlat_halo, nlon_kx, _ = kx.shape
    _, nlat_out, nlon_out, _ = qy.shape
    dt = dkx.dtype
    for ho in range(nlat_out):
        for hi, hl, sel, wl in _entries(col_idx, row_off, ho, nlon_in, pscale, lon_lo_kx, nlon_kx, lat_halo_start, nlat_halo, nlon_out):
            k, v, q, g = kx[:, hl, wl, :].to(dt), vx[:, hl, wl, :].to(dt), qy[:, ho, sel, :].to(dt), dy[:, ho, sel, :].to(dt)
            s = (q * k).sum(-1)
            gv = (g * v).sum(-1)
            p = torch.exp(s - qdotk_max[:, ho, sel]) * float(quad_weights[hi]) / alpha_sum[:, ho, sel]
            # several output longitudes may map to one input point only through different entries, never inside one entry
            # (wl is injective in wo for pscale >= 1), so plain indexed adds are exact here
            dkx[:, hl, wl, :] += ((gv - integral_norm[:, ho, sel]) * p)[..., None] * q
            dvx[:, hl, wl, :] += p[..., None] * g


def split_csr_rows(row_idx, row_off, nlat_out, thres=0.1, split_len=1024):
    """attention_cuda_utils.cu:352-379 (host path): rows listed by decreasing length; long rows are the leading ones of at
    least max(split_len, int(float32(longest) * thres)) entries."""
    if nlat_out == 0:
        return 0, 0, 0
    lens = [int(row_off[int(r) + 1]) - int(row_off[int(r)]) for r in row_idx[:nlat_out]]
    max_rlen = lens[0]
    thres_len = int(float(torch.tensor(float(max_rlen), dtype=torch.float32) * torch.tensor(thres, dtype=torch.float32)))
    min_long = max(split_len, thres_len)
    n_long = 0
    for n in lens:
        if n >= min_long:
            n_long += 1
        else:
            break
    return n_long, (max_rlen if n_long else 0), (lens[n_long] if n_long < nlat_out else 0)


# ---- up-sampling (scatter) direction --------------------------------------------------------------------------------
# psi keyed by the chunk's local input latitude; col_idx = ho_local * nlon_out_global + wo_shifted,
# wo_shifted = (wo - first local output longitude) mod nlon_out_global.  Pinned like the gather direction: chunks fold to
# the dense float64 attention over the scatter-direction mask (tests/test_oracle_ring.py).
def _up_entries(col_idx, row_off, hi, nlon_kx, lon_lo_kx, nlon_out_global, pscale_out, nlon_out):
    """For the chunk's input latitude hi: yields (ho_local, sel, w) per CSR entry; sel masks the chunk's input longitudes
    whose target cell (ho_local, w = (wo_shifted + pscale_out * wi_global) mod nlon_out_global) is local, w their local
    output longitudes (attention_cuda_fwd_ring_upsample.cu:93-101)."""
    wi_global = lon_lo_kx + torch.arange(nlon_kx)
    for z in range(int(row_off[hi]), int(row_off[hi + 1])):
        col = int(col_idx[z])
        ho = col // nlon_out_global
        w = (col - ho * nlon_out_global + pscale_out * wi_global) % nlon_out_global
        sel = w < nlon_out
        if bool(sel.any()):
            yield ho, sel, w[sel]


def forward_step_upsample(kx, vx, qy, y_acc, alpha_sum, qdotk_max, quad_weights, col_idx, row_off, nlon_out_global, pscale_out, lon_lo_kx, lat_halo_start):
    """attention_cuda_fwd_ring_upsample.cu:108-300: (1) the chunk's maxima per local output cell, (2) rescale the state of
    the cells whose maximum moved, (3) add exp(q.k - max) w and that times v."""
    B, nlat_halo, nlon_kx, _ = kx.shape
    _, nlat_out, nlon_out, _ = qy.shape
    dt = y_acc.dtype
    m_new = qdotk_max.clone()
    for phase in ("max", "acc"):
        if phase == "acc":
            moved = m_new != qdotk_max
            corr = torch.where(moved, torch.exp(qdotk_max - m_new), torch.ones_like(m_new))
            y_acc *= corr[..., None]
            alpha_sum *= corr
            qdotk_max.copy_(m_new)
        for hi in range(nlat_halo):
            for ho, sel, w in _up_entries(col_idx, row_off, hi, nlon_kx, lon_lo_kx, nlon_out_global, pscale_out, nlon_out):
                k, q = kx[:, hi, sel, :].to(dt), qy[:, ho, w, :].to(dt)
                s = (q * k).sum(-1)
                if phase == "max":
                    m_new[:, ho, w] = torch.maximum(m_new[:, ho, w], s)  # w is injective in the chunk longitude: no duplicates
                else:
                    alpha = torch.exp(s - qdotk_max[:, ho, w]) * float(quad_weights[lat_halo_start + hi])
                    alpha_sum[:, ho, w] += alpha
                    y_acc[:, ho, w, :] += alpha[..., None] * vx[:, hi, sel, :].to(dt)


def backward_pass1_upsample(kx, vx, qy, dy, qdotk_max, integral, alpha_k, alpha_kvw, quad_weights, col_idx, row_off, nlon_out_global, pscale_out, lon_lo_kx, lat_halo_start):
    """attention_cuda_bwd_ring_upsample.cu:88-160: with the forward's final maximum, integral += alpha <dy, v>,
    alpha_k += alpha k, alpha_kvw += alpha <dy, v> k."""
    _, nlat_halo, nlon_kx, _ = kx.shape
    nlon_out = qy.shape[2]
    dt = integral.dtype
    for hi in range(nlat_halo):
        for ho, sel, w in _up_entries(col_idx, row_off, hi, nlon_kx, lon_lo_kx, nlon_out_global, pscale_out, nlon_out):
            k, v, q, g = kx[:, hi, sel, :].to(dt), vx[:, hi, sel, :].to(dt), qy[:, ho, w, :].to(dt), dy[:, ho, w, :].to(dt)
            alpha = torch.exp((q * k).sum(-1) - qdotk_max[:, ho, w]) * float(quad_weights[lat_halo_start + hi])
            ag = alpha * (g * v).sum(-1)
            integral[:, ho, w] += ag
            alpha_k[:, ho, w, :] += alpha[..., None] * k
            alpha_kvw[:, ho, w, :] += ag[..., None] * k


def backward_pass2_upsample(kx, vx, qy, dy, alpha_sum, qdotk_max, integral_norm, dkx, dvx, quad_weights, col_idx, row_off, nlon_out_global, pscale_out, lon_lo_kx, lat_halo_start):
    """attention_cuda_bwd_ring_upsample.cu:162-240: dkx, dvx of every chunk cell are WRITTEN: sums over the cell's own row of
    p (<dy, v> - integral_norm) q and p dy, p = exp(q.k - max) w / alpha_sum."""
    _, nlat_halo, nlon_kx, _ = kx.shape
    nlon_out = qy.shape[2]
    dt = dkx.dtype
    dkx.zero_()
    dvx.zero_()
    for hi in range(nlat_halo):
        for ho, sel, w in _up_entries(col_idx, row_off, hi, nlon_kx, lon_lo_kx, nlon_out_global, pscale_out, nlon_out):
            k, v, q, g = kx[:, hi, sel, :].to(dt), vx[:, hi, sel, :].to(dt), qy[:, ho, w, :].to(dt), dy[:, ho, w, :].to(dt)
            p = torch.exp((q * k).sum(-1) - qdotk_max[:, ho, w]) * float(quad_weights[lat_halo_start + hi]) / alpha_sum[:, ho, w]
            dkx[:, hi, sel, :] += (((g * v).sum(-1) - integral_norm[:, ho, w]) * p)[..., None] * q
            dvx[:, hi, sel, :] += p[..., None] * g
