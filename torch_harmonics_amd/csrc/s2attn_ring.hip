// Ring-step variants of the gather direction: one longitude chunk of K/V at a time, softmax state kept by the caller.
//
// These are the building blocks of a longitude-sharded layer (K/V chunks travel around a ring of devices while q and
// the per-point state stay put; torch_harmonics/distributed/distributed_attention.py:141-176, 303-431).  Nothing here
// talks to another device: each call folds ONE chunk into the state (forward, backward pass 1) or produces that chunk's
// dk/dv (backward pass 2).  They walk the CSR directly -- membership of a neighbor in the current chunk is a test per
// entry, as in the reference's generic kernels (attention_cuda_fwd_ring.cu:66-175, attention_cuda_bwd_ring.cu:78-205,
// 1312-1440) -- and are written for correctness, one wavefront per output point, not tuned like the single-device path.
//
// Conventions (the reference's): heads are folded into the batch; state is fp32 in the natural-exponential domain
// (qdotk_max = running max of q.k, alpha_sum = sum of exp(q.k - max) * w, y_acc = the same sum weighted with v);
// col_idx = hi_global * nlon_in + wi with wi already shifted by pscale * (first local output longitude); a neighbor
// (hi_global, wip = (wi + pscale * wo_local) mod nlon_in) is used iff lon_lo_kx <= wip < lon_lo_kx + nlon_kx and
// 0 <= hi_global - lat_halo_start < nlat_halo.

#include "s2attn_internal.h"

#include <hip/hip_bf16.h>
#include <hip/hip_fp16.h>
#include <hip/hip_runtime.h>

#include <cstdint>

namespace s2ring {

constexpr int MAXC = 512;      // channels per (folded) head
constexpr int NCI = MAXC / 64; // channels per lane (up-sampling kernels: one wavefront per chunk cell)

struct Args {
    const void *k, *v, *q, *dy;
    float *y_acc, *alpha_sum, *qdotk_max, *integral, *alpha_k, *alpha_kvw; // state (read-only in pass 2 where they are inputs)
    const float *integral_norm;
    float *dk, *dv;
    const float *quad_w;
    const int64_t *col_idx, *row_off;
    const int32_t *row_idx; // launch order of the output latitudes (may be null: natural order)
    const int64_t *t_off;   // transposed neighborhood (pass 2): entries of halo latitude r are t_off[r] .. t_off[r + 1]
    const int32_t *t_ho, *t_dlon;
    int B, nlat_halo, nlon_kx, Ho, Wo, ck, cv, nlon_in, pscale, lon_lo_kx, lat_halo_start;
};

template <typename T> __device__ inline float ld(const T *p);
template <> __device__ inline float ld<float>(const float *p) { return *p; }
template <> __device__ inline float ld<__hip_bfloat16>(const __hip_bfloat16 *p) { return __bfloat162float(*p); }
template <> __device__ inline float ld<__half>(const __half *p) { return __half2float(*p); }

__device__ inline float wave_sum(float x)
{
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) x += __shfl_xor(x, o);
    return x;
}

// ---------------------------------------------------------------------------------------------------------------------
// Gather direction.  A wavefront owns P = 64 / G consecutive output longitudes of one (batch, output latitude); the G
// lanes of a point hold 8 consecutive channels each (G = 4 for up to 32 channels ... 64 for up to 512).  The wavefront
// reads the CSR row 64 entries at a time, one entry per lane: the split of col into (latitude, longitude), the halo test
// and a test whether ANY of the wavefront's points can see the entry in this chunk run once per entry in parallel; the
// surviving entries are then taken U at a time by all points together (every point at its own shifted longitude, so the
// P rows of K/V read for one entry are consecutive in memory), with U independent loads in flight per lane.
// ---------------------------------------------------------------------------------------------------------------------
constexpr int CPL = 8; // channels per lane

template <int G> __device__ inline float group_sum(float x)
{
#pragma unroll
    for (int o = G / 2; o > 0; o >>= 1) x += __shfl_xor(x, o);
    return x;
}

template <typename T> __device__ inline void unpack8(float (&x)[CPL], const T *p);
template <> __device__ inline void unpack8<float>(float (&x)[CPL], const float *p)
{
    const float4 lo = reinterpret_cast<const float4 *>(p)[0], hi = reinterpret_cast<const float4 *>(p)[1];
    x[0] = lo.x, x[1] = lo.y, x[2] = lo.z, x[3] = lo.w, x[4] = hi.x, x[5] = hi.y, x[6] = hi.z, x[7] = hi.w;
}
template <> __device__ inline void unpack8<__hip_bfloat16>(float (&x)[CPL], const __hip_bfloat16 *p)
{
    const uint4 r = *reinterpret_cast<const uint4 *>(p);
    const unsigned w[4] = {r.x, r.y, r.z, r.w};
#pragma unroll
    for (int i = 0; i < 4; i++) x[2 * i] = __uint_as_float(w[i] << 16), x[2 * i + 1] = __uint_as_float(w[i] & 0xffff0000u);
}
template <> __device__ inline void unpack8<__half>(float (&x)[CPL], const __half *p)
{
    const uint4 r = *reinterpret_cast<const uint4 *>(p);
    const unsigned w[4] = {r.x, r.y, r.z, r.w};
#pragma unroll
    for (int i = 0; i < 4; i++) {
        const __half2 h = *reinterpret_cast<const __half2 *>(&w[i]);
        x[2 * i] = __low2float(h), x[2 * i + 1] = __high2float(h);
    }
}

// channels c0 .. c0 + 7 of a row of n channels (zeros past the end); vec: n is a multiple of 8 and the row is 16-byte aligned
template <typename T> __device__ inline void load8(float (&x)[CPL], const T *row, int c0, int n, bool vec)
{
    if (vec) {
        if (c0 < n) {
            unpack8(x, row + c0);
        } else {
#pragma unroll
            for (int i = 0; i < CPL; i++) x[i] = 0.f;
        }
    } else {
#pragma unroll
        for (int i = 0; i < CPL; i++) x[i] = c0 + i < n ? ld(row + c0 + i) : 0.f;
    }
}

__device__ inline void store8(float *row, const float (&x)[CPL], int c0, int n, bool vec)
{
    if (vec) {
        if (c0 < n) {
            reinterpret_cast<float4 *>(row + c0)[0] = make_float4(x[0], x[1], x[2], x[3]);
            reinterpret_cast<float4 *>(row + c0)[1] = make_float4(x[4], x[5], x[6], x[7]);
        }
    } else {
#pragma unroll
        for (int i = 0; i < CPL; i++)
            if (c0 + i < n) row[c0 + i] = x[i];
    }
}

// The wavefront's place: batch b, output latitude ho, first output longitude wo0 of its P points; this lane's point wo
// (valid: inside the row) and first channel c0.  False past the end of the grid.
template <int G> struct Place {
    int b, ho, wo, c0, pw, pw0;
    bool valid;
    long out;
    __device__ inline bool locate(const Args &a)
    {
        constexpr int P = 64 / G;
        const int lane = threadIdx.x & 63;
        const long wid = (long)blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
        const int nb = (a.Wo + P - 1) / P;
        if (wid >= (long)a.B * a.Ho * nb) return false;
        const int wb = (int)(wid % nb);
        const int h = (int)((wid / nb) % a.Ho);
        b = (int)(wid / ((long)nb * a.Ho));
        ho = a.row_idx ? a.row_idx[h] : h;
        const int w = wb * P + lane / G;
        valid = w < a.Wo;
        wo = valid ? w : a.Wo - 1;
        c0 = (lane % G) * CPL;
        pw = (int)(((long)a.pscale * wo) % a.nlon_in);
        pw0 = (int)(((long)a.pscale * wb * P) % a.nlon_in);
        out = ((long)b * a.Ho + ho) * a.Wo + wo;
        return true;
    }
};

// One CSR entry per lane: (longitude wi, chunk row base, quadrature weight) and whether any point of the wavefront can see it.
template <int G> __device__ inline bool scan_entry(const Args &a, int64_t z, int64_t z1, int pw0, int &wi, int &rowbase, float &wq)
{
    constexpr int P = 64 / G;
    wi = 0, rowbase = 0, wq = 0.f;
    if (z >= z1) return false;
    const int64_t col = a.col_idx[z];
    int hi;
    if ((uint64_t)col < 0x80000000ull) {
        hi = (int)((uint32_t)col / (uint32_t)a.nlon_in);
        wi = (int)((uint32_t)col - (uint32_t)hi * (uint32_t)a.nlon_in);
    } else {
        hi = (int)(col / a.nlon_in);
        wi = (int)(col - (int64_t)hi * a.nlon_in);
    }
    const int hl = hi - a.lat_halo_start;
    if (hl < 0 || hl >= a.nlat_halo) return false;
    // first point's longitude relative to the chunk; the others follow at pscale apart, up to span further (cyclically)
    int u = wi + pw0 - a.lon_lo_kx;
    if (u < 0) u += a.nlon_in;
    if (u >= a.nlon_in) u -= a.nlon_in;
    const long span = (long)a.pscale * (P - 1);
    if (!(u < a.nlon_kx || u + span >= a.nlon_in)) return false;
    rowbase = hl * a.nlon_kx;
    wq = a.quad_w[hi];
    return true;
}

// chunk-local point of entry (wi, rowbase) for the lane's own output longitude, or -1
__device__ inline int own_point(const Args &a, int wi, int rowbase, int pw, bool valid)
{
    int wip = wi + pw;
    if (wip >= a.nlon_in) wip -= a.nlon_in;
    const int rel = wip - a.lon_lo_kx;
    return valid && (unsigned)rel < (unsigned)a.nlon_kx ? rowbase + rel : -1;
}

#define S2_RING_TAKE(u)                                                                                                  \
    {                                                                                                                    \
        const bool has = cand != 0;                                                                                      \
        const int j = has ? __builtin_ctzll(cand) : 0;                                                                   \
        cand &= cand - 1;                                                                                                \
        const int wj = __builtin_amdgcn_readlane(wi, j), rj = __builtin_amdgcn_readlane(rowbase, j);                     \
        wgt[u] = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(wq), j));                                       \
        pt[u] = has ? own_point(a, wj, rj, pl.pw, pl.valid) : -1;                                                        \
    }

// Forward: folds the chunk into (y_acc, alpha_sum, qdotk_max).  attention_cuda_fwd_ring.cu:66-175.
template <typename T, int G> __global__ __launch_bounds__(256) void fwd_kernel(const Args a, const bool vec)
{
    constexpr int U = 4;
    Place<G> pl;
    if (!pl.locate(a)) return;
    const int lane = threadIdx.x & 63;
    const T *__restrict__ kx = static_cast<const T *>(a.k) + (long)pl.b * a.nlat_halo * a.nlon_kx * a.ck;
    const T *__restrict__ vx = static_cast<const T *>(a.v) + (long)pl.b * a.nlat_halo * a.nlon_kx * a.cv;
    float qr[CPL], y[CPL];
    load8(qr, static_cast<const T *>(a.q) + pl.out * a.ck, pl.c0, a.ck, vec);
    load8(y, a.y_acc + pl.out * a.cv, pl.c0, a.cv, vec);
    float S = a.alpha_sum[pl.out], m = a.qdotk_max[pl.out];
    const int64_t z0 = a.row_off[pl.ho], z1 = a.row_off[pl.ho + 1];
    for (int64_t zb = z0; zb < z1; zb += 64) {
        int wi, rowbase;
        float wq;
        const bool ok = scan_entry<G>(a, zb + lane, z1, pl.pw0, wi, rowbase, wq);
        unsigned long long cand = __ballot(ok);
        while (cand) {
            int pt[U];
            float wgt[U], kk[U][CPL], vv[U][CPL], s[U];
#pragma unroll
            for (int u = 0; u < U; u++) S2_RING_TAKE(u)
#pragma unroll
            for (int u = 0; u < U; u++) {
                const long p = pt[u] < 0 ? 0 : pt[u];
                load8(kk[u], kx + p * a.ck, pl.c0, a.ck, vec);
                load8(vv[u], vx + p * a.cv, pl.c0, a.cv, vec);
            }
            float mn = m;
#pragma unroll
            for (int u = 0; u < U; u++) {
                float d = 0.f;
#pragma unroll
                for (int i = 0; i < CPL; i++) d = fmaf(qr[i], kk[u][i], d);
                s[u] = group_sum<G>(d);
                if (pt[u] >= 0) mn = fmaxf(mn, s[u]);
            }
            if (mn == -INFINITY) continue; // nothing seen yet, nothing in these entries (the condition is the same in a whole group)
            const float corr = __expf(m - mn); // m = -inf before the first neighbor: 0
            S *= corr;
#pragma unroll
            for (int i = 0; i < CPL; i++) y[i] *= corr;
#pragma unroll
            for (int u = 0; u < U; u++) {
                const float alpha = pt[u] >= 0 ? __expf(s[u] - mn) * wgt[u] : 0.f;
                S += alpha;
#pragma unroll
                for (int i = 0; i < CPL; i++) y[i] = fmaf(alpha, vv[u][i], y[i]);
            }
            m = mn;
        }
    }
    if (!pl.valid) return;
    if (pl.c0 == 0) {
        a.alpha_sum[pl.out] = S;
        a.qdotk_max[pl.out] = m;
    }
    store8(a.y_acc + pl.out * a.cv, y, pl.c0, a.cv, vec);
}

// Backward pass 1: folds the chunk into (alpha_sum, qdotk_max, integral = sum alpha <dy, v>, alpha_k = sum alpha k,
// alpha_kvw = sum alpha <dy, v> k).  attention_cuda_bwd_ring.cu:78-205.
template <typename T, int G> __global__ __launch_bounds__(256) void pass1_kernel(const Args a, const bool vec)
{
    constexpr int U = 2;
    Place<G> pl;
    if (!pl.locate(a)) return;
    const int lane = threadIdx.x & 63;
    const T *__restrict__ kx = static_cast<const T *>(a.k) + (long)pl.b * a.nlat_halo * a.nlon_kx * a.ck;
    const T *__restrict__ vx = static_cast<const T *>(a.v) + (long)pl.b * a.nlat_halo * a.nlon_kx * a.cv;
    float qr[CPL], gr[CPL], ak[CPL], akg[CPL];
    load8(qr, static_cast<const T *>(a.q) + pl.out * a.ck, pl.c0, a.ck, vec);
    load8(gr, static_cast<const T *>(a.dy) + pl.out * a.cv, pl.c0, a.cv, vec);
    load8(ak, a.alpha_k + pl.out * a.ck, pl.c0, a.ck, vec);
    load8(akg, a.alpha_kvw + pl.out * a.ck, pl.c0, a.ck, vec);
    float S = a.alpha_sum[pl.out], m = a.qdotk_max[pl.out], I = a.integral[pl.out];
    const int64_t z0 = a.row_off[pl.ho], z1 = a.row_off[pl.ho + 1];
    for (int64_t zb = z0; zb < z1; zb += 64) {
        int wi, rowbase;
        float wq;
        const bool ok = scan_entry<G>(a, zb + lane, z1, pl.pw0, wi, rowbase, wq);
        unsigned long long cand = __ballot(ok);
        while (cand) {
            int pt[U];
            float wgt[U], kk[U][CPL], vv[U][CPL], s[U], gv[U];
#pragma unroll
            for (int u = 0; u < U; u++) S2_RING_TAKE(u)
#pragma unroll
            for (int u = 0; u < U; u++) {
                const long p = pt[u] < 0 ? 0 : pt[u];
                load8(kk[u], kx + p * a.ck, pl.c0, a.ck, vec);
                load8(vv[u], vx + p * a.cv, pl.c0, a.cv, vec);
            }
            float mn = m;
#pragma unroll
            for (int u = 0; u < U; u++) {
                float d = 0.f, e = 0.f;
#pragma unroll
                for (int i = 0; i < CPL; i++) d = fmaf(qr[i], kk[u][i], d), e = fmaf(gr[i], vv[u][i], e);
                s[u] = group_sum<G>(d);
                gv[u] = group_sum<G>(e);
                if (pt[u] >= 0) mn = fmaxf(mn, s[u]);
            }
            if (mn == -INFINITY) continue;
            const float corr = __expf(m - mn);
            S *= corr, I *= corr;
#pragma unroll
            for (int i = 0; i < CPL; i++) ak[i] *= corr, akg[i] *= corr;
#pragma unroll
            for (int u = 0; u < U; u++) {
                const float alpha = pt[u] >= 0 ? __expf(s[u] - mn) * wgt[u] : 0.f;
                const float ag = alpha * gv[u];
                S += alpha, I += ag;
#pragma unroll
                for (int i = 0; i < CPL; i++) ak[i] = fmaf(alpha, kk[u][i], ak[i]), akg[i] = fmaf(ag, kk[u][i], akg[i]);
            }
            m = mn;
        }
    }
    if (!pl.valid) return;
    if (pl.c0 == 0) {
        a.alpha_sum[pl.out] = S;
        a.qdotk_max[pl.out] = m;
        a.integral[pl.out] = I;
    }
    store8(a.alpha_k + pl.out * a.ck, ak, pl.c0, a.ck, vec);
    store8(a.alpha_kvw + pl.out * a.ck, akg, pl.c0, a.ck, vec);
}

// output point of this wavefront; false past the end
__device__ inline bool locate(const Args &a, int &b, int &ho, int &wo, int &lane)
{
    lane = threadIdx.x & 63;
    const long pid = (long)blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
    if (pid >= (long)a.B * a.Ho * a.Wo) return false;
    wo = (int)(pid % a.Wo);
    const int h = (int)((pid / a.Wo) % a.Ho);
    b = (int)(pid / ((long)a.Wo * a.Ho));
    ho = a.row_idx ? a.row_idx[h] : h;
    return true;
}

// chunk-local point index of CSR entry `col` for local output longitude wo, or -1 when it is not in this chunk
__device__ inline long chunk_point(const Args &a, int64_t col, int wo, int &hi_global)
{
    hi_global = (int)(col / a.nlon_in);
    const int wi = (int)(col - (int64_t)hi_global * a.nlon_in);
    const int wip = (wi + a.pscale * wo) % a.nlon_in;
    if (wip < a.lon_lo_kx || wip >= a.lon_lo_kx + a.nlon_kx) return -1;
    const int hi_local = hi_global - a.lat_halo_start;
    if (hi_local < 0 || hi_local >= a.nlat_halo) return -1;
    return (long)hi_local * a.nlon_kx + (wip - a.lon_lo_kx);
}

// Backward pass 2 straight from the CSR, one wavefront per output point: with the final statistics, adds this chunk's dk and
// dv with fp32 atomics (several output points see the same input point).  attention_cuda_bwd_ring.cu:1312-1440.
// An atomic instruction of a wavefront covers one row of consecutive channels, the cheapest form for the L2.
template <typename T> __global__ __launch_bounds__(256) void pass2_atomic_kernel(const Args a)
{
    int b, ho, wo, lane;
    if (!locate(a, b, ho, wo, lane)) return;
    const long out = ((long)b * a.Ho + ho) * a.Wo + wo;
    const T *q = static_cast<const T *>(a.q) + out * a.ck;
    const T *g = static_cast<const T *>(a.dy) + out * a.cv;
    const long boff = (long)b * a.nlat_halo * a.nlon_kx;
    const T *kx = static_cast<const T *>(a.k) + boff * a.ck;
    const T *vx = static_cast<const T *>(a.v) + boff * a.cv;
    float *dk = a.dk + boff * a.ck, *dv = a.dv + boff * a.cv;
    float qr[NCI], gr[NCI];
#pragma unroll
    for (int i = 0; i < NCI; i++) {
        const int c = lane + 64 * i;
        qr[i] = c < a.ck ? ld(q + c) : 0.f;
        gr[i] = c < a.cv ? ld(g + c) : 0.f;
    }
    const float inv = 1.0f / a.alpha_sum[out], m = a.qdotk_max[out], In = a.integral_norm[out];
    for (int64_t z = a.row_off[ho]; z < a.row_off[ho + 1]; z++) {
        int hi;
        const long pt = chunk_point(a, a.col_idx[z], wo, hi);
        if (pt < 0) continue;
        const T *kr = kx + pt * a.ck, *vr = vx + pt * a.cv;
        float s = 0.f, gv = 0.f;
#pragma unroll
        for (int i = 0; i < NCI; i++) {
            const int c = lane + 64 * i;
            if (c < a.ck) s = fmaf(qr[i], ld(kr + c), s);
            if (c < a.cv) gv = fmaf(gr[i], ld(vr + c), gv);
        }
        s = wave_sum(s);
        gv = wave_sum(gv);
        const float p = __expf(s - m) * a.quad_w[hi] * inv;
        const float sk = (gv - In) * p;
#pragma unroll
        for (int i = 0; i < NCI; i++) {
            const int c = lane + 64 * i;
            if (c < a.ck) atomicAdd(dk + pt * a.ck + c, sk * qr[i]);
            if (c < a.cv) atomicAdd(dv + pt * a.cv + c, p * gr[i]);
        }
    }
}

// Backward pass 2 on the TRANSPOSED neighborhood, no atomics: a wavefront owns P consecutive longitudes of one chunk row
// (batch, input latitude) and walks the CSR entries that have this input latitude (t_off / t_ho / t_dlon: for every input
// latitude of the halo, the (local output latitude, longitude offset col mod nlon_in) of those entries in CSR order).  The
// output point of an entry for input longitude wg is wo = ((wg - dlon) mod nlon_in) / pscale when that division is exact
// and wo is inside the local window.  dk and dv of a chunk point are summed in registers in a fixed order and added to the
// caller's arrays once.  Same arithmetic as attention_cuda_bwd_ring.cu:1312-1440, loop order turned inside out.
template <typename T, int G> __global__ __launch_bounds__(256) void pass2t_kernel(const Args a, const bool vec)
{
    constexpr int P = 64 / G, U = 2;
    const int lane = threadIdx.x & 63;
    const long wid = (long)blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
    const int nb = (a.nlon_kx + P - 1) / P;
    if (wid >= (long)a.B * a.nlat_halo * nb) return;
    const int wb = (int)(wid % nb);
    const int hl = (int)((wid / nb) % a.nlat_halo);
    const int b = (int)(wid / ((long)nb * a.nlat_halo));
    const int64_t z0 = a.t_off[hl], z1 = a.t_off[hl + 1];
    if (z0 >= z1) return; // nothing sees this latitude
    const int w = wb * P + lane / G;
    const bool valid = w < a.nlon_kx;
    const int wl = valid ? w : a.nlon_kx - 1;
    const int c0 = (lane % G) * CPL;
    const long pt = ((long)b * a.nlat_halo + hl) * a.nlon_kx + wl;
    float kr[CPL], vr[CPL], dk[CPL], dv[CPL];
    load8(kr, static_cast<const T *>(a.k) + pt * a.ck, c0, a.ck, vec);
    load8(vr, static_cast<const T *>(a.v) + pt * a.cv, c0, a.cv, vec);
#pragma unroll
    for (int i = 0; i < CPL; i++) dk[i] = dv[i] = 0.f;
    const float wq = a.quad_w[a.lat_halo_start + hl];
    const int wg = a.lon_lo_kx + wl, wg0 = a.lon_lo_kx + wb * P;
    const long lim = (long)a.Wo * a.pscale;
    const long obase = (long)b * a.Ho * a.Wo;
    const T *__restrict__ qb = static_cast<const T *>(a.q) + obase * a.ck;
    const T *__restrict__ gb = static_cast<const T *>(a.dy) + obase * a.cv;
    for (int64_t zb = z0; zb < z1; zb += 64) {
        const int64_t z = zb + lane;
        int ho = 0, dl = 0;
        bool ok = z < z1;
        if (ok) {
            ho = a.t_ho[z], dl = a.t_dlon[z];
            int u = wg0 - dl; // first point's output longitude times pscale; the others follow one apart (cyclically)
            if (u < 0) u += a.nlon_in;
            ok = u < lim || u + (P - 1) >= a.nlon_in;
        }
        unsigned long long cand = __ballot(ok);
        while (cand) {
            long o[U];
            bool in[U];
            float qq[U][CPL], gg[U][CPL], S[U], m[U], In[U];
#pragma unroll
            for (int u = 0; u < U; u++) {
                const bool has = cand != 0;
                const int j = has ? __builtin_ctzll(cand) : 0;
                cand &= cand - 1;
                const int hj = __builtin_amdgcn_readlane(ho, j), dj = __builtin_amdgcn_readlane(dl, j);
                int t = wg - dj;
                if (t < 0) t += a.nlon_in;
                int wo = t;
                bool exact = true;
                if (a.pscale != 1) wo = t / a.pscale, exact = wo * a.pscale == t;
                in[u] = has && valid && exact && wo < a.Wo;
                o[u] = in[u] ? (long)hj * a.Wo + wo : 0;
            }
#pragma unroll
            for (int u = 0; u < U; u++) {
                load8(qq[u], qb + o[u] * a.ck, c0, a.ck, vec);
                load8(gg[u], gb + o[u] * a.cv, c0, a.cv, vec);
                S[u] = a.alpha_sum[obase + o[u]], m[u] = a.qdotk_max[obase + o[u]], In[u] = a.integral_norm[obase + o[u]];
            }
#pragma unroll
            for (int u = 0; u < U; u++) {
                float d = 0.f, e = 0.f;
#pragma unroll
                for (int i = 0; i < CPL; i++) d = fmaf(qq[u][i], kr[i], d), e = fmaf(gg[u][i], vr[i], e);
                const float s = group_sum<G>(d), gv = group_sum<G>(e);
                const float p = in[u] ? __expf(s - m[u]) * wq / S[u] : 0.f;
                const float sk = in[u] ? (gv - In[u]) * p : 0.f;
#pragma unroll
                for (int i = 0; i < CPL; i++) dk[i] = fmaf(sk, qq[u][i], dk[i]), dv[i] = fmaf(p, gg[u][i], dv[i]);
            }
        }
    }
    if (!valid) return;
    float cur[CPL];
    load8(cur, a.dk + pt * a.ck, c0, a.ck, vec);
#pragma unroll
    for (int i = 0; i < CPL; i++) cur[i] += dk[i];
    store8(a.dk + pt * a.ck, cur, c0, a.ck, vec);
    load8(cur, a.dv + pt * a.cv, c0, a.cv, vec);
#pragma unroll
    for (int i = 0; i < CPL; i++) cur[i] += dv[i];
    store8(a.dv + pt * a.cv, cur, c0, a.cv, vec);
}

#undef S2_RING_TAKE

// ---------------------------------------------------------------------------------------------------------------------
// Up-sampling (scatter) direction.  psi is keyed by the chunk's LOCAL input latitude hi_local (row_off has nlat_halo + 1
// entries, empty rows for pole padding), col_idx = ho_local * nlon_out_global + wo_shifted with
// wo_shifted = (wo - first local output longitude) mod nlon_out_global; input cell (hi_local, wi_global) is seen by the
// local output cell (ho_local, w) with w = (wo_shifted + pscale_out * wi_global) mod nlon_out_global iff w < nlon_out.
// The cell that normalises the softmax is not the row key here, so a step runs in three phases like the reference's
// (attention_cuda_fwd_ring_upsample.cu:40-66): scatter the chunk's maxima, rescale the state, scatter the sums.
// ---------------------------------------------------------------------------------------------------------------------
struct UpArgs {
    const void *k, *v, *q, *dy;
    float *y_acc, *alpha_sum, *qdotk_max, *max_curr, *integral, *alpha_k, *alpha_kvw;
    const float *integral_norm;
    float *dk, *dv;
    const float *quad_w;
    const int64_t *col_idx, *row_off;
    int B, nlat_halo, nlon_kx, Ho, Wo, ck, cv, nlon_out_global, pscale_out, lon_lo_kx, lat_halo_start;
};

__device__ inline void atomic_max_float(float *addr, float val)
{
    int *ai = reinterpret_cast<int *>(addr);
    int old = *ai;
    while (val > __int_as_float(old)) {
        const int assumed = old;
        old = atomicCAS(ai, assumed, __float_as_int(val));
        if (old == assumed) break;
    }
}

// chunk cell of this wavefront; false past the end or when its psi row is empty
__device__ inline bool up_locate(const UpArgs &a, int &b, int &hi, int &wi_local, int &lane, int64_t &z0, int64_t &z1)
{
    lane = threadIdx.x & 63;
    const long pid = (long)blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
    if (pid >= (long)a.B * a.nlat_halo * a.nlon_kx) return false;
    wi_local = (int)(pid % a.nlon_kx);
    hi = (int)((pid / a.nlon_kx) % a.nlat_halo);
    b = (int)(pid / ((long)a.nlon_kx * a.nlat_halo));
    z0 = a.row_off[hi], z1 = a.row_off[hi + 1];
    return z1 > z0;
}

// local output cell index of entry `col` for global input longitude wi_global, or -1 when another rank owns it
__device__ inline long up_cell(const UpArgs &a, int64_t col, int wi_global)
{
    const int ho = (int)(col / a.nlon_out_global);
    int w = (int)(col - (int64_t)ho * a.nlon_out_global) + a.pscale_out * wi_global;
    if (w >= a.nlon_out_global) w -= a.nlon_out_global;
    return w < a.Wo ? (long)ho * a.Wo + w : -1;
}

template <typename T> __device__ inline float up_dot(const float (&x)[NCI], const T *row, int n, int lane)
{
    float s = 0.f;
#pragma unroll
    for (int i = 0; i < NCI; i++) {
        const int c = lane + 64 * i;
        if (c < n) s = fmaf(x[i], ld(row + c), s);
    }
    return wave_sum(s);
}

template <typename T> __device__ inline void up_load(float (&x)[NCI], const T *row, int n, int lane)
{
#pragma unroll
    for (int i = 0; i < NCI; i++) {
        const int c = lane + 64 * i;
        x[i] = c < n ? ld(row + c) : 0.f;
    }
}

// phase 1: max_curr (a copy of qdotk_max) takes in the chunk's scores.  attention_cuda_fwd_ring_upsample.cu:108-151.
template <typename T> __global__ __launch_bounds__(256) void up_max_kernel(const UpArgs a)
{
    int b, hi, wl, lane;
    int64_t z0, z1;
    if (!up_locate(a, b, hi, wl, lane, z0, z1)) return;
    float kr[NCI];
    up_load(kr, static_cast<const T *>(a.k) + (((long)b * a.nlat_halo + hi) * a.nlon_kx + wl) * a.ck, a.ck, lane);
    const T *q = static_cast<const T *>(a.q) + (long)b * a.Ho * a.Wo * a.ck;
    for (int64_t z = z0; z < z1; z++) {
        const long cell = up_cell(a, a.col_idx[z], a.lon_lo_kx + wl);
        if (cell < 0) continue;
        const float s = up_dot(kr, q + cell * a.ck, a.ck, lane);
        if (lane == 0) atomic_max_float(a.max_curr + (long)b * a.Ho * a.Wo + cell, s);
    }
}

// phase 2: rescale the state of every local output cell whose maximum moved.  :153-181.
__global__ __launch_bounds__(256) void up_rescale_kernel(const UpArgs a)
{
    const int lane = threadIdx.x & 63;
    const long cell = (long)blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
    if (cell >= (long)a.B * a.Ho * a.Wo) return;
    const float m_old = a.qdotk_max[cell], m_new = a.max_curr[cell];
    if (m_old == m_new) return; // untouched, including -inf == -inf
    const float corr = __expf(m_old - m_new);
    for (int c = lane; c < a.cv; c += 64) a.y_acc[cell * a.cv + c] *= corr;
    if (lane == 0) {
        a.alpha_sum[cell] *= corr;
        a.qdotk_max[cell] = m_new;
    }
}

// phase 3: scatter alpha = exp(q.k - max) w into alpha_sum and alpha v into y_acc.  :183-243.
template <typename T> __global__ __launch_bounds__(256) void up_acc_kernel(const UpArgs a)
{
    int b, hi, wl, lane;
    int64_t z0, z1;
    if (!up_locate(a, b, hi, wl, lane, z0, z1)) return;
    float kr[NCI], vr[NCI];
    const long pt = ((long)b * a.nlat_halo + hi) * a.nlon_kx + wl;
    up_load(kr, static_cast<const T *>(a.k) + pt * a.ck, a.ck, lane);
    up_load(vr, static_cast<const T *>(a.v) + pt * a.cv, a.cv, lane);
    const long boff = (long)b * a.Ho * a.Wo;
    const T *q = static_cast<const T *>(a.q) + boff * a.ck;
    const float w = a.quad_w[a.lat_halo_start + hi];
    for (int64_t z = z0; z < z1; z++) {
        const long cell = up_cell(a, a.col_idx[z], a.lon_lo_kx + wl);
        if (cell < 0) continue;
        const float s = up_dot(kr, q + cell * a.ck, a.ck, lane);
        const float alpha = __expf(s - a.qdotk_max[boff + cell]) * w;
        if (lane == 0) atomicAdd(a.alpha_sum + boff + cell, alpha);
#pragma unroll
        for (int i = 0; i < NCI; i++) {
            const int c = lane + 64 * i;
            if (c < a.cv) atomicAdd(a.y_acc + (boff + cell) * a.cv + c, alpha * vr[i]);
        }
    }
}

// backward pass 1: with the forward's final maximum, scatter integral, alpha_k, alpha_kvw.  attention_cuda_bwd_ring_upsample.cu:88-160.
template <typename T> __global__ __launch_bounds__(256) void up_pass1_kernel(const UpArgs a)
{
    int b, hi, wl, lane;
    int64_t z0, z1;
    if (!up_locate(a, b, hi, wl, lane, z0, z1)) return;
    float kr[NCI], vr[NCI];
    const long pt = ((long)b * a.nlat_halo + hi) * a.nlon_kx + wl;
    up_load(kr, static_cast<const T *>(a.k) + pt * a.ck, a.ck, lane);
    up_load(vr, static_cast<const T *>(a.v) + pt * a.cv, a.cv, lane);
    const long boff = (long)b * a.Ho * a.Wo;
    const T *q = static_cast<const T *>(a.q) + boff * a.ck;
    const T *g = static_cast<const T *>(a.dy) + boff * a.cv;
    const float w = a.quad_w[a.lat_halo_start + hi];
    for (int64_t z = z0; z < z1; z++) {
        const long cell = up_cell(a, a.col_idx[z], a.lon_lo_kx + wl);
        if (cell < 0) continue;
        const float s = up_dot(kr, q + cell * a.ck, a.ck, lane);
        const float gv = up_dot(vr, g + cell * a.cv, a.cv, lane);
        const float alpha = __expf(s - a.qdotk_max[boff + cell]) * w;
        const float ag = alpha * gv;
        if (lane == 0) atomicAdd(a.integral + boff + cell, ag);
#pragma unroll
        for (int i = 0; i < NCI; i++) {
            const int c = lane + 64 * i;
            if (c < a.ck) {
                atomicAdd(a.alpha_k + (boff + cell) * a.ck + c, alpha * kr[i]);
                atomicAdd(a.alpha_kvw + (boff + cell) * a.ck + c, ag * kr[i]);
            }
        }
    }
}

// backward pass 2: dk, dv of every chunk cell, summed over its own row and WRITTEN (no atomics).  :162-240.
template <typename T> __global__ __launch_bounds__(256) void up_pass2_kernel(const UpArgs a)
{
    int b, hi, wl, lane;
    int64_t z0, z1;
    const bool any = up_locate(a, b, hi, wl, lane, z0, z1);
    const long pid = (long)blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
    if (pid >= (long)a.B * a.nlat_halo * a.nlon_kx) return;
    const long pt = pid; // = ((b * nlat_halo + hi) * nlon_kx + wl)
    float kr[NCI], vr[NCI], dk[NCI], dv[NCI];
#pragma unroll
    for (int i = 0; i < NCI; i++) dk[i] = dv[i] = 0.f;
    if (any) {
        up_load(kr, static_cast<const T *>(a.k) + pt * a.ck, a.ck, lane);
        up_load(vr, static_cast<const T *>(a.v) + pt * a.cv, a.cv, lane);
        const long boff = (long)b * a.Ho * a.Wo;
        const T *q = static_cast<const T *>(a.q) + boff * a.ck;
        const T *g = static_cast<const T *>(a.dy) + boff * a.cv;
        const float w = a.quad_w[a.lat_halo_start + hi];
        for (int64_t z = z0; z < z1; z++) {
            const long cell = up_cell(a, a.col_idx[z], a.lon_lo_kx + wl);
            if (cell < 0) continue;
            const T *qc = q + cell * a.ck, *gc = g + cell * a.cv;
            const float s = up_dot(kr, qc, a.ck, lane);
            const float gv = up_dot(vr, gc, a.cv, lane);
            const float p = __expf(s - a.qdotk_max[boff + cell]) * w / a.alpha_sum[boff + cell];
            const float sk = (gv - a.integral_norm[boff + cell]) * p;
#pragma unroll
            for (int i = 0; i < NCI; i++) {
                const int c = lane + 64 * i;
                if (c < a.ck) dk[i] = fmaf(sk, ld(qc + c), dk[i]);
                if (c < a.cv) dv[i] = fmaf(p, ld(gc + c), dv[i]);
            }
        }
    }
#pragma unroll
    for (int i = 0; i < NCI; i++) {
        const int c = lane + 64 * i;
        if (c < a.ck) a.dk[pt * a.ck + c] = dk[i];
        if (c < a.cv) a.dv[pt * a.cv + c] = dv[i];
    }
}

} // namespace s2ring

namespace {

using namespace s2ring;

int check(const s2attn_ring_shape *sh)
{
    if (!sh) return s2attn_fail(S2ATTN_E_INVALID, "ring shape is null");
    if (sh->batch < 1 || sh->nlat_halo < 1 || sh->nlon_kx < 1 || sh->nlat_out < 1 || sh->nlon_out < 1 || sh->nlon_in < 1)
        return s2attn_fail(S2ATTN_E_INVALID, "batch and grid extents must be positive");
    if (sh->ck < 1 || sh->cv < 1) return s2attn_fail(S2ATTN_E_INVALID, "channel counts must be positive");
    if (sh->ck > MAXC || sh->cv > MAXC)
        return s2attn_fail(S2ATTN_E_UNSUPPORTED, "channels above %d are not instantiated (ck=%d, cv=%d)", MAXC, sh->ck, sh->cv);
    if (sh->pscale < 1) return s2attn_fail(S2ATTN_E_INVALID, "pscale must be positive, got %d", sh->pscale);
    if (sh->lon_lo_kx < 0 || sh->lon_lo_kx + sh->nlon_kx > sh->nlon_in)
        return s2attn_fail(S2ATTN_E_INVALID, "chunk [%d, %d) leaves the input grid of %d longitudes", sh->lon_lo_kx, sh->lon_lo_kx + sh->nlon_kx, sh->nlon_in);
    if (sh->dtype != S2ATTN_F32 && sh->dtype != S2ATTN_BF16 && sh->dtype != S2ATTN_F16)
        return s2attn_fail(S2ATTN_E_INVALID, "unknown dtype code %d", sh->dtype);
    return S2ATTN_OK;
}

void fill(Args &a, const s2attn_ring_shape *sh)
{
    a.B = sh->batch, a.nlat_halo = sh->nlat_halo, a.nlon_kx = sh->nlon_kx, a.Ho = sh->nlat_out, a.Wo = sh->nlon_out;
    a.ck = sh->ck, a.cv = sh->cv, a.nlon_in = sh->nlon_in, a.pscale = sh->pscale, a.lon_lo_kx = sh->lon_lo_kx;
    a.lat_halo_start = sh->lat_halo_start;
}

enum Step { FWD, PASS1, PASS2, PASS2T };

template <typename T, int G> int launch_g(Step step, const Args &a, hipStream_t stream)
{
    constexpr int P = 64 / G;
    const long nwaves = step == PASS2T ? (long)a.B * a.nlat_halo * ((a.nlon_kx + P - 1) / P) : (long)a.B * a.Ho * ((a.Wo + P - 1) / P);
    const long nblocks = (nwaves + 3) / 4;
    if (nblocks > 0x7fffffffL) return s2attn_fail(S2ATTN_E_UNSUPPORTED, "problem needs %ld workgroups, more than one grid holds", nblocks);
    if ((long)a.nlat_halo * a.nlon_kx > 0x7fffffffL) return s2attn_fail(S2ATTN_E_UNSUPPORTED, "chunk of more than 2^31 points");
    // 16-byte rows: vector loads and stores
    auto al = [](const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; };
    bool vec = a.ck % CPL == 0 && a.cv % CPL == 0 && al(a.k) && al(a.v) && al(a.q);
    if (step == FWD) vec = vec && al(a.y_acc);
    if (step == PASS1) vec = vec && al(a.dy) && al(a.alpha_k) && al(a.alpha_kvw);
    if (step == PASS2T) vec = vec && al(a.dy) && al(a.dk) && al(a.dv);
    void (*kern)(const Args, const bool) = step == FWD ? fwd_kernel<T, G> : step == PASS1 ? pass1_kernel<T, G> : pass2t_kernel<T, G>;
    hipLaunchKernelGGL(kern, dim3((unsigned)nblocks), dim3(256), 0, stream, a, vec);
    const hipError_t e = hipGetLastError();
    if (e != hipSuccess) return s2attn_fail(S2ATTN_E_LAUNCH, "kernel launch: %s", hipGetErrorString(e));
    return S2ATTN_OK;
}

template <typename T> int launch_t(Step step, const Args &a, hipStream_t stream)
{
    if (step == PASS2) { // one wavefront per output point
        const long nblocks = ((long)a.B * a.Ho * a.Wo + 3) / 4;
        if (nblocks > 0x7fffffffL) return s2attn_fail(S2ATTN_E_UNSUPPORTED, "problem needs %ld workgroups, more than one grid holds", nblocks);
        hipLaunchKernelGGL(pass2_atomic_kernel<T>, dim3((unsigned)nblocks), dim3(256), 0, stream, a);
        const hipError_t e = hipGetLastError();
        if (e != hipSuccess) return s2attn_fail(S2ATTN_E_LAUNCH, "kernel launch: %s", hipGetErrorString(e));
        return S2ATTN_OK;
    }
    const int c = a.ck > a.cv ? a.ck : a.cv; // lanes per point: 8 channels each
    if (c <= 32) return launch_g<T, 4>(step, a, stream);
    if (c <= 64) return launch_g<T, 8>(step, a, stream);
    if (c <= 128) return launch_g<T, 16>(step, a, stream);
    if (c <= 256) return launch_g<T, 32>(step, a, stream);
    return launch_g<T, 64>(step, a, stream);
}

int launch(Step step, const Args &a, int dtype, void *stream)
{
    hipStream_t st = static_cast<hipStream_t>(stream);
    if (dtype == S2ATTN_F32) return launch_t<float>(step, a, st);
    if (dtype == S2ATTN_BF16) return launch_t<__hip_bfloat16>(step, a, st);
    return launch_t<__half>(step, a, st);
}

} // namespace

extern "C" int s2attn_ring_forward_step(const void *k, const void *v, const void *q, float *y_acc, float *alpha_sum, float *qdotk_max,
                                        const float *quad_weights, const int64_t *col_idx, const int64_t *row_off, const int32_t *row_idx,
                                        const s2attn_ring_shape *shape, void *stream)
{
    const int rc = check(shape);
    if (rc != S2ATTN_OK) return rc;
    if (!k || !v || !q || !y_acc || !alpha_sum || !qdotk_max || !quad_weights || !col_idx || !row_off)
        return s2attn_fail(S2ATTN_E_INVALID, "null tensor pointer");
    Args a = {};
    fill(a, shape);
    a.k = k, a.v = v, a.q = q, a.y_acc = y_acc, a.alpha_sum = alpha_sum, a.qdotk_max = qdotk_max;
    a.quad_w = quad_weights, a.col_idx = col_idx, a.row_off = row_off, a.row_idx = row_idx;
    return launch(FWD, a, shape->dtype, stream);
}

extern "C" int s2attn_ring_backward_pass1(const void *k, const void *v, const void *q, const void *dy, float *alpha_sum, float *qdotk_max,
                                          float *integral, float *alpha_k, float *alpha_kvw, const float *quad_weights,
                                          const int64_t *col_idx, const int64_t *row_off, const int32_t *row_idx,
                                          const s2attn_ring_shape *shape, void *stream)
{
    const int rc = check(shape);
    if (rc != S2ATTN_OK) return rc;
    if (!k || !v || !q || !dy || !alpha_sum || !qdotk_max || !integral || !alpha_k || !alpha_kvw || !quad_weights || !col_idx || !row_off)
        return s2attn_fail(S2ATTN_E_INVALID, "null tensor pointer");
    Args a = {};
    fill(a, shape);
    a.k = k, a.v = v, a.q = q, a.dy = dy, a.alpha_sum = alpha_sum, a.qdotk_max = qdotk_max, a.integral = integral;
    a.alpha_k = alpha_k, a.alpha_kvw = alpha_kvw;
    a.quad_w = quad_weights, a.col_idx = col_idx, a.row_off = row_off, a.row_idx = row_idx;
    return launch(PASS1, a, shape->dtype, stream);
}

extern "C" int s2attn_ring_backward_pass2(const void *k, const void *v, const void *q, const void *dy, const float *alpha_sum,
                                          const float *qdotk_max, const float *integral_norm, float *dk, float *dv,
                                          const float *quad_weights, const int64_t *col_idx, const int64_t *row_off,
                                          const int32_t *row_idx, const s2attn_ring_shape *shape, void *stream)
{
    const int rc = check(shape);
    if (rc != S2ATTN_OK) return rc;
    if (!k || !v || !q || !dy || !alpha_sum || !qdotk_max || !integral_norm || !dk || !dv || !quad_weights || !col_idx || !row_off)
        return s2attn_fail(S2ATTN_E_INVALID, "null tensor pointer");
    Args a = {};
    fill(a, shape);
    a.k = k, a.v = v, a.q = q, a.dy = dy;
    a.alpha_sum = const_cast<float *>(alpha_sum), a.qdotk_max = const_cast<float *>(qdotk_max), a.integral_norm = integral_norm;
    a.dk = dk, a.dv = dv;
    a.quad_w = quad_weights, a.col_idx = col_idx, a.row_off = row_off, a.row_idx = row_idx;
    return launch(PASS2, a, shape->dtype, stream);
}

extern "C" int s2attn_ring_backward_pass2_transposed(const void *k, const void *v, const void *q, const void *dy, const float *alpha_sum,
                                                     const float *qdotk_max, const float *integral_norm, float *dk, float *dv,
                                                     const float *quad_weights, const int32_t *t_ho, const int32_t *t_dlon,
                                                     const int64_t *t_off, const s2attn_ring_shape *shape, void *stream)
{
    const int rc = check(shape);
    if (rc != S2ATTN_OK) return rc;
    if (!k || !v || !q || !dy || !alpha_sum || !qdotk_max || !integral_norm || !dk || !dv || !quad_weights || !t_ho || !t_dlon || !t_off)
        return s2attn_fail(S2ATTN_E_INVALID, "null tensor pointer");
    Args a = {};
    fill(a, shape);
    a.k = k, a.v = v, a.q = q, a.dy = dy;
    a.alpha_sum = const_cast<float *>(alpha_sum), a.qdotk_max = const_cast<float *>(qdotk_max), a.integral_norm = integral_norm;
    a.dk = dk, a.dv = dv;
    a.quad_w = quad_weights, a.t_ho = t_ho, a.t_dlon = t_dlon, a.t_off = t_off;
    return launch(PASS2T, a, shape->dtype, stream);
}

namespace {

int check_up(const s2attn_ring_up_shape *sh)
{
    if (!sh) return s2attn_fail(S2ATTN_E_INVALID, "ring shape is null");
    if (sh->batch < 1 || sh->nlat_halo < 1 || sh->nlon_kx < 1 || sh->nlat_out < 1 || sh->nlon_out < 1 || sh->nlon_out_global < 1)
        return s2attn_fail(S2ATTN_E_INVALID, "batch and grid extents must be positive");
    if (sh->ck < 1 || sh->cv < 1) return s2attn_fail(S2ATTN_E_INVALID, "channel counts must be positive");
    if (sh->ck > MAXC || sh->cv > MAXC)
        return s2attn_fail(S2ATTN_E_UNSUPPORTED, "channels above %d are not instantiated (ck=%d, cv=%d)", MAXC, sh->ck, sh->cv);
    if (sh->pscale_out < 1 || sh->nlon_out > sh->nlon_out_global)
        return s2attn_fail(S2ATTN_E_INVALID, "pscale_out must be positive and the local output width at most the global one");
    if (sh->lon_lo_kx < 0 || (int64_t)sh->pscale_out * (sh->lon_lo_kx + sh->nlon_kx) > sh->nlon_out_global)
        return s2attn_fail(S2ATTN_E_INVALID, "chunk [%d, %d) leaves the input grid of %d longitudes", sh->lon_lo_kx, sh->lon_lo_kx + sh->nlon_kx,
                           sh->nlon_out_global / sh->pscale_out);
    if (sh->dtype != S2ATTN_F32 && sh->dtype != S2ATTN_BF16 && sh->dtype != S2ATTN_F16)
        return s2attn_fail(S2ATTN_E_INVALID, "unknown dtype code %d", sh->dtype);
    return S2ATTN_OK;
}

void fill_up(UpArgs &a, const s2attn_ring_up_shape *sh)
{
    a.B = sh->batch, a.nlat_halo = sh->nlat_halo, a.nlon_kx = sh->nlon_kx, a.Ho = sh->nlat_out, a.Wo = sh->nlon_out;
    a.ck = sh->ck, a.cv = sh->cv, a.nlon_out_global = sh->nlon_out_global, a.pscale_out = sh->pscale_out;
    a.lon_lo_kx = sh->lon_lo_kx, a.lat_halo_start = sh->lat_halo_start;
}

enum UpStep { UP_MAX, UP_RESCALE, UP_ACC, UP_PASS1, UP_PASS2 };

template <typename T> int launch_up_t(UpStep step, const UpArgs &a, hipStream_t stream)
{
    const long n = step == UP_RESCALE ? (long)a.B * a.Ho * a.Wo : (long)a.B * a.nlat_halo * a.nlon_kx;
    const long nblocks = (n + 3) / 4;
    if (nblocks > 0x7fffffffL) return s2attn_fail(S2ATTN_E_UNSUPPORTED, "problem needs %ld workgroups, more than one grid holds", nblocks);
    void (*kern)(const UpArgs) = nullptr;
    switch (step) {
    case UP_MAX: kern = up_max_kernel<T>; break;
    case UP_RESCALE: kern = up_rescale_kernel; break;
    case UP_ACC: kern = up_acc_kernel<T>; break;
    case UP_PASS1: kern = up_pass1_kernel<T>; break;
    default: kern = up_pass2_kernel<T>; break;
    }
    hipLaunchKernelGGL(kern, dim3((unsigned)nblocks), dim3(256), 0, stream, a);
    const hipError_t e = hipGetLastError();
    if (e != hipSuccess) return s2attn_fail(S2ATTN_E_LAUNCH, "kernel launch: %s", hipGetErrorString(e));
    return S2ATTN_OK;
}

int launch_up(UpStep step, const UpArgs &a, int dtype, void *stream)
{
    hipStream_t st = static_cast<hipStream_t>(stream);
    if (dtype == S2ATTN_F32) return launch_up_t<float>(step, a, st);
    if (dtype == S2ATTN_BF16) return launch_up_t<__hip_bfloat16>(step, a, st);
    return launch_up_t<__half>(step, a, st);
}

} // namespace

extern "C" int s2attn_ring_forward_step_upsample(const void *k, const void *v, const void *q, float *y_acc, float *alpha_sum, float *qdotk_max,
                                                 float *max_scratch, const float *quad_weights, const int64_t *col_idx,
                                                 const int64_t *row_off, const s2attn_ring_up_shape *shape, void *stream)
{
    int rc = check_up(shape);
    if (rc != S2ATTN_OK) return rc;
    if (!k || !v || !q || !y_acc || !alpha_sum || !qdotk_max || !max_scratch || !quad_weights || !col_idx || !row_off)
        return s2attn_fail(S2ATTN_E_INVALID, "null tensor pointer");
    UpArgs a = {};
    fill_up(a, shape);
    a.k = k, a.v = v, a.q = q, a.y_acc = y_acc, a.alpha_sum = alpha_sum, a.qdotk_max = qdotk_max, a.max_curr = max_scratch;
    a.quad_w = quad_weights, a.col_idx = col_idx, a.row_off = row_off;
    const size_t bytes = sizeof(float) * (size_t)a.B * a.Ho * a.Wo;
    const hipError_t e = hipMemcpyAsync(max_scratch, qdotk_max, bytes, hipMemcpyDeviceToDevice, static_cast<hipStream_t>(stream));
    if (e != hipSuccess) return s2attn_fail(S2ATTN_E_LAUNCH, "hipMemcpyAsync: %s", hipGetErrorString(e));
    if ((rc = launch_up(UP_MAX, a, shape->dtype, stream)) != S2ATTN_OK) return rc;
    if ((rc = launch_up(UP_RESCALE, a, shape->dtype, stream)) != S2ATTN_OK) return rc;
    return launch_up(UP_ACC, a, shape->dtype, stream);
}

extern "C" int s2attn_ring_backward_pass1_upsample(const void *k, const void *v, const void *q, const void *dy, const float *qdotk_max,
                                                   float *integral, float *alpha_k, float *alpha_kvw, const float *quad_weights,
                                                   const int64_t *col_idx, const int64_t *row_off, const s2attn_ring_up_shape *shape,
                                                   void *stream)
{
    const int rc = check_up(shape);
    if (rc != S2ATTN_OK) return rc;
    if (!k || !v || !q || !dy || !qdotk_max || !integral || !alpha_k || !alpha_kvw || !quad_weights || !col_idx || !row_off)
        return s2attn_fail(S2ATTN_E_INVALID, "null tensor pointer");
    UpArgs a = {};
    fill_up(a, shape);
    a.k = k, a.v = v, a.q = q, a.dy = dy, a.qdotk_max = const_cast<float *>(qdotk_max);
    a.integral = integral, a.alpha_k = alpha_k, a.alpha_kvw = alpha_kvw;
    a.quad_w = quad_weights, a.col_idx = col_idx, a.row_off = row_off;
    return launch_up(UP_PASS1, a, shape->dtype, stream);
}

extern "C" int s2attn_ring_backward_pass2_upsample(const void *k, const void *v, const void *q, const void *dy, const float *alpha_sum,
                                                   const float *qdotk_max, const float *integral_norm, float *dk, float *dv,
                                                   const float *quad_weights, const int64_t *col_idx, const int64_t *row_off,
                                                   const s2attn_ring_up_shape *shape, void *stream)
{
    const int rc = check_up(shape);
    if (rc != S2ATTN_OK) return rc;
    if (!k || !v || !q || !dy || !alpha_sum || !qdotk_max || !integral_norm || !dk || !dv || !quad_weights || !col_idx || !row_off)
        return s2attn_fail(S2ATTN_E_INVALID, "null tensor pointer");
    UpArgs a = {};
    fill_up(a, shape);
    a.k = k, a.v = v, a.q = q, a.dy = dy;
    a.alpha_sum = const_cast<float *>(alpha_sum), a.qdotk_max = const_cast<float *>(qdotk_max), a.integral_norm = integral_norm;
    a.dk = dk, a.dv = dv;
    a.quad_w = quad_weights, a.col_idx = col_idx, a.row_off = row_off;
    return launch_up(UP_PASS2, a, shape->dtype, stream);
}
