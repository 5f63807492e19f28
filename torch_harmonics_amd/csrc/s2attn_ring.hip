// Ring-step operators: one longitude chunk of K/V at a time, softmax state kept by the caller.
//
// These are the building blocks of a longitude-sharded layer (K/V chunks travel around a ring of devices while q and
// the per-point state stay put; torch_harmonics/distributed/distributed_attention.py:141-176, 303-431).  Nothing here
// talks to another device: each call folds ONE chunk into the state (forward, backward pass 1) or produces that chunk's
// dk/dv (backward pass 2).  Both directions are covered: gather (psi keyed by output latitude;
// attention_cuda_fwd_ring.cu:66-175, attention_cuda_bwd_ring.cu:78-205, 1312-1440) and up-sampling (psi keyed by input
// latitude; attention_cuda_fwd_ring_upsample.cu:108-300, attention_cuda_bwd_ring_upsample.cu:88-240).
//
// Conventions (the reference's): heads are folded into the batch; state is fp32 in the natural-exponential domain
// (qdotk_max = running max of q.k, alpha_sum = sum of exp(q.k - max) * w, y_acc = the same sum weighted with v).
//
// Every kernel is a GATHER: a cell that owns a sum (an output cell in the forward and pass 1, a chunk point in pass 2)
// walks the neighborhood entries of its own latitude and adds up in registers, in a fixed order, without atomics.  Where
// psi is keyed by the other grid (pass 2 of the gather direction, forward and pass 1 of the up-sampling direction) the
// caller passes the entries regrouped by the owner's latitude (a stable sort, see include/s2attn.h).  Two relations
// between an owner at longitude x and its partner, both with a modulus N, a scale and a window [win_lo, win_lo + win_n):
//   as given:    partner longitude p = (off + scale * x) mod N, used iff p is inside the window (partner units);
//   transposed:  t = (x - off) mod N must be inside the window (owner units times scale) and divisible by scale,
//                partner longitude = (t - win_lo) / scale.
// A wavefront owns P = 64 / G consecutive longitudes of one (batch, latitude); the G lanes of a cell hold 8 consecutive
// channels each (G = 4 for up to 32 channels ... 64 for up to 512).  The wavefront reads the entries 64 at a time, one
// per lane: splitting col, the latitude test and a test whether ANY of its cells can use the entry run once per entry in
// parallel; the surviving entries are then taken U at a time by all cells together (each at its own shifted longitude, so
// the partner rows read for one entry are consecutive in memory), with U independent loads in flight per lane.

#include "s2attn_internal.h"

#include <hip/hip_bf16.h>
#include <hip/hip_fp16.h>
#include <hip/hip_runtime.h>

#include <cstdint>

namespace s2ring {

constexpr int MAXC = 512;      // channels per (folded) head
constexpr int CPL = 8;         // channels per lane in the lane-group kernels
constexpr int NCI = MAXC / 64; // channels per lane in the one-wavefront-per-point kernel

struct Args {
    const void *k, *v, *q, *dy;
    float *y_acc, *alpha_sum, *qdotk_max, *integral, *alpha_k, *alpha_kvw; // state (read-only where they are inputs)
    const float *integral_norm;
    float *dk, *dv;
    const float *quad_w;
    const int64_t *col_idx, *row_off; // psi as given: col = partner latitude * N + off
    const int32_t *row_idx;           // launch order of the owners' latitudes, longest first (may be null: natural order)
    const int64_t *t_off;             // psi regrouped by the owner's latitude: entries t_off[r] .. t_off[r + 1] of latitude r
    const int32_t *t_lat, *t_lon;     //   (partner's local latitude, off)
    int B, nlat_halo, nlon_kx, Ho, Wo, ck, cv;
    int N, scale, win_lo, win_n; // longitude relation, see the top of the file
    int M, win_q;                // N / scale and win_n / scale (regrouped psi: the relation in partner units)
    int lat_off;                 // as given: partner's local latitude = col / N - lat_off
    int lat_halo_start;          // global input latitude of the chunk's row 0 (quadrature weights)
    int lon_lo_kx;               // first global input longitude of the chunk
    bool fixed_max;              // pass 1 of the up-sampling direction: qdotk_max is the forward's final one, not updated
    bool overwrite;              // pass 2: dk, dv are written instead of added to
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

// x of lane (l ^ 1), (l ^ 2) [quad permutes], (7 - l % 8) [half-row mirror], (15 - l % 16) [row mirror] by data-parallel
// primitives: no LDS round trip
template <int CTRL> __device__ inline float dpp_read(float x)
{
    return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(x), CTRL, 0xf, 0xf, false));
}

// sum over the G lanes of a cell, in every lane of it
template <int G> __device__ inline float group_sum(float x)
{
    x += dpp_read<0xB1>(x); // quad_perm [1, 0, 3, 2]
    x += dpp_read<0x4E>(x); // quad_perm [2, 3, 0, 1]
    if constexpr (G >= 8) x += dpp_read<0x141>(x);  // the other quad of the 8 lanes holds its own sum in every lane
    if constexpr (G >= 16) x += dpp_read<0x140>(x); // likewise the other half of the 16 lanes
    if constexpr (G >= 32) x += __shfl_xor(x, 16);
    if constexpr (G >= 64) x += __shfl_xor(x, 32);
    return x;
}

template <typename T> __device__ inline void unpack8(float (&x)[CPL], const T *p);
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

// A lane's 8 channels are [ca, ca + 4) and [cb, cb + 4) of a row of n channels (zeros past the end).  VEC: n is a multiple
// of 8 and the rows are 16-byte aligned; 16-bit storage then has cb = ca + 4 and takes both pieces with one 16-byte load.
template <typename T, bool VEC> __device__ inline void load8(float (&x)[CPL], const T *row, int ca, int cb, int n)
{
    if constexpr (VEC) {
        if constexpr (sizeof(T) == 4) {
            const float4 lo = ca < n ? *reinterpret_cast<const float4 *>(row + ca) : make_float4(0.f, 0.f, 0.f, 0.f);
            const float4 hi = cb < n ? *reinterpret_cast<const float4 *>(row + cb) : make_float4(0.f, 0.f, 0.f, 0.f);
            x[0] = lo.x, x[1] = lo.y, x[2] = lo.z, x[3] = lo.w, x[4] = hi.x, x[5] = hi.y, x[6] = hi.z, x[7] = hi.w;
        } else if (ca < n) {
            unpack8(x, row + ca);
        } else {
#pragma unroll
            for (int i = 0; i < CPL; i++) x[i] = 0.f;
        }
    } else {
#pragma unroll
        for (int i = 0; i < 4; i++) x[i] = ca + i < n ? ld(row + ca + i) : 0.f, x[4 + i] = cb + i < n ? ld(row + cb + i) : 0.f;
    }
}

template <bool VEC> __device__ inline void store8(float *row, const float (&x)[CPL], int ca, int cb, int n)
{
    if constexpr (VEC) {
        if (ca < n) *reinterpret_cast<float4 *>(row + ca) = make_float4(x[0], x[1], x[2], x[3]);
        if (cb < n) *reinterpret_cast<float4 *>(row + cb) = make_float4(x[4], x[5], x[6], x[7]);
    } else {
#pragma unroll
        for (int i = 0; i < 4; i++) {
            if (ca + i < n) row[ca + i] = x[i];
            if (cb + i < n) row[cb + i] = x[4 + i];
        }
    }
}

// The wavefront's place on a grid of nrow x ncol cells per batch: P longitudes of one row, `stride` apart (the regrouped
// relation only joins cells of one residue class modulo scale with an entry, so a wavefront takes its cells from one class).
template <int G> struct Place {
    int b, row, x, x0; // batch, latitude (after the launch order), this lane's longitude (clamped), the wavefront's first one
    int ca, cb;        // the lane's channels: [ca, ca + 4) and [cb, cb + 4)
    bool valid, first; // the lane's longitude is inside the row; first lane of its cell
    static __host__ __device__ inline long blocks_per_row(int ncol, int stride) { return (long)stride * (((ncol + stride - 1) / stride + 64 / G - 1) / (64 / G)); }
    // split: with 32-bit vector loads the G lanes of a cell take 16 consecutive bytes each, twice (channels 4 s .. and
    // 4 G + 4 s ..), so that one load instruction of the wavefront reads whole 64-byte blocks; otherwise 8 s .. 8 s + 7.
    __device__ inline bool locate(int B, int nrow, int ncol, const int32_t *order, int stride, bool split)
    {
        constexpr int P = 64 / G;
        const int lane = threadIdx.x & 63;
        const long wid = (long)blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
        const int nb = (int)blocks_per_row(ncol, stride);
        if (wid >= (long)B * nrow * nb) return false;
        const int wb = (int)(wid % nb);
        const int h = (int)((wid / nb) % nrow);
        b = (int)(wid / ((long)nb * nrow));
        row = order ? order[h] : h;
        x0 = wb % stride + stride * ((wb / stride) * P);
        const int w = x0 + stride * (lane / G);
        valid = w < ncol;
        x = valid ? w : ncol - 1;
        const int sub = lane % G;
        first = sub == 0;
        ca = split ? 4 * sub : CPL * sub;
        cb = split ? 4 * G + 4 * sub : CPL * sub + 4;
        return true;
    }
};

// One entry per lane.  TR = false: entry z of psi as given; the partner grid has nlat2 rows of pwidth cells.  TR = true:
// entry z of the regrouped psi.  x0 = the wavefront's first longitude (TR) or scale * first longitude mod N (as given).
// Returns whether any of the wavefront's P cells can use the entry; off, rowbase (partner row start) and lat (the partner's
// latitude: as given in col for TR = false, local for TR = true) describe it.
template <int G, bool TR> __device__ inline bool scan_entry(const Args &a, int64_t z, int64_t z1, int x0, int nlat2, int pwidth, int &off, int &rowbase, int &lat)
{
    constexpr int P = 64 / G;
    off = 0, rowbase = 0, lat = 0;
    if (z >= z1) return false;
    if constexpr (TR) {
        lat = a.t_lat[z];
        if (lat < 0 || lat >= nlat2) return false;
        int t = x0 - a.t_lon[z]; // first cell; the others follow at scale apart (cyclically): one apart in partner units
        if (t < 0) t += a.N;
        int u = t - a.win_lo;
        if (u < 0) u += a.N;
        int q = u;
        if (a.scale != 1) {
            q = u / a.scale;
            if (q * a.scale != u) return false; // this residue class never meets the entry
        }
        if (!(q < a.win_q || q + (P - 1) >= a.M)) return false;
        off = q; // the first cell's partner longitude relative to the window
        rowbase = lat * pwidth;
    } else {
        const int64_t col = a.col_idx[z];
        if ((uint64_t)col < 0x80000000ull) {
            lat = (int)((uint32_t)col / (uint32_t)a.N);
            off = (int)((uint32_t)col - (uint32_t)lat * (uint32_t)a.N);
        } else {
            lat = (int)(col / a.N);
            off = (int)(col - (int64_t)lat * a.N);
        }
        const int l = lat - a.lat_off;
        if (l < 0 || l >= nlat2) return false;
        int u = off + x0 - a.win_lo; // first cell's partner relative to the window; the others follow at scale apart (cyclically)
        if (u < 0) u += a.N;
        if (u >= a.N) u -= a.N;
        const long span = (long)a.scale * (P - 1);
        if (!(u < a.win_n || u + span >= a.N)) return false;
        rowbase = l * pwidth;
    }
    return true;
}

// index of the lane's partner inside the partner row of entry `off` (relative to the window), or -1.  Regrouped: x = the
// cell's index in the wavefront, off = the first cell's partner longitude relative to the window.  As given: x = scale *
// longitude mod N.
template <bool TR> __device__ inline int partner(const Args &a, int off, int x, bool valid)
{
    if constexpr (TR) {
        int r = off + x;
        if (r >= a.M) r -= a.M;
        return valid && r < a.win_q ? r : -1;
    } else {
        int p = off + x;
        if (p >= a.N) p -= a.N;
        const int rel = p - a.win_lo;
        return valid && (unsigned)rel < (unsigned)a.win_n ? rel : -1;
    }
}

// takes the next surviving entry of the batch: the start of its partner row (the same for the whole wavefront), this lane's
// partner inside that row (or -1) and, for W, the entry's quadrature weight
#define S2_RING_TAKE(u, W)                                                                                               \
    {                                                                                                                    \
        const bool has = cand != 0;                                                                                      \
        const int j = has ? __builtin_ctzll(cand) : 0;                                                                   \
        cand &= cand - 1;                                                                                                \
        const int oj = __builtin_amdgcn_readlane(off, j);                                                                \
        rb[u] = __builtin_amdgcn_readlane(rowbase, j);                                                                   \
        if (W) wgt[u] = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(wq), j));                                \
        pt[u] = has ? partner<TR>(a, oj, xs, pl.valid) : -1;                                                             \
    }

// Channels of row r (an index inside a run of rows that starts at the wavefront-uniform pointer `rows`, n channels each).
// VEC: the address is the uniform row start plus a 32-bit byte offset per lane (the launcher checks that a run of rows
// stays below 2 GiB and r below 2^24), which spares the 64-bit address arithmetic per load.
template <typename T, bool VEC> __device__ inline void load_row(float (&x)[CPL], const T *rows, int r, int n, int ca, int cb)
{
    if constexpr (VEC) {
        const char *base = reinterpret_cast<const char *>(rows);
        const unsigned o = __umul24((unsigned)r, (unsigned)(n * sizeof(T)));
        if constexpr (sizeof(T) == 4) {
            const float4 lo = *reinterpret_cast<const float4 *>(base + (o + 4u * ca)), hi = *reinterpret_cast<const float4 *>(base + (o + 4u * cb));
            x[0] = lo.x, x[1] = lo.y, x[2] = lo.z, x[3] = lo.w, x[4] = hi.x, x[5] = hi.y, x[6] = hi.z, x[7] = hi.w;
        } else {
            unpack8(x, reinterpret_cast<const T *>(base + (o + 2u * ca)));
        }
    } else {
        load8<T, false>(x, rows + (size_t)r * n, ca, cb, n);
    }
}

// entries of the owner's latitude `row`
template <bool TR> __device__ inline void entry_range(const Args &a, int row, int64_t &z0, int64_t &z1)
{
    const int64_t *o = TR ? a.t_off : a.row_off;
    z0 = o[row], z1 = o[row + 1];
}

// quadrature weight of a partner chunk row (forward, pass 1): as given the entry names the global latitude, regrouped the local one
template <bool TR> __device__ inline float partner_weight(const Args &a, bool ok, int lat)
{
    return ok ? a.quad_w[TR ? a.lat_halo_start + lat : lat] : 0.f;
}

// Forward: folds the chunk into (y_acc, alpha_sum, qdotk_max) of every output cell.  attention_cuda_fwd_ring.cu:66-175;
// TR (up-sampling, psi regrouped by output latitude): the result of the three scatter phases of
// attention_cuda_fwd_ring_upsample.cu:108-243 with the running maximum kept per cell instead.
template <typename T, int G, bool TR, bool VEC> __global__ __launch_bounds__(256) void fwd_kernel(const Args a)
{
    constexpr int U = 4;
    Place<G> pl;
    if (!pl.locate(a.B, a.Ho, a.Wo, a.row_idx, TR ? a.scale : 1, VEC && sizeof(T) == 4)) return;
    const int lane = threadIdx.x & 63;
    // channels of the inner-loop rows, clamped into the row: the vector loads there are unconditional (lanes past the end
    // re-read channels 0 .. 7; what they compute meets a zero operand or is never stored)
    const int ka = VEC && pl.ca >= a.ck ? 0 : pl.ca, kb = VEC && pl.cb >= a.ck ? 4 : pl.cb;
    const int va = VEC && pl.ca >= a.cv ? 0 : pl.ca, vb = VEC && pl.cb >= a.cv ? 4 : pl.cb;
    const long out = ((long)pl.b * a.Ho + pl.row) * a.Wo + pl.x;
    const int xs = TR ? lane / G : (int)(((long)a.scale * pl.x) % a.N), xs0 = TR ? pl.x0 : (int)(((long)a.scale * pl.x0) % a.N);
    const T *__restrict__ kx = static_cast<const T *>(a.k) + (long)pl.b * a.nlat_halo * a.nlon_kx * a.ck;
    const T *__restrict__ vx = static_cast<const T *>(a.v) + (long)pl.b * a.nlat_halo * a.nlon_kx * a.cv;
    float qr[CPL], y[CPL];
    load8<T, VEC>(qr, static_cast<const T *>(a.q) + out * a.ck, pl.ca, pl.cb, a.ck);
    load8<float, VEC>(y, a.y_acc + out * a.cv, pl.ca, pl.cb, a.cv);
    float S = a.alpha_sum[out], m = a.qdotk_max[out];
    int64_t z0, z1;
    entry_range<TR>(a, pl.row, z0, z1);
    for (int64_t zb = z0; zb < z1; zb += 64) {
        int off, rowbase, lat;
        const bool ok = scan_entry<G, TR>(a, zb + lane, z1, xs0, a.nlat_halo, a.nlon_kx, off, rowbase, lat);
        const float wq = partner_weight<TR>(a, ok, lat);
        unsigned long long cand = __ballot(ok);
        while (cand) {
            int pt[U], rb[U];
            float wgt[U], kk[U][CPL], vv[U][CPL], s[U];
#pragma unroll
            for (int u = 0; u < U; u++) S2_RING_TAKE(u, true)
#pragma unroll
            for (int u = 0; u < U; u++) {
                const int r = pt[u] < 0 ? 0 : pt[u];
                load_row<T, VEC>(kk[u], kx + (long)rb[u] * a.ck, r, a.ck, ka, kb);
                load_row<T, VEC>(vv[u], vx + (long)rb[u] * a.cv, r, a.cv, va, vb);
            }
            __builtin_amdgcn_sched_barrier(0); // every load of the step is in flight before the first use
            float mn = m;
#pragma unroll
            for (int u = 0; u < U; u++) {
                float d = 0.f;
#pragma unroll
                for (int i = 0; i < CPL; i++) d = fmaf(qr[i], kk[u][i], d);
                s[u] = group_sum<G>(d);
                if (pt[u] >= 0) mn = fmaxf(mn, s[u]);
            }
            if (__any(mn > m)) { // a maximum moved somewhere in the wavefront; m = -inf before the first neighbor: factor 0
                const float corr = mn > m ? __expf(m - mn) : 1.f;
                S *= corr;
#pragma unroll
                for (int i = 0; i < CPL; i++) y[i] *= corr;
            }
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
    if (pl.first) {
        a.alpha_sum[out] = S;
        a.qdotk_max[out] = m;
    }
    store8<VEC>(a.y_acc + out * a.cv, y, pl.ca, pl.cb, a.cv);
}

// Backward pass 1: folds the chunk into (integral = sum alpha <dy, v>, alpha_k = sum alpha k, alpha_kvw = sum alpha
// <dy, v> k) and, with a running maximum, (alpha_sum, qdotk_max) (attention_cuda_bwd_ring.cu:78-205); with fixed_max the
// maximum is the forward's final one and only the three sums are touched (attention_cuda_bwd_ring_upsample.cu:88-160).
template <typename T, int G, bool TR, bool VEC> __global__ __launch_bounds__(256) void pass1_kernel(const Args a)
{
    constexpr int U = 3;
    Place<G> pl;
    if (!pl.locate(a.B, a.Ho, a.Wo, a.row_idx, TR ? a.scale : 1, VEC && sizeof(T) == 4)) return;
    const int lane = threadIdx.x & 63;
    // channels of the inner-loop rows, clamped into the row: the vector loads there are unconditional (lanes past the end
    // re-read channels 0 .. 7; what they compute meets a zero operand or is never stored)
    const int ka = VEC && pl.ca >= a.ck ? 0 : pl.ca, kb = VEC && pl.cb >= a.ck ? 4 : pl.cb;
    const int va = VEC && pl.ca >= a.cv ? 0 : pl.ca, vb = VEC && pl.cb >= a.cv ? 4 : pl.cb;
    const long out = ((long)pl.b * a.Ho + pl.row) * a.Wo + pl.x;
    const int xs = TR ? lane / G : (int)(((long)a.scale * pl.x) % a.N), xs0 = TR ? pl.x0 : (int)(((long)a.scale * pl.x0) % a.N);
    const T *__restrict__ kx = static_cast<const T *>(a.k) + (long)pl.b * a.nlat_halo * a.nlon_kx * a.ck;
    const T *__restrict__ vx = static_cast<const T *>(a.v) + (long)pl.b * a.nlat_halo * a.nlon_kx * a.cv;
    float qr[CPL], gr[CPL], ak[CPL], akg[CPL];
    load8<T, VEC>(qr, static_cast<const T *>(a.q) + out * a.ck, pl.ca, pl.cb, a.ck);
    load8<T, VEC>(gr, static_cast<const T *>(a.dy) + out * a.cv, pl.ca, pl.cb, a.cv);
    load8<float, VEC>(ak, a.alpha_k + out * a.ck, pl.ca, pl.cb, a.ck);
    load8<float, VEC>(akg, a.alpha_kvw + out * a.ck, pl.ca, pl.cb, a.ck);
    const bool fixed = a.fixed_max;
    float S = fixed ? 0.f : a.alpha_sum[out], m = a.qdotk_max[out], I = a.integral[out];
    int64_t z0, z1;
    entry_range<TR>(a, pl.row, z0, z1);
    for (int64_t zb = z0; zb < z1; zb += 64) {
        int off, rowbase, lat;
        const bool ok = scan_entry<G, TR>(a, zb + lane, z1, xs0, a.nlat_halo, a.nlon_kx, off, rowbase, lat);
        const float wq = partner_weight<TR>(a, ok, lat);
        unsigned long long cand = __ballot(ok);
        while (cand) {
            int pt[U], rb[U];
            float wgt[U], kk[U][CPL], vv[U][CPL], s[U], gv[U];
#pragma unroll
            for (int u = 0; u < U; u++) S2_RING_TAKE(u, true)
#pragma unroll
            for (int u = 0; u < U; u++) {
                const int r = pt[u] < 0 ? 0 : pt[u];
                load_row<T, VEC>(kk[u], kx + (long)rb[u] * a.ck, r, a.ck, ka, kb);
                load_row<T, VEC>(vv[u], vx + (long)rb[u] * a.cv, r, a.cv, va, vb);
            }
            __builtin_amdgcn_sched_barrier(0); // every load of the step is in flight before the first use
            float mn = m;
#pragma unroll
            for (int u = 0; u < U; u++) {
                float d = 0.f, e = 0.f;
#pragma unroll
                for (int i = 0; i < CPL; i++) d = fmaf(qr[i], kk[u][i], d), e = fmaf(gr[i], vv[u][i], e);
                s[u] = group_sum<G>(d);
                gv[u] = group_sum<G>(e);
                if (pt[u] >= 0 && !fixed) mn = fmaxf(mn, s[u]);
            }
            if (__any(mn > m)) { // never with a fixed maximum
                const float corr = mn > m ? __expf(m - mn) : 1.f;
                S *= corr, I *= corr;
#pragma unroll
                for (int i = 0; i < CPL; i++) ak[i] *= corr, akg[i] *= corr;
            }
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
    if (pl.first) {
        if (!fixed) {
            a.alpha_sum[out] = S;
            a.qdotk_max[out] = m;
        }
        a.integral[out] = I;
    }
    store8<VEC>(a.alpha_k + out * a.ck, ak, pl.ca, pl.cb, a.ck);
    store8<VEC>(a.alpha_kvw + out * a.ck, akg, pl.ca, pl.cb, a.ck);
}

// Backward pass 2: with the final statistics, dk and dv of every chunk point, summed over the output cells that see it and
// added to (or, with overwrite, written into) the caller's arrays once.  Same arithmetic as attention_cuda_bwd_ring.cu:
// 1312-1440 (TR: psi regrouped by input latitude, loop order turned inside out) and
// attention_cuda_bwd_ring_upsample.cu:162-240 (psi as given, keyed by the chunk's own latitude).
template <typename T, int G, bool TR, bool VEC> __global__ __launch_bounds__(256) void pass2_kernel(const Args a)
{
    constexpr int U = 4;
    Place<G> pl;
    if (!pl.locate(a.B, a.nlat_halo, a.nlon_kx, a.row_idx, TR ? a.scale : 1, VEC && sizeof(T) == 4)) return;
    const int lane = threadIdx.x & 63;
    // channels of the inner-loop rows, clamped into the row: the vector loads there are unconditional (lanes past the end
    // re-read channels 0 .. 7; what they compute meets a zero operand or is never stored)
    const int ka = VEC && pl.ca >= a.ck ? 0 : pl.ca, kb = VEC && pl.cb >= a.ck ? 4 : pl.cb;
    const int va = VEC && pl.ca >= a.cv ? 0 : pl.ca, vb = VEC && pl.cb >= a.cv ? 4 : pl.cb;
    int64_t z0, z1;
    entry_range<TR>(a, pl.row, z0, z1);
    if (z0 >= z1 && !a.overwrite) return; // nothing sees this latitude
    const long pt0 = ((long)pl.b * a.nlat_halo + pl.row) * a.nlon_kx + pl.x;
    float kr[CPL], vr[CPL], dk[CPL], dv[CPL];
    load8<T, VEC>(kr, static_cast<const T *>(a.k) + pt0 * a.ck, pl.ca, pl.cb, a.ck);
    load8<T, VEC>(vr, static_cast<const T *>(a.v) + pt0 * a.cv, pl.ca, pl.cb, a.cv);
#pragma unroll
    for (int i = 0; i < CPL; i++) dk[i] = dv[i] = 0.f;
    const float wq = z0 < z1 ? a.quad_w[a.lat_halo_start + pl.row] : 0.f; // a padded row outside the grid has no entries and no weight
    const int gx = a.lon_lo_kx + pl.x, gx0 = a.lon_lo_kx + pl.x0;           // global input longitudes
    const int xs = TR ? lane / G : (int)(((long)a.scale * gx) % a.N), xs0 = TR ? gx0 : (int)(((long)a.scale * gx0) % a.N);
    const long obase = (long)pl.b * a.Ho * a.Wo;
    const T *__restrict__ qb = static_cast<const T *>(a.q) + obase * a.ck;
    const T *__restrict__ gb = static_cast<const T *>(a.dy) + obase * a.cv;
    for (int64_t zb = z0; zb < z1; zb += 64) {
        int off, rowbase, lat;
        const bool ok = scan_entry<G, TR>(a, zb + lane, z1, xs0, a.Ho, a.Wo, off, rowbase, lat);
        unsigned long long cand = __ballot(ok);
        while (cand) {
            int pt[U], rb[U];
            float wgt[1], qq[U][CPL], gg[U][CPL], S[U], m[U], In[U];
            (void)wgt;
#pragma unroll
            for (int u = 0; u < U; u++) S2_RING_TAKE(u, false)
#pragma unroll
            for (int u = 0; u < U; u++) {
                const int r = pt[u] < 0 ? 0 : pt[u];
                load_row<T, VEC>(qq[u], qb + (long)rb[u] * a.ck, r, a.ck, ka, kb);
                load_row<T, VEC>(gg[u], gb + (long)rb[u] * a.cv, r, a.cv, va, vb);
                const long o = obase + rb[u] + r;
                S[u] = a.alpha_sum[o], m[u] = a.qdotk_max[o], In[u] = a.integral_norm[o];
            }
            __builtin_amdgcn_sched_barrier(0); // every load of the step is in flight before the first use
#pragma unroll
            for (int u = 0; u < U; u++) {
                float d = 0.f, e = 0.f;
#pragma unroll
                for (int i = 0; i < CPL; i++) d = fmaf(qq[u][i], kr[i], d), e = fmaf(gg[u][i], vr[i], e);
                const float s = group_sum<G>(d), gv = group_sum<G>(e);
                const float p = pt[u] >= 0 ? __expf(s - m[u]) * wq / S[u] : 0.f;
                const float sk = pt[u] >= 0 ? (gv - In[u]) * p : 0.f;
#pragma unroll
                for (int i = 0; i < CPL; i++) dk[i] = fmaf(sk, qq[u][i], dk[i]), dv[i] = fmaf(p, gg[u][i], dv[i]);
            }
        }
    }
    if (!pl.valid) return;
    if (!a.overwrite) {
        float cur[CPL];
        load8<float, VEC>(cur, a.dk + pt0 * a.ck, pl.ca, pl.cb, a.ck);
#pragma unroll
        for (int i = 0; i < CPL; i++) dk[i] += cur[i];
        load8<float, VEC>(cur, a.dv + pt0 * a.cv, pl.ca, pl.cb, a.cv);
#pragma unroll
        for (int i = 0; i < CPL; i++) dv[i] += cur[i];
    }
    store8<VEC>(a.dk + pt0 * a.ck, dk, pl.ca, pl.cb, a.ck);
    store8<VEC>(a.dv + pt0 * a.cv, dv, pl.ca, pl.cb, a.cv);
}

#undef S2_RING_TAKE

// ---------------------------------------------------------------------------------------------------------------------
// Pass 2 of the gather direction straight from psi as given, for callers without the regrouped entries.
// ---------------------------------------------------------------------------------------------------------------------
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
    hi_global = (int)(col / a.N);
    const int wi = (int)(col - (int64_t)hi_global * a.N);
    const int wip = (wi + a.scale * wo) % a.N;
    if (wip < a.win_lo || wip >= a.win_lo + a.nlon_kx) return -1;
    const int hi_local = hi_global - a.lat_halo_start;
    if (hi_local < 0 || hi_local >= a.nlat_halo) return -1;
    return (long)hi_local * a.nlon_kx + (wip - a.win_lo);
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
    if (sh->pscale < 1 || sh->nlon_in % sh->pscale != 0)
        return s2attn_fail(S2ATTN_E_INVALID, "pscale must be a positive divisor of nlon_in = %d, got %d", sh->nlon_in, sh->pscale);
    if (sh->lon_lo_kx < 0 || sh->lon_lo_kx + sh->nlon_kx > sh->nlon_in)
        return s2attn_fail(S2ATTN_E_INVALID, "chunk [%d, %d) leaves the input grid of %d longitudes", sh->lon_lo_kx, sh->lon_lo_kx + sh->nlon_kx, sh->nlon_in);
    if ((int64_t)sh->pscale * sh->nlon_out > sh->nlon_in)
        return s2attn_fail(S2ATTN_E_INVALID, "pscale * nlon_out = %ld exceeds nlon_in = %d", (long)sh->pscale * sh->nlon_out, sh->nlon_in);
    if (sh->dtype != S2ATTN_F32 && sh->dtype != S2ATTN_BF16 && sh->dtype != S2ATTN_F16)
        return s2attn_fail(S2ATTN_E_INVALID, "unknown dtype code %d", sh->dtype);
    return S2ATTN_OK;
}

// gather direction; transposed: the relation seen from a chunk point (pass 2 on the regrouped psi)
void fill(Args &a, const s2attn_ring_shape *sh, bool transposed)
{
    a.B = sh->batch, a.nlat_halo = sh->nlat_halo, a.nlon_kx = sh->nlon_kx, a.Ho = sh->nlat_out, a.Wo = sh->nlon_out;
    a.ck = sh->ck, a.cv = sh->cv, a.N = sh->nlon_in, a.scale = sh->pscale, a.lon_lo_kx = sh->lon_lo_kx;
    a.lat_halo_start = a.lat_off = sh->lat_halo_start;
    if (transposed)
        a.win_lo = 0, a.win_n = sh->pscale * sh->nlon_out;
    else
        a.win_lo = sh->lon_lo_kx, a.win_n = sh->nlon_kx;
    a.M = a.N / a.scale, a.win_q = a.win_n / a.scale;
}

enum Step { FWD, PASS1, PASS2 };

template <typename T, int G, bool TR> int launch_g(Step step, const Args &a, hipStream_t stream)
{
    constexpr int P = 64 / G;
    const int stride = TR ? a.scale : 1;
    const long nwaves = step == PASS2 ? (long)a.B * a.nlat_halo * Place<G>::blocks_per_row(a.nlon_kx, stride) : (long)a.B * a.Ho * Place<G>::blocks_per_row(a.Wo, stride);
    (void)P;
    const long nblocks = (nwaves + 3) / 4;
    if (nblocks > 0x7fffffffL) return s2attn_fail(S2ATTN_E_UNSUPPORTED, "problem needs %ld workgroups, more than one grid holds", nblocks);
    if ((long)a.nlat_halo * a.nlon_kx > 0x7fffffffL || (long)a.Ho * a.Wo > 0x7fffffffL)
        return s2attn_fail(S2ATTN_E_UNSUPPORTED, "more than 2^31 points per batch entry");
    const long wmax = a.nlon_kx > a.Wo ? a.nlon_kx : a.Wo; // 32-bit byte offsets inside one latitude row
    if (wmax >= (1L << 24) || wmax * (a.ck > a.cv ? a.ck : a.cv) * 4 > 0x7fffffffL)
        return s2attn_fail(S2ATTN_E_UNSUPPORTED, "a latitude row of %ld points is too long", wmax);
    // 16-byte rows: vector loads and stores
    auto al = [](const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; };
    bool vec = a.ck % CPL == 0 && a.cv % CPL == 0 && al(a.k) && al(a.v) && al(a.q);
    if (step == FWD) vec = vec && al(a.y_acc);
    if (step == PASS1) vec = vec && al(a.dy) && al(a.alpha_k) && al(a.alpha_kvw);
    if (step == PASS2) vec = vec && al(a.dy) && al(a.dk) && al(a.dv);
    void (*kern)(const Args) = nullptr;
    if (vec)
        kern = step == FWD ? fwd_kernel<T, G, TR, true> : step == PASS1 ? pass1_kernel<T, G, TR, true> : pass2_kernel<T, G, TR, true>;
    else
        kern = step == FWD ? fwd_kernel<T, G, TR, false> : step == PASS1 ? pass1_kernel<T, G, TR, false> : pass2_kernel<T, G, TR, false>;
    hipLaunchKernelGGL(kern, dim3((unsigned)nblocks), dim3(256), 0, stream, a);
    const hipError_t e = hipGetLastError();
    if (e != hipSuccess) return s2attn_fail(S2ATTN_E_LAUNCH, "kernel launch: %s", hipGetErrorString(e));
    return S2ATTN_OK;
}

template <typename T, bool TR> int launch_t(Step step, const Args &a, hipStream_t stream)
{
    const int c = a.ck > a.cv ? a.ck : a.cv; // lanes per cell: 8 channels each
    if (c <= 32) return launch_g<T, 4, TR>(step, a, stream);
    if (c <= 64) return launch_g<T, 8, TR>(step, a, stream);
    if (c <= 128) return launch_g<T, 16, TR>(step, a, stream);
    if (c <= 256) return launch_g<T, 32, TR>(step, a, stream);
    return launch_g<T, 64, TR>(step, a, stream);
}

template <bool TR> int launch(Step step, const Args &a, int dtype, void *stream)
{
    hipStream_t st = static_cast<hipStream_t>(stream);
    if (dtype == S2ATTN_F32) return launch_t<float, TR>(step, a, st);
    if (dtype == S2ATTN_BF16) return launch_t<__hip_bfloat16, TR>(step, a, st);
    return launch_t<__half, TR>(step, a, st);
}

template <typename T> int launch_atomic_t(const Args &a, hipStream_t stream)
{
    const long nblocks = ((long)a.B * a.Ho * a.Wo + 3) / 4; // one wavefront per output point
    if (nblocks > 0x7fffffffL) return s2attn_fail(S2ATTN_E_UNSUPPORTED, "problem needs %ld workgroups, more than one grid holds", nblocks);
    hipLaunchKernelGGL(pass2_atomic_kernel<T>, dim3((unsigned)nblocks), dim3(256), 0, stream, a);
    const hipError_t e = hipGetLastError();
    if (e != hipSuccess) return s2attn_fail(S2ATTN_E_LAUNCH, "kernel launch: %s", hipGetErrorString(e));
    return S2ATTN_OK;
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
    fill(a, shape, false);
    a.k = k, a.v = v, a.q = q, a.y_acc = y_acc, a.alpha_sum = alpha_sum, a.qdotk_max = qdotk_max;
    a.quad_w = quad_weights, a.col_idx = col_idx, a.row_off = row_off, a.row_idx = row_idx;
    return launch<false>(FWD, a, shape->dtype, stream);
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
    fill(a, shape, false);
    a.k = k, a.v = v, a.q = q, a.dy = dy, a.alpha_sum = alpha_sum, a.qdotk_max = qdotk_max, a.integral = integral;
    a.alpha_k = alpha_k, a.alpha_kvw = alpha_kvw;
    a.quad_w = quad_weights, a.col_idx = col_idx, a.row_off = row_off, a.row_idx = row_idx;
    return launch<false>(PASS1, a, shape->dtype, stream);
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
    fill(a, shape, false);
    a.k = k, a.v = v, a.q = q, a.dy = dy;
    a.alpha_sum = const_cast<float *>(alpha_sum), a.qdotk_max = const_cast<float *>(qdotk_max), a.integral_norm = integral_norm;
    a.dk = dk, a.dv = dv;
    a.quad_w = quad_weights, a.col_idx = col_idx, a.row_off = row_off, a.row_idx = row_idx;
    hipStream_t st = static_cast<hipStream_t>(stream);
    if (shape->dtype == S2ATTN_F32) return launch_atomic_t<float>(a, st);
    if (shape->dtype == S2ATTN_BF16) return launch_atomic_t<__hip_bfloat16>(a, st);
    return launch_atomic_t<__half>(a, st);
}

extern "C" int s2attn_ring_backward_pass2_transposed(const void *k, const void *v, const void *q, const void *dy, const float *alpha_sum,
                                                     const float *qdotk_max, const float *integral_norm, float *dk, float *dv,
                                                     const float *quad_weights, const int32_t *t_ho, const int32_t *t_dlon,
                                                     const int64_t *t_off, const int32_t *row_order, const s2attn_ring_shape *shape,
                                                     void *stream)
{
    const int rc = check(shape);
    if (rc != S2ATTN_OK) return rc;
    if (!k || !v || !q || !dy || !alpha_sum || !qdotk_max || !integral_norm || !dk || !dv || !quad_weights || !t_ho || !t_dlon || !t_off)
        return s2attn_fail(S2ATTN_E_INVALID, "null tensor pointer");
    Args a = {};
    fill(a, shape, true);
    a.k = k, a.v = v, a.q = q, a.dy = dy;
    a.alpha_sum = const_cast<float *>(alpha_sum), a.qdotk_max = const_cast<float *>(qdotk_max), a.integral_norm = integral_norm;
    a.dk = dk, a.dv = dv;
    a.quad_w = quad_weights, a.t_lat = t_ho, a.t_lon = t_dlon, a.t_off = t_off, a.row_idx = row_order;
    return launch<true>(PASS2, a, shape->dtype, stream);
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
    if (sh->pscale_out < 1 || sh->nlon_out_global % sh->pscale_out != 0 || sh->nlon_out > sh->nlon_out_global)
        return s2attn_fail(S2ATTN_E_INVALID, "pscale_out must be a positive divisor of nlon_out_global and the local output width at most the global one");
    if (sh->lon_lo_kx < 0 || (int64_t)sh->pscale_out * (sh->lon_lo_kx + sh->nlon_kx) > sh->nlon_out_global)
        return s2attn_fail(S2ATTN_E_INVALID, "chunk [%d, %d) leaves the input grid of %d longitudes", sh->lon_lo_kx, sh->lon_lo_kx + sh->nlon_kx,
                           sh->nlon_out_global / sh->pscale_out);
    if (sh->dtype != S2ATTN_F32 && sh->dtype != S2ATTN_BF16 && sh->dtype != S2ATTN_F16)
        return s2attn_fail(S2ATTN_E_INVALID, "unknown dtype code %d", sh->dtype);
    return S2ATTN_OK;
}

// up-sampling direction; transposed: the relation seen from an output cell (forward and pass 1 on the regrouped psi)
void fill_up(Args &a, const s2attn_ring_up_shape *sh, bool transposed)
{
    a.B = sh->batch, a.nlat_halo = sh->nlat_halo, a.nlon_kx = sh->nlon_kx, a.Ho = sh->nlat_out, a.Wo = sh->nlon_out;
    a.ck = sh->ck, a.cv = sh->cv, a.N = sh->nlon_out_global, a.scale = sh->pscale_out, a.lon_lo_kx = sh->lon_lo_kx;
    a.lat_halo_start = sh->lat_halo_start, a.lat_off = 0;
    if (transposed)
        a.win_lo = sh->pscale_out * sh->lon_lo_kx, a.win_n = sh->pscale_out * sh->nlon_kx;
    else
        a.win_lo = 0, a.win_n = sh->nlon_out;
    a.M = a.N / a.scale, a.win_q = a.win_n / a.scale;
}

} // namespace

extern "C" int s2attn_ring_forward_step_upsample(const void *k, const void *v, const void *q, float *y_acc, float *alpha_sum, float *qdotk_max,
                                                 const float *quad_weights, const int32_t *t_hi, const int32_t *t_dlon, const int64_t *t_off,
                                                 const s2attn_ring_up_shape *shape, void *stream)
{
    const int rc = check_up(shape);
    if (rc != S2ATTN_OK) return rc;
    if (!k || !v || !q || !y_acc || !alpha_sum || !qdotk_max || !quad_weights || !t_hi || !t_dlon || !t_off)
        return s2attn_fail(S2ATTN_E_INVALID, "null tensor pointer");
    Args a = {};
    fill_up(a, shape, true);
    a.k = k, a.v = v, a.q = q, a.y_acc = y_acc, a.alpha_sum = alpha_sum, a.qdotk_max = qdotk_max;
    a.quad_w = quad_weights, a.t_lat = t_hi, a.t_lon = t_dlon, a.t_off = t_off;
    return launch<true>(FWD, a, shape->dtype, stream);
}

extern "C" int s2attn_ring_backward_pass1_upsample(const void *k, const void *v, const void *q, const void *dy, const float *qdotk_max,
                                                   float *integral, float *alpha_k, float *alpha_kvw, const float *quad_weights,
                                                   const int32_t *t_hi, const int32_t *t_dlon, const int64_t *t_off,
                                                   const s2attn_ring_up_shape *shape, void *stream)
{
    const int rc = check_up(shape);
    if (rc != S2ATTN_OK) return rc;
    if (!k || !v || !q || !dy || !qdotk_max || !integral || !alpha_k || !alpha_kvw || !quad_weights || !t_hi || !t_dlon || !t_off)
        return s2attn_fail(S2ATTN_E_INVALID, "null tensor pointer");
    Args a = {};
    fill_up(a, shape, true);
    a.k = k, a.v = v, a.q = q, a.dy = dy, a.qdotk_max = const_cast<float *>(qdotk_max);
    a.integral = integral, a.alpha_k = alpha_k, a.alpha_kvw = alpha_kvw, a.fixed_max = true;
    a.quad_w = quad_weights, a.t_lat = t_hi, a.t_lon = t_dlon, a.t_off = t_off;
    return launch<true>(PASS1, a, shape->dtype, stream);
}

extern "C" int s2attn_ring_backward_pass2_upsample(const void *k, const void *v, const void *q, const void *dy, const float *alpha_sum,
                                                   const float *qdotk_max, const float *integral_norm, float *dk, float *dv,
                                                   const float *quad_weights, const int64_t *col_idx, const int64_t *row_off,
                                                   const int32_t *row_order, const s2attn_ring_up_shape *shape, void *stream)
{
    const int rc = check_up(shape);
    if (rc != S2ATTN_OK) return rc;
    if (!k || !v || !q || !dy || !alpha_sum || !qdotk_max || !integral_norm || !dk || !dv || !quad_weights || !col_idx || !row_off)
        return s2attn_fail(S2ATTN_E_INVALID, "null tensor pointer");
    Args a = {};
    fill_up(a, shape, false);
    a.k = k, a.v = v, a.q = q, a.dy = dy;
    a.alpha_sum = const_cast<float *>(alpha_sum), a.qdotk_max = const_cast<float *>(qdotk_max), a.integral_norm = integral_norm;
    a.dk = dk, a.dv = dv, a.overwrite = true;
    a.quad_w = quad_weights, a.col_idx = col_idx, a.row_off = row_off, a.row_idx = row_order;
    return launch<false>(PASS2, a, shape->dtype, stream);
}
