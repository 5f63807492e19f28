// Spherical neighborhood attention on gfx950: forward, dq and dk/dv kernels, layout
// permutes, and the C entry points declared in include/s2attn.h.
//
// Work decomposition (all attention kernels)
//   One wavefront (= one workgroup of 64 threads) owns a tile of consecutive longitudes of
//   one latitude for one (batch, head) and keeps its per-point vectors (q and the y
//   accumulator, or k, v and the dk, dv accumulators) in registers.  The neighborhood of
//   a whole latitude is a short list of runs (lat, ws, len): for the tile a run touches
//   one contiguous, circular band of the other grid's longitudes, which the wavefront
//   copies into LDS with coalesced 16-byte loads and then slides over (point i reads band
//   rows i + t).  No atomics anywhere: dk/dv are produced by a transposed gather (runs
//   regrouped by input latitude) instead of a scatter.  Longitude ratios between the two
//   grids are removed by the plan (virtual latitudes, see key_point() / query_point()).
//
// Kernel families, chosen on the host from the shape (launch_t):
//   *_h16_kernel<T, D>     16-bit storage, head dim 32/64/128: 16-longitude tiles, 16-bit matrix cores   (s2attn_h16.hpp)
//   *_mfma_kernel<T>       head dim 32: 32-longitude tiles, fp32 matrix cores for runs >= LMIN, vector path below
//   *_fast_kernel<T, P>    head dim P in {4, 8, 16, 32}: 64-longitude tiles, lane = grid point, register-prefetched band
//   *_wide_kernel<T, LPQ>  head dims 33..512: 2 to 16 lanes per grid point
//   *_kernel<T, P, VEC>    everything else (ck != cv, odd head dims, unaligned pointers, narrow grids)
//   Workgroups are issued longest latitude first; the linear block index has (batch, head)
//   fastest (16-bit family: one (batch, head) per XCD at a time), so the 8 XCDs each see one
//   head's band of K/V.
//
// Numerics: storage dtype in/out (fp32, bf16, fp16), softmax and accumulation fp32.  Scores
// are kept in the log2 domain (q, or the score, is multiplied by log2(e)) so the softmax uses
// the hardware exp2.

#include <hip/hip_runtime.h>

#include <cstdarg>
#include <cstdio>
#include <mutex>
#include <type_traits>

#include "s2attn_internal.h"

// This file is compiled four times (see the Makefile), so that the groups of kernel instantiations build side by
// side: S2_PART 1 = everything but the launchers of the 16-longitude matrix-core families, 2 = the 16-bit family
// (s2attn_h16.hpp), 3 = the fp32 family (s2attn_m32.hpp), 4 = its ring-step kernels for 16-bit storage.  S2_PART 0 (the
// default) is the whole library in one unit.
#ifndef S2_PART
#define S2_PART 0
#endif

#if S2_PART <= 1
// ---------------------------------------------------------------------------------
// error reporting
// ---------------------------------------------------------------------------------
static thread_local char g_err[512] = "";

int s2attn_fail(int code, const char *fmt, ...)
{
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
    return code;
}

extern "C" const char *s2attn_last_error(void) { return g_err; }
extern "C" int s2attn_abi_version(void) { return 12; }
#endif

namespace s2 {

constexpr int TQ = 64;          // grid points per wavefront tile (one per lane)
constexpr int TL = 8;           // neighbors per lane between two LDS refills
constexpr float LOG2E = 1.4426950408889634f;
constexpr float NEG_BIG = -3.0e38f;

struct Run {
    int lat, ws, len, pad;
};

// ---- storage types -----------------------------------------------------------------
struct bf16_t {
    unsigned short bits;
};
struct f16_t {
    _Float16 v;
};

__device__ inline float to_f32(float x) { return x; }
__device__ inline float to_f32(bf16_t x) { return __uint_as_float(((unsigned)x.bits) << 16); }
__device__ inline float to_f32(f16_t x) { return (float)x.v; }

__device__ inline void from_f32(float &d, float x) { d = x; }
__device__ inline void from_f32(bf16_t &d, float x)
{
    unsigned u = __float_as_uint(x);
    if ((u & 0x7fffffffu) > 0x7f800000u) { // NaN
        d.bits = (unsigned short)((u >> 16) | 0x0040u);
    } else {
        u += 0x7fffu + ((u >> 16) & 1u); // round to nearest even
        d.bits = (unsigned short)(u >> 16);
    }
}
__device__ inline void from_f32(f16_t &d, float x) { d.v = (_Float16)x; }

template <typename T> struct Vec4;
template <> struct Vec4<float> {
    typedef float4 type;
};
template <> struct Vec4<bf16_t> {
    typedef uint2 type;
};
template <> struct Vec4<f16_t> {
    typedef uint2 type;
};

__device__ inline float4 load4(const float *p) { return *reinterpret_cast<const float4 *>(p); }
__device__ inline float4 load4(const bf16_t *p)
{
    const uint2 r = *reinterpret_cast<const uint2 *>(p);
    return make_float4(__uint_as_float(r.x << 16), __uint_as_float(r.x & 0xffff0000u), __uint_as_float(r.y << 16),
                       __uint_as_float(r.y & 0xffff0000u));
}
__device__ inline float4 load4(const f16_t *p)
{
    union {
        uint2 u;
        _Float16 h[4];
    } r;
    r.u = *reinterpret_cast<const uint2 *>(p);
    return make_float4((float)r.h[0], (float)r.h[1], (float)r.h[2], (float)r.h[3]);
}
__device__ inline void store4(float *p, float4 v) { *reinterpret_cast<float4 *>(p) = v; }
__device__ inline void store4(bf16_t *p, float4 v)
{
    bf16_t a, b, c, d;
    from_f32(a, v.x);
    from_f32(b, v.y);
    from_f32(c, v.z);
    from_f32(d, v.w);
    uint2 r;
    r.x = (unsigned)a.bits | ((unsigned)b.bits << 16);
    r.y = (unsigned)c.bits | ((unsigned)d.bits << 16);
    *reinterpret_cast<uint2 *>(p) = r;
}
__device__ inline void store4(f16_t *p, float4 v)
{
    union {
        uint2 u;
        _Float16 h[4];
    } r;
    r.h[0] = (_Float16)v.x;
    r.h[1] = (_Float16)v.y;
    r.h[2] = (_Float16)v.z;
    r.h[3] = (_Float16)v.w;
    *reinterpret_cast<uint2 *>(p) = r.u;
}


// raw 4-channel fetch (kept in registers while a band is in flight) and its widening to fp32
__device__ inline float4 widen4(float4 r, const float *) { return r; }
__device__ inline float4 widen4(uint2 r, const bf16_t *)
{
    return make_float4(__uint_as_float(r.x << 16), __uint_as_float(r.x & 0xffff0000u), __uint_as_float(r.y << 16), __uint_as_float(r.y & 0xffff0000u));
}
__device__ inline float4 widen4(uint2 r, const f16_t *)
{
    union {
        uint2 u;
        _Float16 h[4];
    } c;
    c.u = r;
    return make_float4((float)c.h[0], (float)c.h[1], (float)c.h[2], (float)c.h[3]);
}

__device__ inline float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }
__device__ inline float fast_log2(float x) { return __builtin_amdgcn_logf(x); }

// Exchange with the lane 32 (16) positions away without going through LDS.  v_permlane32_swap swaps the upper half of its
// first operand with the lower half of its second: called with (x, x) it returns (x of the lower half, x of the upper
// half), each replicated in both halves.  v_permlane16_swap does the same with the odd and even rows of 16 lanes.
__device__ inline float xor32_sum(float x)
{
    const auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
    return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}
__device__ inline float xor32_max(float x)
{
    const auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
    return fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
}
__device__ inline float xor16_sum(float x)
{
    const auto r = __builtin_amdgcn_permlane16_swap(__float_as_uint(x), __float_as_uint(x), false, false);
    return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}
__device__ inline float xor16_max(float x)
{
    const auto r = __builtin_amdgcn_permlane16_swap(__float_as_uint(x), __float_as_uint(x), false, false);
    return fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
}

// Values that a kernel loads from global memory before its main loop and keeps in registers for the whole walk are
// passed through settle() right before the loop.  The empty asm uses the register, so the wait for the load is placed
// there; without it the compiler (which cannot see that the loop only runs on a path that has already waited) puts a
// vmcnt(0) at the first use INSIDE the loop, and that also waits for the tile prefetch issued just before it, every step.
// Uniform reads of the plan and the weights inside a walk that also stores to global memory: through the constant address
// space the load stays a scalar load (neither array is ever written by a kernel); through a plain pointer the compiler must
// assume the store may have changed it and makes it a vector load with a full wait.
template <typename V> __device__ inline V const_load(const V *p)
{
    typedef const V __attribute__((address_space(4))) * cptr;
    return *(cptr)(p);
}
__device__ inline Run const_load(const Run *p)
{
    typedef int i4v __attribute__((ext_vector_type(4)));
    const i4v r = const_load(reinterpret_cast<const i4v *>(p));
    return Run{r[0], r[1], r[2], r[3]};
}
__device__ inline void settle(float &x) { asm("" : "+v"(x)); }
__device__ inline void settle(unsigned &x) { asm("" : "+v"(x)); }
__device__ inline void settle(uint4 &x) { asm("" : "+v"(x.x), "+v"(x.y), "+v"(x.z), "+v"(x.w)); }
template <typename V, int N> __device__ inline void settle(V (&x)[N])
{
#pragma unroll
    for (int i = 0; i < N; i++) settle(x[i]);
}

// ---- LDS staging -------------------------------------------------------------------
// Copies `nrows` grid points (longitudes c0, c0+1, ... wrapping at W) of one latitude and
// one head into LDS as fp32 rows of P floats (zero padded past d), row stride P+4 floats so
// that 128-bit reads by consecutive lanes fall in distinct banks.
//   src : first element of (batch, latitude, longitude 0, head)
//   ld  : elements between two longitudes (num_heads * d)
template <typename T, int P, bool VEC, int NT = TQ>
__device__ inline void stage_rows(float *dst, const T *src, long ld, int d, int c0, int W, int nrows, int lane)
{
    constexpr int LS = P + 4;
    if (VEC) {
        constexpr int V4 = P / 4;
        for (int idx = lane; idx < nrows * V4; idx += NT) {
            const int r = idx / V4, c = 4 * (idx % V4);
            int col = c0 + r;
            while (col >= W) col -= W;
            float4 val = make_float4(0.f, 0.f, 0.f, 0.f);
            if (c < d) val = load4(src + (long)col * ld + c);
            *reinterpret_cast<float4 *>(dst + r * LS + c) = val;
        }
    } else {
        for (int idx = lane; idx < nrows * P; idx += NT) {
            const int r = idx / P, c = idx % P;
            int col = c0 + r;
            while (col >= W) col -= W;
            dst[r * LS + c] = (c < d) ? to_f32(src[(long)col * ld + c]) : 0.f;
        }
    }
}

// Writes `nrows` LDS rows back to consecutive longitudes c0.. (no wrap) of one latitude/head.
template <typename T, int P, bool VEC, int NT = TQ>
__device__ inline void unstage_rows(T *dst, const float *src, long ld, int d, int c0, int nrows, int lane)
{
    constexpr int LS = P + 4;
    if (VEC) {
        constexpr int V4 = P / 4;
        for (int idx = lane; idx < nrows * V4; idx += NT) {
            const int r = idx / V4, c = 4 * (idx % V4);
            if (c < d) store4(dst + (long)(c0 + r) * ld + c, *reinterpret_cast<const float4 *>(src + r * LS + c));
        }
    } else {
        for (int idx = lane; idx < nrows * P; idx += NT) {
            const int r = idx / P, c = idx % P;
            if (c < d) from_f32(dst[(long)(c0 + r) * ld + c], src[r * LS + c]);
        }
    }
}

template <int P> __device__ inline float dot_row(const float (&a)[P], const float *row)
{
    float s0 = 0.f, s1 = 0.f, s2 = 0.f, s3 = 0.f;
#pragma unroll
    for (int c = 0; c < P; c += 4) {
        const float4 x = *reinterpret_cast<const float4 *>(row + c);
        s0 = fmaf(a[c + 0], x.x, s0);
        s1 = fmaf(a[c + 1], x.y, s1);
        s2 = fmaf(a[c + 2], x.z, s2);
        s3 = fmaf(a[c + 3], x.w, s3);
    }
    return (s0 + s1) + (s2 + s3);
}

struct PRun;

struct Args {
    const void *k, *v, *q, *dy;
    void *y, *dk, *dv, *dq;
    float2 *stats; // per (batch, head, ho, wo): (log2-sum-exp of the scaled scores, sum_j p_j <dy, v_j>)
    float *lse;    // forward, optional: log2-sum-exp per (batch, head, ho, wo); backward with saved statistics: the same array
    const void *ysaved; // backward with saved statistics: the forward output
    const float *quad_w;
    const int *goff, *gorder, *soff, *sorder;
    const int *gorder_mixed, *sorder_mixed; // launch orders with long-run and short-run latitudes interleaved
    const Run *gruns, *sruns;
    // work lists of the hybrid kernels: (latitude, pair index or -1) per workgroup row, merged runs of the pairs (see s2attn_pair.hpp)
    const int *gitems, *sitems, *gpoff, *spoff;
    const PRun *gpruns, *spruns;
    int n_gitems, n_sitems;
    // elements between two consecutive grid points of each tensor: num_heads * channels when packed, more when the tensor is a
    // column block of a wider buffer (q | k | v of one fused projection); only the hybrid kernels take unpacked tensors
    unsigned ldk, ldv, ldq, ldy, ldg, lddk, lddv, lddq;
    int unpacked; // any of them differs from the packed value
    int B, nh, Hi, Wi, Ho, Wo, dk_, dv_;
    int kps; // nlon_in / nlon_out when the input grid is the finer one, else 1; see key_point()
    int qps; // nlon_out / nlon_in when the output grid is the finer one, else 1; see query_point()
    int tile_rows; // LDS rows per staged band
    int row_first; // first entry of gorder / sorder this launch covers (dense rows come first, see s2attn_plan_split)
    // one ring step of the forward (ring_fwd_m32_kernel): the chunk's first real input longitude and latitude, its extents,
    // and the caller's running state
    int r_lon_lo, r_nkx, r_lat0, r_nlat;
    int r_qps;   // nlon_out / nlon_in in the up-sampling direction (the plan's output latitudes are then virtual), else 1
    int r_wo;    // local output longitudes
    int r_wlat0; // quadrature weight of a run's input latitude Run::pad is quad_w[pad + r_wlat0]
    float *r_yacc, *r_asum, *r_qmax;
    float *r_integral, *r_ak, *r_akvw; // pass 1 of the backward
    const int2 *gspan; // per virtual output latitude: the arc of neighbor columns of query column 0 (see the plan)
};

// Key-side addressing.  With nlon_in = kps * nlon_out, query column wo sees input columns ws + t + kps * wo: on the
// sub-lattice {par, par + kps, ...} of a real input latitude that is a unit-stride problem.  The plan therefore lists
// neighborhoods over Hi = nlat_in * kps "virtual" latitudes (real latitude * kps + par) of Wi = nlon_out columns each,
// every kernel works as if nlon_in == nlon_out, and only the address of a virtual grid point differs:
// key_point() is the real point index of column 0 of a virtual latitude, consecutive columns lie kps points apart.
// Gather runs carry the real latitude in Run::pad (also the index of the quadrature weight).
__device__ inline long key_point(const Args &a, int b, int vlat, int rlat)
{
    return ((long)b * a.Hi + (long)rlat * a.kps) * a.Wi + (vlat - rlat * a.kps);
}
__device__ inline long key_row(const Args &a, int vlat, int rlat) { return (long)rlat * a.kps * a.Wi + (vlat - rlat * a.kps); }
// The same on the query side for the up-sampling direction (nlon_out = qps * nlon_in): Ho = nlat_out * qps virtual output
// latitudes of Wo = nlon_in columns; scatter runs carry the real output latitude in Run::pad.  The per-point statistics
// (lse, stats) are private to the library and simply indexed by virtual coordinates.
__device__ inline long query_point(const Args &a, int b, int vlat, int rlat)
{
    return ((long)b * a.Ho + (long)rlat * a.qps) * a.Wo + (vlat - rlat * a.qps);
}
__device__ inline long query_row(const Args &a, int vlat, int rlat) { return (long)rlat * a.qps * a.Wo + (vlat - rlat * a.qps); }

// ---------------------------------------------------------------------------------
// forward:  y = sum_j a_j v_j / sum_j a_j
// ---------------------------------------------------------------------------------
template <typename T, int P, bool VEC> __global__ __launch_bounds__(TQ) void fwd_kernel(const Args a)
{
    extern __shared__ float4 smem4[];
    float *Ks = reinterpret_cast<float *>(smem4);
    constexpr int LS = P + 4;
    float *Vs = Ks + a.tile_rows * LS;

    const int lane = threadIdx.x;
    const int BH = a.B * a.nh;
    const int ntile = (a.Wo + TQ - 1) / TQ;
    int id = blockIdx.x;
    const int bh = id % BH;
    id /= BH;
    const int wt = id % ntile;
    const int ho = a.gorder[a.row_first + id / ntile];
    const int b = bh / a.nh, h = bh % a.nh;
    const int wo0 = wt * TQ;
    const int nvalid = min(TQ, a.Wo - wo0);
    constexpr int ps = 1; // the plan removed the longitude stride (virtual latitudes, see key_point())
    const long ldk = (long)a.nh * a.dk_, ldv = (long)a.nh * a.dv_;

    const T *kx = static_cast<const T *>(a.k);
    const T *vx = static_cast<const T *>(a.v);
    const T *qy = static_cast<const T *>(a.q);
    T *y = static_cast<T *>(a.y);

    // q for this lane, pre-multiplied by log2(e)
    stage_rows<T, P, VEC>(Ks, qy + query_point(a, b, ho, ho / a.qps) * ldk + (long)h * a.dk_, ldk * a.qps, a.dk_, wo0, a.Wo, nvalid, lane);
    __syncthreads();
    float qr[P], acc[P];
#pragma unroll
    for (int c = 0; c < P; c++) {
        qr[c] = Ks[lane * LS + c] * LOG2E;
        acc[c] = 0.f;
    }
    float m = NEG_BIG, S = 0.f;

    for (int ri = a.goff[ho]; ri < a.goff[ho + 1]; ri++) {
        const Run run = a.gruns[ri];
        const float w = a.quad_w[run.pad];
        const T *kl = kx + key_point(a, b, run.lat, run.pad) * ldk + (long)h * a.dk_;
        const T *vl = vx + key_point(a, b, run.lat, run.pad) * ldv + (long)h * a.dv_;
        for (int t0 = 0; t0 < run.len; t0 += TL) {
            const int L = min(TL, run.len - t0);
            const int c0 = (run.ws + t0 + ps * wo0) % a.Wi;
            const int nrows = ps * (nvalid - 1) + L;
            __syncthreads();
            stage_rows<T, P, VEC>(Ks, kl, ldk * a.kps, a.dk_, c0, a.Wi, nrows, lane);
            stage_rows<T, P, VEC>(Vs, vl, ldv * a.kps, a.dv_, c0, a.Wi, nrows, lane);
            __syncthreads();

            const float *krow = Ks + (ps * lane) * LS;
            const float *vrow = Vs + (ps * lane) * LS;
            float s[TL];
            float cm = NEG_BIG;
#pragma unroll
            for (int t = 0; t < TL; t++) {
                s[t] = NEG_BIG;
                if (t < L) {
                    s[t] = dot_row<P>(qr, krow + t * LS);
                    cm = fmaxf(cm, s[t]);
                }
            }
            const float mn = fmaxf(m, cm);
            const float corr = fast_exp2(m - mn);
            m = mn;
            S *= corr;
#pragma unroll
            for (int c = 0; c < P; c++) acc[c] *= corr;
#pragma unroll
            for (int t = 0; t < TL; t++) {
                if (t < L) {
                    const float p = fast_exp2(s[t] - mn) * w;
                    S += p;
                    const float *vr = vrow + t * LS;
#pragma unroll
                    for (int c = 0; c < P; c += 4) {
                        const float4 x = *reinterpret_cast<const float4 *>(vr + c);
                        acc[c + 0] = fmaf(p, x.x, acc[c + 0]);
                        acc[c + 1] = fmaf(p, x.y, acc[c + 1]);
                        acc[c + 2] = fmaf(p, x.z, acc[c + 2]);
                        acc[c + 3] = fmaf(p, x.w, acc[c + 3]);
                    }
                }
            }
        }
    }

    if (a.lse && lane < nvalid) a.lse[((long)bh * a.Ho + ho) * a.Wo + wo0 + lane] = m + fast_log2(S);
    const float inv = 1.0f / S;
    __syncthreads();
#pragma unroll
    for (int c = 0; c < P; c += 4)
        *reinterpret_cast<float4 *>(Ks + lane * LS + c) = make_float4(acc[c] * inv, acc[c + 1] * inv, acc[c + 2] * inv, acc[c + 3] * inv);
    __syncthreads();
    unstage_rows<T, P, VEC>(y + query_point(a, b, ho, ho / a.qps) * ldv + (long)h * a.dv_, Ks, ldv * a.qps, a.dv_, wo0, nvalid, lane);
}

// ---------------------------------------------------------------------------------
// backward, query side:  dq = sum_j p_j (g_j - I) k_j   with g_j = <dy, v_j>, I = sum_j p_j g_j
// accumulated online as (A_kg - I A_k) / S, A_k = sum a_j k_j, A_kg = sum a_j g_j k_j; also
// emits (log2 sum a_j + max, I) per query for the dk/dv kernel.
// ---------------------------------------------------------------------------------
template <typename T, int P, bool VEC> __global__ __launch_bounds__(TQ) void dq_kernel(const Args a)
{
    extern __shared__ float4 smem4[];
    float *Ks = reinterpret_cast<float *>(smem4);
    constexpr int LS = P + 4;
    float *Vs = Ks + a.tile_rows * LS;

    const int lane = threadIdx.x;
    const int BH = a.B * a.nh;
    const int ntile = (a.Wo + TQ - 1) / TQ;
    int id = blockIdx.x;
    const int bh = id % BH;
    id /= BH;
    const int wt = id % ntile;
    const int ho = a.gorder[a.row_first + id / ntile];
    const int b = bh / a.nh, h = bh % a.nh;
    const int wo0 = wt * TQ;
    const int nvalid = min(TQ, a.Wo - wo0);
    constexpr int ps = 1; // the plan removed the longitude stride (virtual latitudes, see key_point())
    const long ldk = (long)a.nh * a.dk_, ldv = (long)a.nh * a.dv_;

    const T *kx = static_cast<const T *>(a.k);
    const T *vx = static_cast<const T *>(a.v);
    const T *qy = static_cast<const T *>(a.q);
    const T *gy = static_cast<const T *>(a.dy);
    T *dq = static_cast<T *>(a.dq);

    stage_rows<T, P, VEC>(Ks, qy + query_point(a, b, ho, ho / a.qps) * ldk + (long)h * a.dk_, ldk * a.qps, a.dk_, wo0, a.Wo, nvalid, lane);
    stage_rows<T, P, VEC>(Vs, gy + query_point(a, b, ho, ho / a.qps) * ldv + (long)h * a.dv_, ldv * a.qps, a.dv_, wo0, a.Wo, nvalid, lane);
    __syncthreads();
    float qr[P], gr[P], Ak[P], Akg[P];
#pragma unroll
    for (int c = 0; c < P; c++) {
        qr[c] = Ks[lane * LS + c] * LOG2E;
        gr[c] = Vs[lane * LS + c];
        Ak[c] = 0.f;
        Akg[c] = 0.f;
    }
    float m = NEG_BIG, S = 0.f, Ag = 0.f;

    for (int ri = a.goff[ho]; ri < a.goff[ho + 1]; ri++) {
        const Run run = a.gruns[ri];
        const float w = a.quad_w[run.pad];
        const T *kl = kx + key_point(a, b, run.lat, run.pad) * ldk + (long)h * a.dk_;
        const T *vl = vx + key_point(a, b, run.lat, run.pad) * ldv + (long)h * a.dv_;
        for (int t0 = 0; t0 < run.len; t0 += TL) {
            const int L = min(TL, run.len - t0);
            const int c0 = (run.ws + t0 + ps * wo0) % a.Wi;
            const int nrows = ps * (nvalid - 1) + L;
            __syncthreads();
            stage_rows<T, P, VEC>(Ks, kl, ldk * a.kps, a.dk_, c0, a.Wi, nrows, lane);
            stage_rows<T, P, VEC>(Vs, vl, ldv * a.kps, a.dv_, c0, a.Wi, nrows, lane);
            __syncthreads();

            const float *krow = Ks + (ps * lane) * LS;
            const float *vrow = Vs + (ps * lane) * LS;
            float s[TL], g[TL];
            float cm = NEG_BIG;
#pragma unroll
            for (int t = 0; t < TL; t++) {
                s[t] = NEG_BIG;
                g[t] = 0.f;
                if (t < L) {
                    s[t] = dot_row<P>(qr, krow + t * LS);
                    g[t] = dot_row<P>(gr, vrow + t * LS);
                    cm = fmaxf(cm, s[t]);
                }
            }
            const float mn = fmaxf(m, cm);
            const float corr = fast_exp2(m - mn);
            m = mn;
            S *= corr;
            Ag *= corr;
#pragma unroll
            for (int c = 0; c < P; c++) {
                Ak[c] *= corr;
                Akg[c] *= corr;
            }
#pragma unroll
            for (int t = 0; t < TL; t++) {
                if (t < L) {
                    const float p = fast_exp2(s[t] - mn) * w;
                    const float pg = p * g[t];
                    S += p;
                    Ag += pg;
                    const float *kr = krow + t * LS;
#pragma unroll
                    for (int c = 0; c < P; c += 4) {
                        const float4 x = *reinterpret_cast<const float4 *>(kr + c);
                        Ak[c + 0] = fmaf(p, x.x, Ak[c + 0]);
                        Ak[c + 1] = fmaf(p, x.y, Ak[c + 1]);
                        Ak[c + 2] = fmaf(p, x.z, Ak[c + 2]);
                        Ak[c + 3] = fmaf(p, x.w, Ak[c + 3]);
                        Akg[c + 0] = fmaf(pg, x.x, Akg[c + 0]);
                        Akg[c + 1] = fmaf(pg, x.y, Akg[c + 1]);
                        Akg[c + 2] = fmaf(pg, x.z, Akg[c + 2]);
                        Akg[c + 3] = fmaf(pg, x.w, Akg[c + 3]);
                    }
                }
            }
        }
    }

    const float inv = 1.0f / S;
    const float I = Ag * inv;
    if (lane < nvalid) a.stats[((long)bh * a.Ho + ho) * a.Wo + wo0 + lane] = make_float2(m + fast_log2(S), I);
    __syncthreads();
#pragma unroll
    for (int c = 0; c < P; c += 4)
        *reinterpret_cast<float4 *>(Ks + lane * LS + c)
            = make_float4((Akg[c] - I * Ak[c]) * inv, (Akg[c + 1] - I * Ak[c + 1]) * inv, (Akg[c + 2] - I * Ak[c + 2]) * inv,
                          (Akg[c + 3] - I * Ak[c + 3]) * inv);
    __syncthreads();
    unstage_rows<T, P, VEC>(dq + query_point(a, b, ho, ho / a.qps) * ldk + (long)h * a.dk_, Ks, ldk * a.qps, a.dk_, wo0, nvalid, lane);
}

// ---------------------------------------------------------------------------------
// backward, key/value side (transposed gather).  Lane = input point (hi, wi).  For a run
// (ho, ws, len) the queries that see this point are wo = (floor(delta/ps) - u) mod Wo with
// delta = (wi - ws) mod Wi and neighbor index t = delta mod ps + ps*u < len:
//   dv += p dy,  dk += p (g - I) q,   p = exp2(log2e q.k - lse2) * quad_w[hi]
// ---------------------------------------------------------------------------------
template <typename T, int P, bool VEC> __global__ __launch_bounds__(TQ) void dkdv_kernel(const Args a)
{
    extern __shared__ float4 smem4[];
    float *Qs = reinterpret_cast<float *>(smem4);
    constexpr int LS = P + 4;
    float *Gs = Qs + a.tile_rows * LS;
    float2 *Ss = reinterpret_cast<float2 *>(Gs + a.tile_rows * LS);

    const int lane = threadIdx.x;
    const int BH = a.B * a.nh;
    const int ntile = (a.Wi + TQ - 1) / TQ;
    int id = blockIdx.x;
    const int bh = id % BH;
    id /= BH;
    const int ct = id % ntile;
    const int hi = a.sorder[a.row_first + id / ntile];
    const int b = bh / a.nh, h = bh % a.nh;
    const int wi0 = ct * TQ;
    const int nvalid = min(TQ, a.Wi - wi0);
    constexpr int ps = 1; // the plan removed the longitude stride (virtual latitudes, see key_point())
    const long ldk = (long)a.nh * a.dk_, ldv = (long)a.nh * a.dv_;

    const T *kx = static_cast<const T *>(a.k);
    const T *vx = static_cast<const T *>(a.v);
    const T *qy = static_cast<const T *>(a.q);
    const T *gy = static_cast<const T *>(a.dy);
    T *dk = static_cast<T *>(a.dk);
    T *dv = static_cast<T *>(a.dv);

    stage_rows<T, P, VEC>(Qs, kx + key_point(a, b, hi, hi / a.kps) * ldk + (long)h * a.dk_, ldk * a.kps, a.dk_, wi0, a.Wi, nvalid, lane);
    stage_rows<T, P, VEC>(Gs, vx + key_point(a, b, hi, hi / a.kps) * ldv + (long)h * a.dv_, ldv * a.kps, a.dv_, wi0, a.Wi, nvalid, lane);
    __syncthreads();
    float kr[P], vr[P], dkr[P], dvr[P];
#pragma unroll
    for (int c = 0; c < P; c++) {
        kr[c] = Qs[lane * LS + c] * LOG2E;
        vr[c] = Gs[lane * LS + c];
        dkr[c] = 0.f;
        dvr[c] = 0.f;
    }
    const float w = a.quad_w[hi / a.kps];

    for (int ri = a.soff[hi]; ri < a.soff[hi + 1]; ri++) {
        const Run run = a.sruns[ri];
        const int ho = run.lat;
        int d0 = wi0 - run.ws;
        if (d0 < 0) d0 += a.Wi;
        // lane geometry relative to the first lane (no wrap: d0 + lane may exceed Wi)
        int al, r0;
        if (ps == 1) {
            al = lane;
            r0 = 0;
        } else {
            al = (d0 + lane) / ps - d0 / ps;
            r0 = (d0 + lane) % ps;
        }
        const int a0 = d0 / ps;
        const int span = (d0 + nvalid - 1) / ps - a0; // al of the last valid lane
        const int U = (run.len + ps - 1) / ps;
        const T *ql = qy + query_point(a, b, ho, run.pad) * ldk + (long)h * a.dk_;
        const T *gl = gy + query_point(a, b, ho, run.pad) * ldv + (long)h * a.dv_;
        const float2 *sl = a.stats + ((long)bh * a.Ho + ho) * a.Wo;

        for (int u0 = 0; u0 < U; u0 += TL) {
            const int UL = min(TL, U - u0);
            int c0 = (a0 - u0 - UL + 1) % a.Wo;
            if (c0 < 0) c0 += a.Wo;
            const int nrows = span + UL;
            __syncthreads();
            stage_rows<T, P, VEC>(Qs, ql, ldk * a.qps, a.dk_, c0, a.Wo, nrows, lane);
            stage_rows<T, P, VEC>(Gs, gl, ldv * a.qps, a.dv_, c0, a.Wo, nrows, lane);
            for (int r = lane; r < nrows; r += TQ) {
                int col = c0 + r;
                while (col >= a.Wo) col -= a.Wo;
                Ss[r] = sl[col];
            }
            __syncthreads();

#pragma unroll
            for (int j = 0; j < TL; j++) {
                if (j < UL) {
                    const int row = al + (UL - 1 - j);
                    const int t = r0 + ps * (u0 + j);
                    const float *qrow = Qs + row * LS;
                    const float *grow = Gs + row * LS;
                    float qq[P], gg[P];
#pragma unroll
                    for (int c = 0; c < P; c += 4) {
                        const float4 x = *reinterpret_cast<const float4 *>(qrow + c);
                        const float4 z = *reinterpret_cast<const float4 *>(grow + c);
                        qq[c] = x.x, qq[c + 1] = x.y, qq[c + 2] = x.z, qq[c + 3] = x.w;
                        gg[c] = z.x, gg[c + 1] = z.y, gg[c + 2] = z.z, gg[c + 3] = z.w;
                    }
                    float s0 = 0.f, s1 = 0.f, g0 = 0.f, g1 = 0.f;
#pragma unroll
                    for (int c = 0; c < P; c += 2) {
                        s0 = fmaf(qq[c], kr[c], s0);
                        s1 = fmaf(qq[c + 1], kr[c + 1], s1);
                        g0 = fmaf(gg[c], vr[c], g0);
                        g1 = fmaf(gg[c + 1], vr[c + 1], g1);
                    }
                    const float2 st = Ss[row];
                    float p = fast_exp2((s0 + s1) - st.x) * w;
                    if (t >= run.len) p = 0.f;
                    const float coef = p * ((g0 + g1) - st.y);
#pragma unroll
                    for (int c = 0; c < P; c++) {
                        dkr[c] = fmaf(coef, qq[c], dkr[c]);
                        dvr[c] = fmaf(p, gg[c], dvr[c]);
                    }
                }
            }
        }
    }

    __syncthreads();
#pragma unroll
    for (int c = 0; c < P; c += 4) {
        *reinterpret_cast<float4 *>(Qs + lane * LS + c) = make_float4(dkr[c], dkr[c + 1], dkr[c + 2], dkr[c + 3]);
        *reinterpret_cast<float4 *>(Gs + lane * LS + c) = make_float4(dvr[c], dvr[c + 1], dvr[c + 2], dvr[c + 3]);
    }
    __syncthreads();
    unstage_rows<T, P, VEC>(dk + key_point(a, b, hi, hi / a.kps) * ldk + (long)h * a.dk_, Qs, ldk * a.kps, a.dk_, wi0, nvalid, lane);
    unstage_rows<T, P, VEC>(dv + key_point(a, b, hi, hi / a.kps) * ldv + (long)h * a.dv_, Gs, ldv * a.kps, a.dv_, wi0, nvalid, lane);
}


// ---------------------------------------------------------------------------------
// Wide heads (32 < head dim <= 512): LPQ = 2, 4, 8 or 16 adjacent lanes share one grid point and each keeps a
// 32-channel slice of its vectors, so the register footprint stays that of a 32-channel head; a dot product is
// completed by LPQ-lane butterfly adds.  A wavefront therefore covers 64 / LPQ longitudes.
// A workgroup is WNW wavefronts over the SAME longitudes: they stage every band together and split its neighbors
// (wavefront w takes the w-th quarter of each staged chunk), each with its own running softmax state; the states
// are merged through LDS at the end, in wavefront order, so results do not depend on timing.  The band in LDS --
// 34 KB at 64 channels -- then serves four wavefronts instead of one, and a pole row, thousands of neighbors per
// grid point, is worked on by four wavefronts at once.
// ---------------------------------------------------------------------------------
constexpr int WNW = 4;        // wavefronts per workgroup
constexpr int WNT = TQ * WNW; // threads per workgroup
// Neighbors staged per band refill: each wavefront takes WSUB groups of TL of them.  Two groups where the band stays
// small (64-channel heads: 95 rows, 52 KB for both tiles), one for wider heads.
template <int LPQ> struct WideCfg {
    static constexpr int WSUB = LPQ <= 2 ? 2 : 1;
    static constexpr int TSW = WNW * WSUB * TL;
};

template <int LPQ> __device__ inline float slice_sum(float x)
{
#pragma unroll
    for (int o = 1; o < LPQ; o <<= 1) x += __shfl_xor(x, o);
    return x;
}

#define S2_WIDE_IDS(W_TILED)                                                  \
    constexpr int TQW = TQ / LPQ;                                             \
    constexpr int PT = 32 * LPQ;                                              \
    constexpr int LS = PT + 4;                                                \
    constexpr int TSW = WideCfg<LPQ>::TSW;                                    \
    const int tid = threadIdx.x;                                              \
    const int lane = tid % TQ, wv = tid / TQ;                                 \
    const int qi = lane / LPQ, sl = lane % LPQ;                               \
    const int BH = a.B * a.nh;                                                \
    const int ntile = ((W_TILED) + TQW - 1) / TQW;                            \
    int id_ = blockIdx.x;                                                     \
    const int bh = id_ % BH;                                                  \
    id_ /= BH;                                                                \
    const int wt = id_ % ntile;                                               \
    const int rowsel = id_ / ntile;                                           \
    const int b = bh / a.nh, h = bh % a.nh;                                   \
    const int w0 = wt * TQW;                                                  \
    const int nvalid = min(TQW, (W_TILED)-w0);                                \
    const long ldk = (long)a.nh * a.dk_, ldv = (long)a.nh * a.dv_;

template <typename T, int LPQ, bool VEC> __global__ __launch_bounds__(WNT) void fwd_wide_kernel(const Args a)
{
    extern __shared__ float4 smem4[];
    float *Ks = reinterpret_cast<float *>(smem4);
    S2_WIDE_IDS(a.Wo)
    float *Vs = Ks + a.tile_rows * LS;
    const int ho = a.gorder[a.row_first + rowsel];
    const T *kx = static_cast<const T *>(a.k);
    const T *vx = static_cast<const T *>(a.v);
    const T *qy = static_cast<const T *>(a.q);
    T *y = static_cast<T *>(a.y);

    stage_rows<T, PT, VEC, WNT>(Ks, qy + query_point(a, b, ho, ho / a.qps) * ldk + (long)h * a.dk_, ldk * a.qps, a.dk_, w0, a.Wo, nvalid, tid);
    __syncthreads();
    float qr[32], acc[32];
#pragma unroll
    for (int c = 0; c < 32; c++) {
        qr[c] = Ks[qi * LS + sl * 32 + c] * LOG2E;
        acc[c] = 0.f;
    }
    float m = NEG_BIG, S = 0.f;

    for (int ri = a.goff[ho]; ri < a.goff[ho + 1]; ri++) {
        const Run run = a.gruns[ri];
        const float w = a.quad_w[run.pad];
        const T *kl = kx + key_point(a, b, run.lat, run.pad) * ldk + (long)h * a.dk_;
        const T *vl = vx + key_point(a, b, run.lat, run.pad) * ldv + (long)h * a.dv_;
        for (int T0 = 0; T0 < run.len; T0 += TSW) {
            const int LT = min(TSW, run.len - T0);
            const int c0 = (run.ws + T0 + w0) % a.Wi;
            const int nrows = nvalid - 1 + LT;
            __syncthreads();
            stage_rows<T, PT, VEC, WNT>(Ks, kl, ldk * a.kps, a.dk_, c0, a.Wi, nrows, tid);
            stage_rows<T, PT, VEC, WNT>(Vs, vl, ldv * a.kps, a.dv_, c0, a.Wi, nrows, tid);
            __syncthreads();
            // this wavefront's share of the chunk: neighbors wv * share .. tend - 1, TL at a time
            const int share = (LT + WNW - 1) / WNW;
            const int tend = min(LT, (wv + 1) * share);
          for (int t0 = wv * share; t0 < tend; t0 += TL) {
            const int L = min(TL, tend - t0);
            const float *krow = Ks + (qi + t0) * LS + sl * 32;
            const float *vrow = Vs + (qi + t0) * LS + sl * 32;
            float s[TL];
            float cm = NEG_BIG;
#pragma unroll
            for (int t = 0; t < TL; t++) {
                s[t] = NEG_BIG;
                if (t < L) {
                    s[t] = slice_sum<LPQ>(dot_row<32>(qr, krow + t * LS));
                    cm = fmaxf(cm, s[t]);
                }
            }
            const float mn = fmaxf(m, cm);
            const float corr = fast_exp2(m - mn);
            m = mn;
            S *= corr;
#pragma unroll
            for (int c = 0; c < 32; c++) acc[c] *= corr;
#pragma unroll
            for (int t = 0; t < TL; t++) {
                if (t < L) {
                    const float p = fast_exp2(s[t] - mn) * w;
                    S += p;
                    const float *vr = vrow + t * LS;
#pragma unroll
                    for (int c = 0; c < 32; c += 4) {
                        const float4 x = *reinterpret_cast<const float4 *>(vr + c);
                        acc[c + 0] = fmaf(p, x.x, acc[c + 0]);
                        acc[c + 1] = fmaf(p, x.y, acc[c + 1]);
                        acc[c + 2] = fmaf(p, x.z, acc[c + 2]);
                        acc[c + 3] = fmaf(p, x.w, acc[c + 3]);
                    }
                }
            }
          }
        }
    }
    // wavefront 0 takes in the other wavefronts' states one after the other (34 floats per lane, stored [value][lane])
    for (int ow = 1; ow < WNW; ow++) {
        __syncthreads();
        if (wv == ow) {
#pragma unroll
            for (int c = 0; c < 32; c++) Ks[c * TQ + lane] = acc[c];
            Ks[32 * TQ + lane] = m;
            Ks[33 * TQ + lane] = S;
        }
        __syncthreads();
        if (wv == 0) {
            const float mo = Ks[32 * TQ + lane];
            const float mn = fmaxf(m, mo);
            const float c0 = fast_exp2(m - mn), c1 = fast_exp2(mo - mn);
            m = mn;
            S = S * c0 + Ks[33 * TQ + lane] * c1;
#pragma unroll
            for (int c = 0; c < 32; c++) acc[c] = acc[c] * c0 + Ks[c * TQ + lane] * c1;
        }
    }
    __syncthreads();
    if (wv == 0) {
        if (a.lse && qi < nvalid && sl == 0) a.lse[((long)bh * a.Ho + ho) * a.Wo + w0 + qi] = m + fast_log2(S);
        const float inv = 1.0f / S;
#pragma unroll
        for (int c = 0; c < 32; c += 4)
            *reinterpret_cast<float4 *>(Ks + qi * LS + sl * 32 + c) = make_float4(acc[c] * inv, acc[c + 1] * inv, acc[c + 2] * inv, acc[c + 3] * inv);
    }
    __syncthreads();
    unstage_rows<T, PT, VEC, WNT>(y + query_point(a, b, ho, ho / a.qps) * ldv + (long)h * a.dv_, Ks, ldv * a.qps, a.dv_, w0, nvalid, tid);
}

template <typename T, int LPQ, bool VEC> __global__ __launch_bounds__(WNT) void dq_wide_kernel(const Args a)
{
    extern __shared__ float4 smem4[];
    float *Ks = reinterpret_cast<float *>(smem4);
    S2_WIDE_IDS(a.Wo)
    float *Vs = Ks + a.tile_rows * LS;
    const int ho = a.gorder[a.row_first + rowsel];
    const T *kx = static_cast<const T *>(a.k);
    const T *vx = static_cast<const T *>(a.v);
    const T *qy = static_cast<const T *>(a.q);
    const T *gy = static_cast<const T *>(a.dy);
    T *dq = static_cast<T *>(a.dq);

    stage_rows<T, PT, VEC, WNT>(Ks, qy + query_point(a, b, ho, ho / a.qps) * ldk + (long)h * a.dk_, ldk * a.qps, a.dk_, w0, a.Wo, nvalid, tid);
    stage_rows<T, PT, VEC, WNT>(Vs, gy + query_point(a, b, ho, ho / a.qps) * ldv + (long)h * a.dv_, ldv * a.qps, a.dv_, w0, a.Wo, nvalid, tid);
    __syncthreads();
    float qr[32], gr[32], Ak[32], Akg[32];
#pragma unroll
    for (int c = 0; c < 32; c++) {
        qr[c] = Ks[qi * LS + sl * 32 + c] * LOG2E;
        gr[c] = Vs[qi * LS + sl * 32 + c];
        Ak[c] = 0.f;
        Akg[c] = 0.f;
    }
    float m = NEG_BIG, S = 0.f, Ag = 0.f;

    for (int ri = a.goff[ho]; ri < a.goff[ho + 1]; ri++) {
        const Run run = a.gruns[ri];
        const float w = a.quad_w[run.pad];
        const T *kl = kx + key_point(a, b, run.lat, run.pad) * ldk + (long)h * a.dk_;
        const T *vl = vx + key_point(a, b, run.lat, run.pad) * ldv + (long)h * a.dv_;
        for (int T0 = 0; T0 < run.len; T0 += TSW) {
            const int LT = min(TSW, run.len - T0);
            const int c0 = (run.ws + T0 + w0) % a.Wi;
            const int nrows = nvalid - 1 + LT;
            __syncthreads();
            stage_rows<T, PT, VEC, WNT>(Ks, kl, ldk * a.kps, a.dk_, c0, a.Wi, nrows, tid);
            stage_rows<T, PT, VEC, WNT>(Vs, vl, ldv * a.kps, a.dv_, c0, a.Wi, nrows, tid);
            __syncthreads();
            const int share = (LT + WNW - 1) / WNW;
            const int tend = min(LT, (wv + 1) * share);
          for (int t0 = wv * share; t0 < tend; t0 += TL) {
            const int L = min(TL, tend - t0);
            const float *krow = Ks + (qi + t0) * LS + sl * 32;
            const float *vrow = Vs + (qi + t0) * LS + sl * 32;
            float s[TL], g[TL];
            float cm = NEG_BIG;
#pragma unroll
            for (int t = 0; t < TL; t++) {
                s[t] = NEG_BIG;
                g[t] = 0.f;
                if (t < L) {
                    s[t] = slice_sum<LPQ>(dot_row<32>(qr, krow + t * LS));
                    g[t] = slice_sum<LPQ>(dot_row<32>(gr, vrow + t * LS));
                    cm = fmaxf(cm, s[t]);
                }
            }
            const float mn = fmaxf(m, cm);
            const float corr = fast_exp2(m - mn);
            m = mn;
            S *= corr;
            Ag *= corr;
#pragma unroll
            for (int c = 0; c < 32; c++) {
                Ak[c] *= corr;
                Akg[c] *= corr;
            }
#pragma unroll
            for (int t = 0; t < TL; t++) {
                if (t < L) {
                    const float p = fast_exp2(s[t] - mn) * w;
                    const float pg = p * g[t];
                    S += p;
                    Ag += pg;
                    const float *kr = krow + t * LS;
#pragma unroll
                    for (int c = 0; c < 32; c += 4) {
                        const float4 x = *reinterpret_cast<const float4 *>(kr + c);
                        Ak[c + 0] = fmaf(p, x.x, Ak[c + 0]);
                        Ak[c + 1] = fmaf(p, x.y, Ak[c + 1]);
                        Ak[c + 2] = fmaf(p, x.z, Ak[c + 2]);
                        Ak[c + 3] = fmaf(p, x.w, Ak[c + 3]);
                        Akg[c + 0] = fmaf(pg, x.x, Akg[c + 0]);
                        Akg[c + 1] = fmaf(pg, x.y, Akg[c + 1]);
                        Akg[c + 2] = fmaf(pg, x.z, Akg[c + 2]);
                        Akg[c + 3] = fmaf(pg, x.w, Akg[c + 3]);
                    }
                }
            }
          }
        }
    }
    // wavefront 0 takes in the other wavefronts' states one after the other (67 floats per lane, stored [value][lane];
    // the K and V tiles are contiguous and together hold them)
    for (int ow = 1; ow < WNW; ow++) {
        __syncthreads();
        if (wv == ow) {
#pragma unroll
            for (int c = 0; c < 32; c++) {
                Ks[c * TQ + lane] = Ak[c];
                Ks[(32 + c) * TQ + lane] = Akg[c];
            }
            Ks[64 * TQ + lane] = m;
            Ks[65 * TQ + lane] = S;
            Ks[66 * TQ + lane] = Ag;
        }
        __syncthreads();
        if (wv == 0) {
            const float mo = Ks[64 * TQ + lane];
            const float mn = fmaxf(m, mo);
            const float c0 = fast_exp2(m - mn), c1 = fast_exp2(mo - mn);
            m = mn;
            S = S * c0 + Ks[65 * TQ + lane] * c1;
            Ag = Ag * c0 + Ks[66 * TQ + lane] * c1;
#pragma unroll
            for (int c = 0; c < 32; c++) {
                Ak[c] = Ak[c] * c0 + Ks[c * TQ + lane] * c1;
                Akg[c] = Akg[c] * c0 + Ks[(32 + c) * TQ + lane] * c1;
            }
        }
    }
    __syncthreads();
    if (wv == 0) {
        const float inv = 1.0f / S;
        const float I = Ag * inv;
        if (qi < nvalid && sl == 0) a.stats[((long)bh * a.Ho + ho) * a.Wo + w0 + qi] = make_float2(m + fast_log2(S), I);
#pragma unroll
        for (int c = 0; c < 32; c += 4)
            *reinterpret_cast<float4 *>(Ks + qi * LS + sl * 32 + c)
                = make_float4((Akg[c] - I * Ak[c]) * inv, (Akg[c + 1] - I * Ak[c + 1]) * inv, (Akg[c + 2] - I * Ak[c + 2]) * inv,
                              (Akg[c + 3] - I * Ak[c + 3]) * inv);
    }
    __syncthreads();
    unstage_rows<T, PT, VEC, WNT>(dq + query_point(a, b, ho, ho / a.qps) * ldk + (long)h * a.dk_, Ks, ldk * a.qps, a.dk_, w0, nvalid, tid);
}

template <typename T, int LPQ, bool VEC> __global__ __launch_bounds__(WNT) void dkdv_wide_kernel(const Args a)
{
    extern __shared__ float4 smem4[];
    float *Qs = reinterpret_cast<float *>(smem4);
    S2_WIDE_IDS(a.Wi)
    float *Gs = Qs + a.tile_rows * LS;
    float2 *Ss = reinterpret_cast<float2 *>(Gs + a.tile_rows * LS);
    const int hi = a.sorder[a.row_first + rowsel];
    const T *kx = static_cast<const T *>(a.k);
    const T *vx = static_cast<const T *>(a.v);
    const T *qy = static_cast<const T *>(a.q);
    const T *gy = static_cast<const T *>(a.dy);
    T *dk = static_cast<T *>(a.dk);
    T *dv = static_cast<T *>(a.dv);

    stage_rows<T, PT, VEC, WNT>(Qs, kx + key_point(a, b, hi, hi / a.kps) * ldk + (long)h * a.dk_, ldk * a.kps, a.dk_, w0, a.Wi, nvalid, tid);
    stage_rows<T, PT, VEC, WNT>(Gs, vx + key_point(a, b, hi, hi / a.kps) * ldv + (long)h * a.dv_, ldv * a.kps, a.dv_, w0, a.Wi, nvalid, tid);
    __syncthreads();
    float kr[32], vr[32], dkr[32], dvr[32];
#pragma unroll
    for (int c = 0; c < 32; c++) {
        kr[c] = Qs[qi * LS + sl * 32 + c] * LOG2E;
        vr[c] = Gs[qi * LS + sl * 32 + c];
        dkr[c] = 0.f;
        dvr[c] = 0.f;
    }
    const float w = a.quad_w[hi / a.kps];

    // Input column w0 + qi is neighbor t of output column (w0 + qi - ws - t) mod W.  A chunk covers t = u0 .. u0 + UL - 1:
    // the output columns c0 .. c0 + nvalid - 2 + UL are staged, and neighbor t = u0 + jj of lane qi sits in staged row
    // qi + UL - 1 - jj.
    for (int ri = a.soff[hi]; ri < a.soff[hi + 1]; ri++) {
        const Run run = a.sruns[ri];
        const int ho = run.lat;
        int d0 = w0 - run.ws;
        if (d0 < 0) d0 += a.Wi;
        const T *ql = qy + query_point(a, b, ho, run.pad) * ldk + (long)h * a.dk_;
        const T *gl = gy + query_point(a, b, ho, run.pad) * ldv + (long)h * a.dv_;
        const float2 *sl2 = a.stats + ((long)bh * a.Ho + ho) * a.Wo;
        for (int u0 = 0; u0 < run.len; u0 += TSW) {
            const int UL = min(TSW, run.len - u0);
            int c0 = (d0 - u0 - UL + 1) % a.Wo;
            if (c0 < 0) c0 += a.Wo;
            const int nrows = nvalid - 1 + UL;
            __syncthreads();
            stage_rows<T, PT, VEC, WNT>(Qs, ql, ldk * a.qps, a.dk_, c0, a.Wo, nrows, tid);
            stage_rows<T, PT, VEC, WNT>(Gs, gl, ldv * a.qps, a.dv_, c0, a.Wo, nrows, tid);
            for (int r = tid; r < nrows; r += WNT) {
                int col = c0 + r;
                while (col >= a.Wo) col -= a.Wo;
                Ss[r] = sl2[col];
            }
            __syncthreads();
            const int share = (UL + WNW - 1) / WNW;
            const int jend = min(UL, (wv + 1) * share);
          for (int j0 = wv * share; j0 < jend; j0 += TL) {
            const int L = min(TL, jend - j0);
#pragma unroll
            for (int jj = 0; jj < TL; jj++) {
                if (jj < L) {
                    const int row = qi + (UL - 1 - j0 - jj);
                    const float *qrow = Qs + row * LS + sl * 32;
                    const float *grow = Gs + row * LS + sl * 32;
                    const float s = slice_sum<LPQ>(dot_row<32>(kr, qrow));
                    const float g = slice_sum<LPQ>(dot_row<32>(vr, grow));
                    const float2 st = Ss[row];
                    const float p = fast_exp2(s - st.x) * w;
                    const float coef = p * (g - st.y);
#pragma unroll
                    for (int c = 0; c < 32; c += 4) {
                        const float4 x = *reinterpret_cast<const float4 *>(qrow + c);
                        const float4 z = *reinterpret_cast<const float4 *>(grow + c);
                        dkr[c + 0] = fmaf(coef, x.x, dkr[c + 0]);
                        dkr[c + 1] = fmaf(coef, x.y, dkr[c + 1]);
                        dkr[c + 2] = fmaf(coef, x.z, dkr[c + 2]);
                        dkr[c + 3] = fmaf(coef, x.w, dkr[c + 3]);
                        dvr[c + 0] = fmaf(p, z.x, dvr[c + 0]);
                        dvr[c + 1] = fmaf(p, z.y, dvr[c + 1]);
                        dvr[c + 2] = fmaf(p, z.z, dvr[c + 2]);
                        dvr[c + 3] = fmaf(p, z.w, dvr[c + 3]);
                    }
                }
            }
          }
        }
    }
    // wavefront 0 adds up the other wavefronts' sums one after the other (64 floats per lane, stored [value][lane])
    for (int ow = 1; ow < WNW; ow++) {
        __syncthreads();
        if (wv == ow) {
#pragma unroll
            for (int c = 0; c < 32; c++) {
                Qs[c * TQ + lane] = dkr[c];
                Qs[(32 + c) * TQ + lane] = dvr[c];
            }
        }
        __syncthreads();
        if (wv == 0) {
#pragma unroll
            for (int c = 0; c < 32; c++) {
                dkr[c] += Qs[c * TQ + lane];
                dvr[c] += Qs[(32 + c) * TQ + lane];
            }
        }
    }
    __syncthreads();
    if (wv == 0) {
#pragma unroll
        for (int c = 0; c < 32; c += 4) {
            *reinterpret_cast<float4 *>(Qs + qi * LS + sl * 32 + c) = make_float4(dkr[c], dkr[c + 1], dkr[c + 2], dkr[c + 3]);
            *reinterpret_cast<float4 *>(Gs + qi * LS + sl * 32 + c) = make_float4(dvr[c], dvr[c + 1], dvr[c + 2], dvr[c + 3]);
        }
    }
    __syncthreads();
    unstage_rows<T, PT, VEC, WNT>(dk + key_point(a, b, hi, hi / a.kps) * ldk + (long)h * a.dk_, Qs, ldk * a.kps, a.dk_, w0, nvalid, tid);
    unstage_rows<T, PT, VEC, WNT>(dv + key_point(a, b, hi, hi / a.kps) * ldv + (long)h * a.dv_, Gs, ldv * a.kps, a.dv_, w0, nvalid, tid);
}

// ---------------------------------------------------------------------------------
// Software-pipelined band staging (fast path: vector loads, at least one band of columns per virtual latitude).
// A band of up to TQ-1+TL grid points is fetched into registers with one 16-byte (8-byte for
// 16-bit storage) load per lane and iteration, NIT iterations, while the previous band is being
// consumed from LDS; it is written to LDS afterwards.  Lane constants: row r0 = lane / (P/4) of
// each group of RPI rows, channel offset cb = 4 * (lane % (P/4)).
// ---------------------------------------------------------------------------------
template <typename T, int P> struct Band {
    static constexpr int V4 = P / 4;
    static constexpr int RPI = TQ / V4;                       // rows fetched per iteration
    static constexpr int NIT = (TQ - 1 + TL + RPI - 1) / RPI; // iterations for the largest band
    static constexpr int LS = P + 4;
    typedef typename Vec4<T>::type raw_t;
    raw_t raw[NIT];

    // src: (batch, latitude, longitude 0, head); ld: elements between longitudes.  All NIT * RPI rows are fetched
    // (rows past the band wrap to valid longitudes and are never read back), so there is no predication; the
    // fast path requires the head dim to equal P, so every lane's channel offset is valid.
    __device__ inline void fetch(const T *src, unsigned ld, int c0, int W, int r0, int cb)
    {
        const int colA = c0 + r0;
#pragma unroll
        for (int it = 0; it < NIT; it++) {
            int col = colA + it * RPI;
            col -= (col >= W) ? W : 0;
            raw[it] = *reinterpret_cast<const raw_t *>(src + (size_t)(__umul24(col, ld) + cb));
        }
    }
    __device__ inline void commit(float *dst, int r0, int cb) const
    {
#pragma unroll
        for (int it = 0; it < NIT; it++) *reinterpret_cast<float4 *>(dst + (r0 + it * RPI) * LS + cb) = widen4(raw[it], (const T *)nullptr);
    }
};

#define S2_TILE_IDS(W_TILED)                                                   \
    const int lane = threadIdx.x;                                             \
    const int BH = a.B * a.nh;                                                \
    const int ntile = ((W_TILED) + TQ - 1) / TQ;                              \
    int id_ = blockIdx.x;                                                     \
    const int bh = id_ % BH;                                                  \
    id_ /= BH;                                                                \
    const int wt = id_ % ntile;                                               \
    const int rowsel = id_ / ntile;                                           \
    const int b = bh / a.nh, h = bh % a.nh;                                   \
    const int w0 = wt * TQ;                                                   \
    const int nvalid = min(TQ, (W_TILED)-w0);

// forward, fast path
template <typename T, int P> __global__ __launch_bounds__(TQ) void fwd_fast_kernel(const Args a)
{
    typedef Band<T, P> BandT;
    constexpr int LS = P + 4;
    constexpr int ROWS = BandT::NIT * BandT::RPI;
    extern __shared__ float4 smem4[];
    float *Ks = reinterpret_cast<float *>(smem4);
    float *Vs = Ks + ROWS * LS;

    S2_TILE_IDS(a.Wo)
    const int ho = a.gorder[a.row_first + rowsel];
    const unsigned ldk = a.nh * a.dk_, ldv = a.nh * a.dv_;
    const int r0 = lane / BandT::V4, cb = 4 * (lane % BandT::V4);

    const T *kx = static_cast<const T *>(a.k) + (size_t)b * a.Hi * a.Wi * ldk + (size_t)h * a.dk_;
    const T *vx = static_cast<const T *>(a.v) + (size_t)b * a.Hi * a.Wi * ldv + (size_t)h * a.dv_;
    const T *qy = static_cast<const T *>(a.q) + (size_t)query_point(a, b, ho, ho / a.qps) * ldk + (size_t)h * a.dk_;
    T *y = static_cast<T *>(a.y) + (size_t)query_point(a, b, ho, ho / a.qps) * ldv + (size_t)h * a.dv_;

    stage_rows<T, P, true>(Ks, qy, ldk * a.qps, a.dk_, w0, a.Wo, nvalid, lane);
    __syncthreads();
    float qr[P], acc[P];
#pragma unroll
    for (int c = 0; c < P; c++) {
        qr[c] = Ks[lane * LS + c] * LOG2E;
        acc[c] = 0.f;
    }
    float m = NEG_BIG, S = 0.f;

    int ri = a.goff[ho];
    const int rend = a.goff[ho + 1];
    int t0 = 0;
    Run run = {0, 0, 0, 0};
    BandT kb, vb;
    auto fetch = [&](const Run &rn, int t) {
        int c0 = rn.ws + t + w0;
        c0 -= (c0 >= a.Wi) ? a.Wi : 0;
        c0 -= (c0 >= a.Wi) ? a.Wi : 0;
        kb.fetch(kx + (size_t)key_row(a, rn.lat, rn.pad) * ldk, ldk * a.kps, c0, a.Wi, r0, cb);
        vb.fetch(vx + (size_t)key_row(a, rn.lat, rn.pad) * ldv, ldv * a.kps, c0, a.Wi, r0, cb);
    };
    if (ri < rend) {
        run = a.gruns[ri];
        fetch(run, 0);
    }
    __syncthreads();
    if (ri < rend) {
        kb.commit(Ks, r0, cb);
        vb.commit(Vs, r0, cb);
    }
    __syncthreads();

    while (ri < rend) {
        const int L = min(TL, run.len - t0);
        const float w = a.quad_w[run.pad];
        int nri = ri, nt0 = t0 + TL;
        Run nrun = run;
        if (nt0 >= run.len) {
            nri++;
            nt0 = 0;
            if (nri < rend) nrun = a.gruns[nri];
        }
        const bool more = nri < rend;
        if (more) fetch(nrun, nt0);

        const float *krow = Ks + lane * LS;
        const float *vrow = Vs + lane * LS;
        float s[TL];
        float cm = NEG_BIG;
#pragma unroll
        for (int t = 0; t < TL; t++) {
            s[t] = NEG_BIG;
            if (t < L) {
                s[t] = dot_row<P>(qr, krow + t * LS);
                cm = fmaxf(cm, s[t]);
            }
        }
        const float mn = fmaxf(m, cm);
        if (__any(mn > m)) {
            const float corr = fast_exp2(m - mn);
            S *= corr;
#pragma unroll
            for (int c = 0; c < P; c++) acc[c] *= corr;
        }
        m = mn;
#pragma unroll
        for (int t = 0; t < TL; t++) {
            if (t < L) {
                const float p = fast_exp2(s[t] - mn) * w;
                S += p;
                const float *vr = vrow + t * LS;
#pragma unroll
                for (int c = 0; c < P; c += 4) {
                    const float4 x = *reinterpret_cast<const float4 *>(vr + c);
                    acc[c + 0] = fmaf(p, x.x, acc[c + 0]);
                    acc[c + 1] = fmaf(p, x.y, acc[c + 1]);
                    acc[c + 2] = fmaf(p, x.z, acc[c + 2]);
                    acc[c + 3] = fmaf(p, x.w, acc[c + 3]);
                }
            }
        }
        __syncthreads();
        if (more) {
            kb.commit(Ks, r0, cb);
            vb.commit(Vs, r0, cb);
        }
        __syncthreads();
        ri = nri;
        t0 = nt0;
        run = nrun;
    }

    if (a.lse && lane < nvalid) a.lse[((size_t)bh * a.Ho + ho) * a.Wo + w0 + lane] = m + fast_log2(S);
    const float inv = 1.0f / S;
#pragma unroll
    for (int c = 0; c < P; c += 4)
        *reinterpret_cast<float4 *>(Ks + lane * LS + c) = make_float4(acc[c] * inv, acc[c + 1] * inv, acc[c + 2] * inv, acc[c + 3] * inv);
    __syncthreads();
    unstage_rows<T, P, true>(y, Ks, ldv * a.qps, a.dv_, w0, nvalid, lane);
}

// backward dq + statistics, fast path
template <typename T, int P> __global__ __launch_bounds__(TQ) void dq_fast_kernel(const Args a)
{
    typedef Band<T, P> BandT;
    constexpr int LS = P + 4;
    constexpr int ROWS = BandT::NIT * BandT::RPI;
    extern __shared__ float4 smem4[];
    float *Ks = reinterpret_cast<float *>(smem4);
    float *Vs = Ks + ROWS * LS;

    S2_TILE_IDS(a.Wo)
    const int ho = a.gorder[a.row_first + rowsel];
    const unsigned ldk = a.nh * a.dk_, ldv = a.nh * a.dv_;
    const int r0 = lane / BandT::V4, cb = 4 * (lane % BandT::V4);

    const T *kx = static_cast<const T *>(a.k) + (size_t)b * a.Hi * a.Wi * ldk + (size_t)h * a.dk_;
    const T *vx = static_cast<const T *>(a.v) + (size_t)b * a.Hi * a.Wi * ldv + (size_t)h * a.dv_;
    const T *qy = static_cast<const T *>(a.q) + (size_t)query_point(a, b, ho, ho / a.qps) * ldk + (size_t)h * a.dk_;
    const T *gy = static_cast<const T *>(a.dy) + (size_t)query_point(a, b, ho, ho / a.qps) * ldv + (size_t)h * a.dv_;
    T *dq = static_cast<T *>(a.dq) + (size_t)query_point(a, b, ho, ho / a.qps) * ldk + (size_t)h * a.dk_;

    stage_rows<T, P, true>(Ks, qy, ldk * a.qps, a.dk_, w0, a.Wo, nvalid, lane);
    stage_rows<T, P, true>(Vs, gy, ldv * a.qps, a.dv_, w0, a.Wo, nvalid, lane);
    __syncthreads();
    float qr[P], gr[P], Ak[P], Akg[P];
#pragma unroll
    for (int c = 0; c < P; c++) {
        qr[c] = Ks[lane * LS + c] * LOG2E;
        gr[c] = Vs[lane * LS + c];
        Ak[c] = 0.f;
        Akg[c] = 0.f;
    }
    float m = NEG_BIG, S = 0.f, Ag = 0.f;

    int ri = a.goff[ho];
    const int rend = a.goff[ho + 1];
    int t0 = 0;
    Run run = {0, 0, 0, 0};
    BandT kb, vb;
    auto fetch = [&](const Run &rn, int t) {
        int c0 = rn.ws + t + w0;
        c0 -= (c0 >= a.Wi) ? a.Wi : 0;
        c0 -= (c0 >= a.Wi) ? a.Wi : 0;
        kb.fetch(kx + (size_t)key_row(a, rn.lat, rn.pad) * ldk, ldk * a.kps, c0, a.Wi, r0, cb);
        vb.fetch(vx + (size_t)key_row(a, rn.lat, rn.pad) * ldv, ldv * a.kps, c0, a.Wi, r0, cb);
    };
    if (ri < rend) {
        run = a.gruns[ri];
        fetch(run, 0);
    }
    __syncthreads();
    if (ri < rend) {
        kb.commit(Ks, r0, cb);
        vb.commit(Vs, r0, cb);
    }
    __syncthreads();

    while (ri < rend) {
        const int L = min(TL, run.len - t0);
        const float w = a.quad_w[run.pad];
        int nri = ri, nt0 = t0 + TL;
        Run nrun = run;
        if (nt0 >= run.len) {
            nri++;
            nt0 = 0;
            if (nri < rend) nrun = a.gruns[nri];
        }
        const bool more = nri < rend;
        if (more) fetch(nrun, nt0);

        const float *krow = Ks + lane * LS;
        const float *vrow = Vs + lane * LS;
        float s[TL], g[TL];
        float cm = NEG_BIG;
#pragma unroll
        for (int t = 0; t < TL; t++) {
            s[t] = NEG_BIG;
            g[t] = 0.f;
            if (t < L) {
                s[t] = dot_row<P>(qr, krow + t * LS);
                g[t] = dot_row<P>(gr, vrow + t * LS);
                cm = fmaxf(cm, s[t]);
            }
        }
        const float mn = fmaxf(m, cm);
        if (__any(mn > m)) {
            const float corr = fast_exp2(m - mn);
            S *= corr;
            Ag *= corr;
#pragma unroll
            for (int c = 0; c < P; c++) {
                Ak[c] *= corr;
                Akg[c] *= corr;
            }
        }
        m = mn;
#pragma unroll
        for (int t = 0; t < TL; t++) {
            if (t < L) {
                const float p = fast_exp2(s[t] - mn) * w;
                const float pg = p * g[t];
                S += p;
                Ag += pg;
                const float *kr = krow + t * LS;
#pragma unroll
                for (int c = 0; c < P; c += 4) {
                    const float4 x = *reinterpret_cast<const float4 *>(kr + c);
                    Ak[c + 0] = fmaf(p, x.x, Ak[c + 0]);
                    Ak[c + 1] = fmaf(p, x.y, Ak[c + 1]);
                    Ak[c + 2] = fmaf(p, x.z, Ak[c + 2]);
                    Ak[c + 3] = fmaf(p, x.w, Ak[c + 3]);
                    Akg[c + 0] = fmaf(pg, x.x, Akg[c + 0]);
                    Akg[c + 1] = fmaf(pg, x.y, Akg[c + 1]);
                    Akg[c + 2] = fmaf(pg, x.z, Akg[c + 2]);
                    Akg[c + 3] = fmaf(pg, x.w, Akg[c + 3]);
                }
            }
        }
        __syncthreads();
        if (more) {
            kb.commit(Ks, r0, cb);
            vb.commit(Vs, r0, cb);
        }
        __syncthreads();
        ri = nri;
        t0 = nt0;
        run = nrun;
    }

    const float inv = 1.0f / S;
    const float I = Ag * inv;
    if (lane < nvalid) a.stats[((size_t)bh * a.Ho + ho) * a.Wo + w0 + lane] = make_float2(m + fast_log2(S), I);
#pragma unroll
    for (int c = 0; c < P; c += 4)
        *reinterpret_cast<float4 *>(Ks + lane * LS + c)
            = make_float4((Akg[c] - I * Ak[c]) * inv, (Akg[c + 1] - I * Ak[c + 1]) * inv, (Akg[c + 2] - I * Ak[c + 2]) * inv,
                          (Akg[c + 3] - I * Ak[c + 3]) * inv);
    __syncthreads();
    unstage_rows<T, P, true>(dq, Ks, ldk * a.qps, a.dk_, w0, nvalid, lane);
}

// backward dk/dv, fast path (the queries that see input longitude wi through run (ho, ws, len)
// are wo = wi - ws - t, t in [0, len))
template <typename T, int P> __global__ __launch_bounds__(TQ) void dkdv_fast_kernel(const Args a)
{
    typedef Band<T, P> BandT;
    constexpr int LS = P + 4;
    constexpr int ROWS = BandT::NIT * BandT::RPI;
    extern __shared__ float4 smem4[];
    float *Qs = reinterpret_cast<float *>(smem4);
    float *Gs = Qs + ROWS * LS;
    float2 *Ss = reinterpret_cast<float2 *>(Gs + ROWS * LS);

    S2_TILE_IDS(a.Wi)
    const int hi = a.sorder[a.row_first + rowsel];
    const unsigned ldk = a.nh * a.dk_, ldv = a.nh * a.dv_;
    const int r0 = lane / BandT::V4, cb = 4 * (lane % BandT::V4);

    const size_t kpt = (size_t)key_point(a, b, hi, hi / a.kps);
    const T *kx = static_cast<const T *>(a.k) + kpt * ldk + (size_t)h * a.dk_;
    const T *vx = static_cast<const T *>(a.v) + kpt * ldv + (size_t)h * a.dv_;
    const T *qy = static_cast<const T *>(a.q) + (size_t)b * a.Ho * a.Wo * ldk + (size_t)h * a.dk_;
    const T *gy = static_cast<const T *>(a.dy) + (size_t)b * a.Ho * a.Wo * ldv + (size_t)h * a.dv_;
    const float2 *stats = a.stats + (size_t)bh * a.Ho * a.Wo;
    T *dk = static_cast<T *>(a.dk) + kpt * ldk + (size_t)h * a.dk_;
    T *dv = static_cast<T *>(a.dv) + kpt * ldv + (size_t)h * a.dv_;

    stage_rows<T, P, true>(Qs, kx, ldk * a.kps, a.dk_, w0, a.Wi, nvalid, lane);
    stage_rows<T, P, true>(Gs, vx, ldv * a.kps, a.dv_, w0, a.Wi, nvalid, lane);
    __syncthreads();
    float kr[P], vr[P], dkr[P], dvr[P];
#pragma unroll
    for (int c = 0; c < P; c++) {
        kr[c] = Qs[lane * LS + c] * LOG2E;
        vr[c] = Gs[lane * LS + c];
        dkr[c] = 0.f;
        dvr[c] = 0.f;
    }
    const float w = a.quad_w[hi / a.kps];

    int ri = a.soff[hi];
    const int rend = a.soff[hi + 1];
    int u0 = 0;
    Run run = {0, 0, 0, 0};
    BandT qb, gb;
    float2 sraw[2];
    auto fetch = [&](const Run &rn, int u) {
        const int UL = min(TL, rn.len - u);
        int c0 = w0 - rn.ws - u - UL + 1; // first query longitude of the band, in (-2 Wo, Wo)
        c0 += (c0 < 0) ? a.Wo : 0;
        c0 += (c0 < 0) ? a.Wo : 0;
        const int nrows = nvalid - 1 + UL;
        qb.fetch(qy + (size_t)query_row(a, rn.lat, rn.pad) * ldk, ldk * a.qps, c0, a.Wo, r0, cb);
        gb.fetch(gy + (size_t)query_row(a, rn.lat, rn.pad) * ldv, ldv * a.qps, c0, a.Wo, r0, cb);
        const float2 *sl = stats + (size_t)rn.lat * a.Wo;
#pragma unroll
        for (int it = 0; it < 2; it++) {
            const int r = lane + it * TQ;
            int col = c0 + r;
            col -= (col >= a.Wo) ? a.Wo : 0;
            sraw[it] = make_float2(0.f, 0.f);
            if (r < nrows) sraw[it] = sl[col];
        }
    };
    auto commit = [&]() {
        qb.commit(Qs, r0, cb);
        gb.commit(Gs, r0, cb);
        Ss[lane] = sraw[0];
        if (lane + TQ < ROWS) Ss[lane + TQ] = sraw[1];
    };
    if (ri < rend) {
        run = a.sruns[ri];
        fetch(run, 0);
    }
    __syncthreads();
    if (ri < rend) commit();
    __syncthreads();

    while (ri < rend) {
        const int UL = min(TL, run.len - u0);
        int nri = ri, nu0 = u0 + TL;
        Run nrun = run;
        if (nu0 >= run.len) {
            nri++;
            nu0 = 0;
            if (nri < rend) nrun = a.sruns[nri];
        }
        const bool more = nri < rend;
        if (more) fetch(nrun, nu0);

#pragma unroll
        for (int j = 0; j < TL; j++) {
            if (j < UL) {
                const int row = lane + (UL - 1 - j);
                const float *qrow = Qs + row * LS;
                const float *grow = Gs + row * LS;
                const float s = dot_row<P>(kr, qrow);
                const float g = dot_row<P>(vr, grow);
                const float2 st = Ss[row];
                const float p = fast_exp2(s - st.x) * w;
                const float coef = p * (g - st.y);
#pragma unroll
                for (int c = 0; c < P; c += 4) {
                    const float4 x = *reinterpret_cast<const float4 *>(qrow + c);
                    const float4 z = *reinterpret_cast<const float4 *>(grow + c);
                    dkr[c + 0] = fmaf(coef, x.x, dkr[c + 0]);
                    dkr[c + 1] = fmaf(coef, x.y, dkr[c + 1]);
                    dkr[c + 2] = fmaf(coef, x.z, dkr[c + 2]);
                    dkr[c + 3] = fmaf(coef, x.w, dkr[c + 3]);
                    dvr[c + 0] = fmaf(p, z.x, dvr[c + 0]);
                    dvr[c + 1] = fmaf(p, z.y, dvr[c + 1]);
                    dvr[c + 2] = fmaf(p, z.z, dvr[c + 2]);
                    dvr[c + 3] = fmaf(p, z.w, dvr[c + 3]);
                }
            }
        }
        __syncthreads();
        if (more) commit();
        __syncthreads();
        ri = nri;
        u0 = nu0;
        run = nrun;
    }

#pragma unroll
    for (int c = 0; c < P; c += 4) {
        *reinterpret_cast<float4 *>(Qs + lane * LS + c) = make_float4(dkr[c], dkr[c + 1], dkr[c + 2], dkr[c + 3]);
        *reinterpret_cast<float4 *>(Gs + lane * LS + c) = make_float4(dvr[c], dvr[c + 1], dvr[c + 2], dvr[c + 3]);
    }
    __syncthreads();
    unstage_rows<T, P, true>(dk, Qs, ldk * a.kps, a.dk_, w0, nvalid, lane);
    unstage_rows<T, P, true>(dv, Gs, ldv * a.kps, a.dv_, w0, nvalid, lane);
}


// ---------------------------------------------------------------------------------
// Dense (matrix-core) kernels for latitudes whose runs are long: near the poles a query sees hundreds to thousands
// of consecutive longitudes per latitude, which is a dense 32 x 32 block problem.  fp32 MFMA (v_mfma_f32_32x32x2_f32)
// runs at twice the non-packed vector rate and keeps fp32 products and accumulation.
//
// One wavefront owns 32 consecutive longitudes (lane l: column j = l % 32, half = l / 32) and walks each run in
// tiles of 32 band positions u (query j sees u - j in [0, len)).  Register layout facts used throughout:
//   A operand: lane l supplies A[i = l % 32][k = l / 32];  B operand: lane l supplies B[k = l / 32][j = l % 32];
//   D: register v of lane l holds D[i = 8 (v / 4) + 4 (l / 32) + v % 4][j = l % 32].
// Scores are produced transposed, S^T[key][query] = K Q^T, so that a lane holds 16 keys of ITS query column: the
// softmax row statistics need one cross-half exchange, and the 16 probability registers are, unchanged, the B
// operand of the second product Y^T[channel][query] += V^T[channel][key] P^T[key][query] when MFMA step v uses the
// keys kappa(v, half) = 8 (v / 4) + 4 half + v % 4.
// ---------------------------------------------------------------------------------
typedef float f16v __attribute__((ext_vector_type(16)));
constexpr int MT = 32;        // queries and keys per tile
constexpr int MLK = 36;       // LDS row stride of the K-side tile (128-bit reads, rows 16 B-group skewed)

__device__ inline int kappa(int v, int half) { return 8 * (v / 4) + 4 * half + (v % 4); }

// Staging unit of the dense kernels: up to 40 consecutive longitudes (rows c0.., wrapping once at W) of one
// latitude/head, fetched into registers with one 16-byte load per lane per 8 rows.  Matrix-core tiles use the first
// 32 rows; the vector path for short runs uses all 40 (32 columns + up to 9 neighbors - 1).
constexpr int MR = 40;  // rows of the LDS tile
constexpr int VC = S2_VC;   // neighbors per vector-path chunk (MT - 1 + VC <= MR)
constexpr int LMIN = S2_LMIN; // runs at least this long go through the matrix cores (measured optimum on cfg3: flat between 24 and 40)
static_assert(MT - 1 + VC <= MR, "a vector chunk must fit the staged tile");
// Vector path of the forward: the running maximum m is only the reference point of the exponentials (any m gives the same
// y = sum p v / sum p), so it is moved, and the accumulators rescaled, only when a score exceeds it by more than this
// (log2 domain: probabilities stay below 2^8); after a query's first neighbor that is rare.
constexpr float RESCALE_THR = 8.0f;

template <typename T> struct Tile40 {
    typedef typename Vec4<T>::type raw_t;
    raw_t raw[5];
    // Tiles that do not cross longitude W - 1 (all but one or two per latitude) are addressed as a wave-uniform base
    // (scalar registers) plus one per-lane byte offset that never changes, so a load costs no vector instruction besides
    // itself; only the wrapping tile computes a column per lane and load.
    __device__ inline void fetch(const T *src, unsigned ld, int c0, int W, int lane, bool fifth)
    {
        const unsigned lane_off = (unsigned)(lane >> 3) * ld + 4u * (unsigned)(lane & 7);
        if (c0 + MR <= W) {
            const T *base = src + (size_t)c0 * ld;
#pragma unroll
            for (int it = 0; it < 4; it++) raw[it] = *reinterpret_cast<const raw_t *>(base + (size_t)(it * 8) * ld + lane_off);
            if (fifth) raw[4] = *reinterpret_cast<const raw_t *>(base + (size_t)32 * ld + lane_off);
            return;
        }
        const int colA = c0 + (lane >> 3), cb = 4 * (lane & 7);
#pragma unroll
        for (int it = 0; it < 4; it++) {
            int col = colA + it * 8;
            col -= (col >= W) ? W : 0;
            raw[it] = *reinterpret_cast<const raw_t *>(src + (size_t)(__umul24(col, ld) + cb));
        }
        if (fifth) {
            int col = colA + 32;
            col -= (col >= W) ? W : 0;
            raw[4] = *reinterpret_cast<const raw_t *>(src + (size_t)(__umul24(col, ld) + cb));
        }
    }
    // The 32 rows of a split tile: lane holds rows 4 (lane / 8) + it (one commit instruction then writes rows 0, 4, .. 28 + it,
    // whose LDS words tile the banks exactly; rows it * 8 + lane / 8 would collide two ways).
    __device__ inline void fetch_split(const T *src, unsigned ld, int c0, int W, int lane)
    {
        const unsigned lane_off = 4u * (unsigned)(lane >> 3) * ld + 4u * (unsigned)(lane & 7);
        if (c0 + MT <= W) {
            const T *base = src + (size_t)c0 * ld;
#pragma unroll
            for (int it = 0; it < 4; it++) raw[it] = *reinterpret_cast<const raw_t *>(base + (size_t)it * ld + lane_off);
            return;
        }
        const int colA = c0 + 4 * (lane >> 3), cb = 4 * (lane & 7);
#pragma unroll
        for (int it = 0; it < 4; it++) {
            int col = colA + it;
            col -= (col >= W) ? W : 0;
            raw[it] = *reinterpret_cast<const raw_t *>(src + (size_t)(__umul24(col, ld) + cb));
        }
    }
    __device__ inline void commit(float *dst, int lane, bool fifth) const
    {
        const int r0 = lane >> 3, cb = 4 * (lane & 7);
#pragma unroll
        for (int it = 0; it < 4; it++) *reinterpret_cast<float4 *>(dst + (r0 + it * 8) * MLK + cb) = widen4(raw[it], (const T *)nullptr);
        if (fifth) *reinterpret_cast<float4 *>(dst + (r0 + 32) * MLK + cb) = widen4(raw[4], (const T *)nullptr);
    }
};

// A run is walked either in matrix-core tiles of 32 band positions (pos = first position, len + 31 positions in all)
// or, when short, in vector chunks of VC neighbors (pos = first neighbor index).
__device__ inline bool run_is_dense(int len) { return len >= LMIN; }
__device__ inline bool run_done(int len, int next_pos) { return run_is_dense(len) ? next_pos >= len + MT - 1 : next_pos >= len; }
__device__ inline int run_stride(int len) { return run_is_dense(len) ? MT : VC; }

#define S2_MFMA_IDS(W_TILED)                                                  \
    const int lane = threadIdx.x;                                             \
    const int j = lane & 31, half = lane >> 5;                                \
    const int BH = a.B * a.nh;                                                \
    const int ntile = ((W_TILED) + MT - 1) / MT;                              \
    int id_ = blockIdx.x;                                                     \
    const int bh = id_ % BH;                                                  \
    id_ /= BH;                                                                \
    const int wt = id_ % ntile;                                               \
    const int rowsel = id_ / ntile;                                           \
    const int b = bh / a.nh, h = bh % a.nh;                                   \
    const int w0 = wt * MT;                                                   \
    const int nvalid = min(MT, (W_TILED)-w0);

#include "s2attn_pair.hpp"
#include "s2attn_split.hpp"

// forward, head dim 32.  Lane (j, half) keeps channels 8g + 4 half + e (g, e < 4) of query j: that is the
// accumulator layout of the matrix-core product, and the vector path for short runs uses the same one (each half
// computes half of a dot product, one cross-half exchange completes it).
template <typename T> __global__ __launch_bounds__(64) void fwd_mfma_kernel(const Args a)
{
    __shared__ __attribute__((aligned(16))) float Ks[MR * MLK];
    __shared__ __attribute__((aligned(16))) float Vs[MR * MLK];
    __shared__ __attribute__((aligned(16))) int Rs[8 * S2_PAIR_MAX_RUNS]; // merged runs of a latitude pair

    S2_MFMA_IDS(a.Wo)
    const int ho = a.gitems[2 * rowsel], pair = a.gitems[2 * rowsel + 1];
    if (pair >= 0) { // two adjacent short-run latitudes in one wavefront
        fwd_pair<T>(a, Ks, Vs, Rs, lane, b, h, w0, nvalid, ho, pair);
        return;
    }
    const unsigned ldk = a.ldk, ldv = a.ldv; // elements between two grid points, per tensor (packed heads, or a row of a fused buffer)
    const T *kx = static_cast<const T *>(a.k) + (size_t)b * a.Hi * a.Wi * ldk + (size_t)h * 32;
    const T *vx = static_cast<const T *>(a.v) + (size_t)b * a.Hi * a.Wi * ldv + (size_t)h * 32;
    const bool mine = j < nvalid;
    const size_t pt = (size_t)query_point(a, b, ho, ho / a.qps) + (size_t)(w0 + (mine ? j : 0)) * a.qps;

    float qb[16];
    {
        const T *qrow = static_cast<const T *>(a.q) + pt * a.ldq + (size_t)h * 32 + 4 * half;
#pragma unroll
        for (int g = 0; g < 4; g++) {
            const float4 x = load4(qrow + 8 * g);
            qb[4 * g] = x.x * LOG2E, qb[4 * g + 1] = x.y * LOG2E, qb[4 * g + 2] = x.z * LOG2E, qb[4 * g + 3] = x.w * LOG2E;
        }
    }
    f16v acc;
#pragma unroll
    for (int v = 0; v < 16; v++) acc[v] = 0.f;
    float m = NEG_BIG, S = 0.f;
    // Two-level summation on long rows (fp32 storage): every FLUSH matrix-core steps the running sums are added to a second
    // level and start again from zero, so the rounding of each addition is relative to a short partial sum and the second
    // level sees few additions (a pole row has 5,760 terms per query; summed in one chain y is off by 2-3e-6 of its size,
    // which the backward's <dy, y> turns into 2e-5 of dq).  The second level of the output sums lives in the output row
    // itself (each lane owns its 16 values of y), that of the normaliser in S2; part_scale collects the rescalings since
    // the last flush.
    constexpr bool two_level = std::is_same<T, float>::value;
    constexpr int FLUSH = 8;
    float S2 = 0.f, part_scale = 1.f;
    int nflush = 0;
    bool have_part = false;
    T *const yout = static_cast<T *>(a.y) + pt * a.ldy + (size_t)h * 32 + 4 * half;

    int ri = a.goff[ho];
    const int rend = a.goff[ho + 1];
    int pos = 0;
    Run run = {0, 0, 0, 0};
    Tile40<T> kt, vt;
    auto fetch = [&](const Run &rn, int p) {
        const int c0 = (rn.ws + w0 + p) % a.Wi;
        const bool fifth = !run_is_dense(rn.len);
        kt.fetch(kx + (size_t)key_row(a, rn.lat, rn.pad) * ldk, ldk * a.kps, c0, a.Wi, lane, fifth);
        vt.fetch(vx + (size_t)key_row(a, rn.lat, rn.pad) * ldv, ldv * a.kps, c0, a.Wi, lane, fifth);
    };
    if (ri < rend) {
        run = const_load(a.gruns + ri);
        fetch(run, 0);
        kt.commit(Ks, lane, !run_is_dense(run.len));
        vt.commit(Vs, lane, !run_is_dense(run.len));
    }
    __syncthreads();

    while (ri < rend) {
        const float w = const_load(a.quad_w + run.pad);
        const int len = run.len;
        int nri = ri, npos = pos + run_stride(len);
        Run nrun = run;
        if (run_done(len, npos)) {
            nri++;
            npos = 0;
            if (nri < rend) nrun = const_load(a.gruns + nri);
        }
        const bool more = nri < rend;
        if (more) fetch(nrun, npos);

        const float *kq = Ks + j * MLK + 4 * half; // row j, this half's channel groups at +8g
        const float *vq = Vs + j * MLK + 4 * half;
        if (run_is_dense(len)) {
            // ---- matrix-core tile: S^T = K Q^T ----
            const int u0 = pos;
            f16v sc;
#pragma unroll
            for (int v = 0; v < 16; v++) sc[v] = 0.f;
#pragma unroll
            for (int g = 0; g < 4; g++) {
                const float4 x = *reinterpret_cast<const float4 *>(kq + 8 * g);
                sc = __builtin_amdgcn_mfma_f32_32x32x2f32(x.x, qb[4 * g + 0], sc, 0, 0, 0);
                sc = __builtin_amdgcn_mfma_f32_32x32x2f32(x.y, qb[4 * g + 1], sc, 0, 0, 0);
                sc = __builtin_amdgcn_mfma_f32_32x32x2f32(x.z, qb[4 * g + 2], sc, 0, 0, 0);
                sc = __builtin_amdgcn_mfma_f32_32x32x2f32(x.w, qb[4 * g + 3], sc, 0, 0, 0);
            }
            // band mask on the first and last tiles: key position u = u0 + kappa is a neighbor of query j iff 0 <= u - j < len
            const bool edge = (u0 < MT - 1) || (u0 + MT - 1 >= len);
            if (edge) {
#pragma unroll
                for (int v = 0; v < 16; v++) {
                    const int t = u0 + kappa(v, half) - j;
                    sc[v] = (t >= 0 && t < len) ? sc[v] : NEG_BIG;
                }
            }
            float mx = sc[0];
#pragma unroll
            for (int v = 1; v < 16; v++) mx = fmaxf(mx, sc[v]);
            mx = xor32_max(mx);
            const float mn = fmaxf(m, mx);
            if (__any(mn > m)) {
                const float corr = fast_exp2(m - mn);
                S *= corr;
                S2 *= corr;
                part_scale *= corr;
#pragma unroll
                for (int v = 0; v < 16; v++) acc[v] *= corr;
            }
            m = mn;
            float rs = 0.f;
            if (edge) {
#pragma unroll
                for (int v = 0; v < 16; v++) {
                    const float p = (sc[v] == NEG_BIG) ? 0.f : fast_exp2(sc[v] - mn) * w;
                    sc[v] = p;
                    rs += p;
                }
            } else {
#pragma unroll
                for (int v = 0; v < 16; v++) {
                    const float p = fast_exp2(sc[v] - mn) * w;
                    sc[v] = p;
                    rs += p;
                }
            }
            rs = xor32_sum(rs);
            S += rs;
            // Y^T += V^T P^T
#pragma unroll
            for (int v = 0; v < 16; v++) {
                const float x = Vs[kappa(v, half) * MLK + j];
                acc = __builtin_amdgcn_mfma_f32_32x32x2f32(x, sc[v], acc, 0, 0, 0);
            }
            if (two_level && ++nflush == FLUSH) {
                if (mine) {
#pragma unroll
                    for (int g = 0; g < 4; g++) {
                        float4 o = make_float4(acc[4 * g], acc[4 * g + 1], acc[4 * g + 2], acc[4 * g + 3]);
                        if (have_part) {
                            const float4 old = load4(yout + 8 * g);
                            o.x = fmaf(old.x, part_scale, o.x), o.y = fmaf(old.y, part_scale, o.y), o.z = fmaf(old.z, part_scale, o.z), o.w = fmaf(old.w, part_scale, o.w);
                        }
                        store4(yout + 8 * g, o);
                    }
                }
#pragma unroll
                for (int v = 0; v < 16; v++) acc[v] = 0.f;
                S2 += S;
                S = 0.f;
                part_scale = 1.f;
                nflush = 0;
                have_part = true;
            }
        } else {
            // ---- vector chunk: neighbors pos .. pos + L - 1, query j reads staged rows j + t; one pass, lazy maximum ----
            const int L = min(VC, len - pos);
            // (LDS reads software-pipelined as in the pair path: K row of the next neighbor while this one's exponential and
            // accumulation run, V row while its dot product does)
            float4 x[4], z[4];
            read_row(x, kq);
#pragma unroll
            for (int t = 0; t < VC; t++) {
                if (t < L) {
                    read_row(z, vq + t * MLK);
                    const float sv = xor32_sum(dot16(qb, x));
                    __builtin_amdgcn_sched_barrier(0);
                    read_row(x, kq + (t + 1) * MLK); // (past the last neighbor: a row nobody uses, still inside the buffer)
                    __builtin_amdgcn_sched_barrier(0);
                    if (__any(sv > m + RESCALE_THR)) {
                        const float mn = sv > m + RESCALE_THR ? sv : m, corr = fast_exp2(m - mn);
                        S *= corr;
                        S2 *= corr;
                        part_scale *= corr;
#pragma unroll
                        for (int v = 0; v < 16; v++) acc[v] *= corr;
                        m = mn;
                    }
                    const float p = fast_exp2(sv - m) * w;
                    S += p;
#pragma unroll
                    for (int g = 0; g < 4; g++) {
                        acc[4 * g] = fmaf(p, z[g].x, acc[4 * g]);
                        acc[4 * g + 1] = fmaf(p, z[g].y, acc[4 * g + 1]);
                        acc[4 * g + 2] = fmaf(p, z[g].z, acc[4 * g + 2]);
                        acc[4 * g + 3] = fmaf(p, z[g].w, acc[4 * g + 3]);
                    }
                }
            }
        }

        __syncthreads();
        if (more) {
            kt.commit(Ks, lane, !run_is_dense(nrun.len));
            vt.commit(Vs, lane, !run_is_dense(nrun.len));
        }
        __syncthreads();
        ri = nri;
        pos = npos;
        run = nrun;
    }

    if (mine) {
        if (two_level && have_part) {
#pragma unroll
            for (int g = 0; g < 4; g++) {
                const float4 old = load4(yout + 8 * g);
                acc[4 * g] = fmaf(old.x, part_scale, acc[4 * g]), acc[4 * g + 1] = fmaf(old.y, part_scale, acc[4 * g + 1]);
                acc[4 * g + 2] = fmaf(old.z, part_scale, acc[4 * g + 2]), acc[4 * g + 3] = fmaf(old.w, part_scale, acc[4 * g + 3]);
            }
            S += S2;
        }
        if (a.lse && half == 0) a.lse[((size_t)bh * a.Ho + ho) * a.Wo + w0 + j] = m + fast_log2(S);
        const float inv = 1.0f / S;
#pragma unroll
        for (int g = 0; g < 4; g++) store4(yout + 8 * g, make_float4(acc[4 * g] * inv, acc[4 * g + 1] * inv, acc[4 * g + 2] * inv, acc[4 * g + 3] * inv));
    }
}

// backward dq from saved forward statistics: with lse = log2 sum_j a_j known per query and I = <dy, y>, the softmax is
// final from the first neighbor on, p_j = exp2(s_j - lse) w_j, and dq = sum_j p_j (g_j - I) k_j needs three matrix
// products per tile (S^T, G^T, dQ^T += K^T C^T) and no running maximum or rescaling.
template <typename T> __global__ __launch_bounds__(64) void dq_saved_mfma_kernel(const Args a)
{
    __shared__ __attribute__((aligned(16))) float Ks[MR * MLK];
    __shared__ __attribute__((aligned(16))) float Vs[MR * MLK];

    S2_MFMA_IDS(a.Wo)
    // One latitude per workgroup row, long-run and short-run latitudes interleaved.  (No latitude pairs in this pass: a lane
    // holding q, dy and dq of two latitudes plus the tile prefetch costs the third resident wavefront per SIMD, which the
    // matrix-core path of the same kernel needs more than the short rows need the shared LDS reads.)
    const int ho = a.gorder_mixed[rowsel];
    const unsigned ldk = a.ldk, ldv = a.ldv;
    const T *kx = static_cast<const T *>(a.k) + (size_t)b * a.Hi * a.Wi * ldk + (size_t)h * 32;
    const T *vx = static_cast<const T *>(a.v) + (size_t)b * a.Hi * a.Wi * ldv + (size_t)h * 32;
    const bool mine = j < nvalid;
    const size_t pt = (size_t)query_point(a, b, ho, ho / a.qps) + (size_t)(w0 + (mine ? j : 0)) * a.qps;
    const size_t sidx = ((size_t)bh * a.Ho + ho) * a.Wo + w0 + (mine ? j : 0);

    // The loads of this point's q, dy and y rows are issued here; what is computed from them (I = <dy, y>, which waits for
    // them) comes after the first tile's loads have been issued too, so that the wavefront starts with one memory round trip
    // instead of two in a row.
    float qb[16], gb[16];
    float4 yv[4];
    {
        const T *qrow = static_cast<const T *>(a.q) + pt * a.ldq + (size_t)h * 32 + 4 * half;
        const T *grow = static_cast<const T *>(a.dy) + pt * a.ldg + (size_t)h * 32 + 4 * half;
        const T *yrow = static_cast<const T *>(a.ysaved) + pt * a.ldy + (size_t)h * 32 + 4 * half;
#pragma unroll
        for (int g = 0; g < 4; g++) {
            const float4 x = load4(qrow + 8 * g);
            const float4 z = load4(grow + 8 * g);
            yv[g] = load4(yrow + 8 * g);
            qb[4 * g] = x.x, qb[4 * g + 1] = x.y, qb[4 * g + 2] = x.z, qb[4 * g + 3] = x.w;
            gb[4 * g] = z.x, gb[4 * g + 1] = z.y, gb[4 * g + 2] = z.z, gb[4 * g + 3] = z.w;
        }
    }
    float lse = a.lse[sidx];
    f16v dqt;
#pragma unroll
    for (int v = 0; v < 16; v++) dqt[v] = 0.f;

    int ri = a.goff[ho];
    const int rend = a.goff[ho + 1];
    int pos = 0;
    Run run = {0, 0, 0, 0};
    Tile40<T> kt, vt;
    auto fetch = [&](const Run &rn, int p) {
        const int c0 = (rn.ws + w0 + p) % a.Wi;
        const bool fifth = !run_is_dense(rn.len);
        kt.fetch(kx + (size_t)key_row(a, rn.lat, rn.pad) * ldk, ldk * a.kps, c0, a.Wi, lane, fifth);
        vt.fetch(vx + (size_t)key_row(a, rn.lat, rn.pad) * ldv, ldv * a.kps, c0, a.Wi, lane, fifth);
    };
    if (ri < rend) {
        run = a.gruns[ri];
        fetch(run, 0);
    }
    __builtin_amdgcn_sched_barrier(0);
    float I = 0.f;
#pragma unroll
    for (int g = 0; g < 4; g++) {
        I = fmaf(gb[4 * g], yv[g].x, I);
        I = fmaf(gb[4 * g + 1], yv[g].y, I);
        I = fmaf(gb[4 * g + 2], yv[g].z, I);
        I = fmaf(gb[4 * g + 3], yv[g].w, I);
    }
    I = xor32_sum(I);
#pragma unroll
    for (int v = 0; v < 16; v++) qb[v] *= LOG2E;
    if (ri < rend) {
        kt.commit(Ks, lane, !run_is_dense(run.len));
        vt.commit(Vs, lane, !run_is_dense(run.len));
    }
    __syncthreads();
    settle(qb);
    settle(gb);
    settle(lse);

    // Run descriptors and quadrature weights are read a run ahead of their use (`ahead` is the run after `run`, `w` arrives
    // with the run it belongs to): a scalar load at the top of the loop would be waited for right there, in front of the
    // addresses of the next tile's loads, on every short run.
    Run ahead = run;
    float w = 0.f;
    if (ri < rend) w = a.quad_w[run.pad];
    if (ri + 1 < rend) ahead = a.gruns[ri + 1];
    while (ri < rend) {
        const int len = run.len;
        int nri = ri, npos = pos + run_stride(len);
        Run nrun = run;
        const bool adv = run_done(len, npos);
        if (adv) {
            nri++;
            npos = 0;
            if (nri < rend) nrun = ahead;
        }
        const bool more = nri < rend;
        if (more) fetch(nrun, npos);
        Run ahead2 = ahead;
        float wn = w;
        if (adv && more) {
            wn = a.quad_w[nrun.pad];
            if (nri + 1 < rend) ahead2 = a.gruns[nri + 1];
        }

        const float *kq = Ks + j * MLK + 4 * half;
        const float *vq = Vs + j * MLK + 4 * half;
        if (run_is_dense(len)) {
            const int u0 = pos;
            f16v sc, gc;
#pragma unroll
            for (int v = 0; v < 16; v++) {
                sc[v] = 0.f;
                gc[v] = 0.f;
            }
#pragma unroll
            for (int g = 0; g < 4; g++) {
                const float4 x = *reinterpret_cast<const float4 *>(kq + 8 * g);
                const float4 z = *reinterpret_cast<const float4 *>(vq + 8 * g);
                sc = __builtin_amdgcn_mfma_f32_32x32x2f32(x.x, qb[4 * g + 0], sc, 0, 0, 0);
                gc = __builtin_amdgcn_mfma_f32_32x32x2f32(z.x, gb[4 * g + 0], gc, 0, 0, 0);
                sc = __builtin_amdgcn_mfma_f32_32x32x2f32(x.y, qb[4 * g + 1], sc, 0, 0, 0);
                gc = __builtin_amdgcn_mfma_f32_32x32x2f32(z.y, gb[4 * g + 1], gc, 0, 0, 0);
                sc = __builtin_amdgcn_mfma_f32_32x32x2f32(x.z, qb[4 * g + 2], sc, 0, 0, 0);
                gc = __builtin_amdgcn_mfma_f32_32x32x2f32(z.z, gb[4 * g + 2], gc, 0, 0, 0);
                sc = __builtin_amdgcn_mfma_f32_32x32x2f32(x.w, qb[4 * g + 3], sc, 0, 0, 0);
                gc = __builtin_amdgcn_mfma_f32_32x32x2f32(z.w, gb[4 * g + 3], gc, 0, 0, 0);
            }
            const bool edge = (u0 < MT - 1) || (u0 + MT - 1 >= len);
            if (edge) {
#pragma unroll
                for (int v = 0; v < 16; v++) {
                    const int t = u0 + kappa(v, half) - j;
                    const float p = (t >= 0 && t < len) ? fast_exp2(sc[v] - lse) * w : 0.f;
                    sc[v] = p * (gc[v] - I);
                }
            } else {
#pragma unroll
                for (int v = 0; v < 16; v++) sc[v] = fast_exp2(sc[v] - lse) * w * (gc[v] - I);
            }
#pragma unroll
            for (int v = 0; v < 16; v++) {
                const float x = Ks[kappa(v, half) * MLK + j];
                dqt = __builtin_amdgcn_mfma_f32_32x32x2f32(x, sc[v], dqt, 0, 0, 0);
            }
        } else {
            const int L = min(VC, len - pos);
#pragma unroll
            for (int t = 0; t < VC; t++) {
                if (t < L) {
                    float4 xk[4], zv[4];
                    read_row(xk, kq + t * MLK);
                    read_row(zv, vq + t * MLK);
                    const float sv = xor32_sum(dot16(qb, xk));
                    const float gv = xor32_sum(dot16(gb, zv));
                    const float coef = fast_exp2(sv - lse) * w * (gv - I);
#pragma unroll
                    for (int g = 0; g < 4; g++) {
                        dqt[4 * g] = fmaf(coef, xk[g].x, dqt[4 * g]);
                        dqt[4 * g + 1] = fmaf(coef, xk[g].y, dqt[4 * g + 1]);
                        dqt[4 * g + 2] = fmaf(coef, xk[g].z, dqt[4 * g + 2]);
                        dqt[4 * g + 3] = fmaf(coef, xk[g].w, dqt[4 * g + 3]);
                    }
                }
            }
        }

        __syncthreads();
        if (more) {
            kt.commit(Ks, lane, !run_is_dense(nrun.len));
            vt.commit(Vs, lane, !run_is_dense(nrun.len));
        }
        __syncthreads();
        ri = nri;
        pos = npos;
        run = nrun;
        ahead = ahead2;
        w = wn;
    }

    // (stored after the walk: a global store ahead of the loop would turn the loop's scalar loads of runs and weights,
    // which the compiler only uses while nothing in the kernel can have written memory, into vector loads with waits)
    if (mine && half == 0) a.stats[sidx] = make_float2(lse, I);
    if (mine) {
        T *dq = static_cast<T *>(a.dq) + pt * a.lddq + (size_t)h * 32 + 4 * half;
#pragma unroll
        for (int g = 0; g < 4; g++) store4(dq + 8 * g, make_float4(dqt[4 * g], dqt[4 * g + 1], dqt[4 * g + 2], dqt[4 * g + 3]));
    }
}


// backward dk/dv: lane (j, half) owns INPUT longitude j of the tile, channels 8g + 4 half + e.  For a run (ho, ws, len)
// the queries that see the tile's keys are the len + 31 longitudes starting at w0 - ws - len + 1; query row r sees key j
// iff 0 <= r - j < len.  Matrix-core tile of 32 query rows:  S = Q K^T and G = dY V^T come out as [query][key] (a lane
// holds 16 queries of ITS key column), P = exp2(S - lse_query) w, C = P (G - I_query), then dK^T += Q^T C and
// dV^T += dY^T P.  Short runs: vector chunks of VC query rows starting at row pos, key j reads staged rows j + i.
template <typename T> __global__ __launch_bounds__(64) void dkdv_mfma_kernel(const Args a)
{
    // fp32 tiles of 40 rows for vector chunks (and the merged runs of a latitude pair behind them), or split tiles of 32 rows for
    // matrix-core steps, in one buffer (see the forward); the statistics of the staged rows behind it
    __shared__ __attribute__((aligned(16))) char smem[2 * SPLIT_TILE_BYTES + 2 * MR * 4];
    float *const Qs = reinterpret_cast<float *>(smem), *const Gs = Qs + MR * MLK;
    int *const Rs = reinterpret_cast<int *>(Gs + MR * MLK);
    char *const Qb = smem, *const Gb = smem + SPLIT_TILE_BYTES;
    float *const Ls = reinterpret_cast<float *>(smem + 2 * SPLIT_TILE_BYTES), *const Is = Ls + MR;

    S2_MFMA_IDS(a.Wi)
    const int hi = a.sitems[2 * rowsel], pair = a.sitems[2 * rowsel + 1];
    if (pair >= 0) {
        dkdv_pair<T>(a, Qs, Gs, Ls, Is, Rs, lane, b, h, w0, nvalid, hi, pair);
        return;
    }
    const unsigned ldq = a.ldq, ldg = a.ldg;
    const T *qy = static_cast<const T *>(a.q) + (size_t)b * a.Ho * a.Wo * ldq + (size_t)h * 32;
    const T *gy = static_cast<const T *>(a.dy) + (size_t)b * a.Ho * a.Wo * ldg + (size_t)h * 32;
    const float2 *stats = a.stats + (size_t)bh * a.Ho * a.Wo;
    const bool mine = j < nvalid;
    const size_t pt = (size_t)key_point(a, b, hi, hi / a.kps) + (size_t)(w0 + (mine ? j : 0)) * a.kps;

    // k (times log2 e) and v in the form the current run needs, one set of registers each (OwnRegs, see the forward)
    OwnRegs ko, vo;
    bool own_split = false;
    const T *const krow = static_cast<const T *>(a.k) + pt * a.ldk + (size_t)h * 32 + 4 * half;
    const T *const vrow = static_cast<const T *>(a.v) + pt * a.ldv + (size_t)h * 32 + 4 * half;
    f16v dkt, dvt;
#pragma unroll
    for (int v = 0; v < 16; v++) {
        dkt[v] = 0.f;
        dvt[v] = 0.f;
    }
    const float w = a.quad_w[hi / a.kps];

    int ri = a.soff[hi];
    const int rend = a.soff[hi + 1];
    int pos = 0;
    Run run = {0, 0, 0, 0};
    Tile40<T> qt, gt;
    float2 st = make_float2(0.f, 0.f);
    auto fetch = [&](const Run &rn, int p) {
        int c0 = (w0 - rn.ws - rn.len + 1 + p) % a.Wo; // longitude of staged row 0
        c0 += (c0 < 0) ? a.Wo : 0;
        if (run_is_dense(rn.len)) {
            qt.fetch_split(qy + (size_t)query_row(a, rn.lat, rn.pad) * ldq, ldq * a.qps, c0, a.Wo, lane);
            gt.fetch_split(gy + (size_t)query_row(a, rn.lat, rn.pad) * ldg, ldg * a.qps, c0, a.Wo, lane);
        } else {
            qt.fetch(qy + (size_t)query_row(a, rn.lat, rn.pad) * ldq, ldq * a.qps, c0, a.Wo, lane, true);
            gt.fetch(gy + (size_t)query_row(a, rn.lat, rn.pad) * ldg, ldg * a.qps, c0, a.Wo, lane, true);
        }
        int col = c0 + lane; // lanes 0..39 fetch the statistics of the staged rows
        col -= (col >= a.Wo) ? a.Wo : 0;
        if (lane < MR) st = stats[(size_t)rn.lat * a.Wo + col];
    };
    auto commit = [&](bool dense) {
        if (dense) {
            commit_split(qt, Qb, lane);
            commit_split(gt, Gb, lane);
        } else {
            qt.commit(Qs, lane, true);
            gt.commit(Gs, lane, true);
        }
        if (lane < MR) {
            Ls[lane] = st.x;
            Is[lane] = st.y;
        }
    };
    if (ri < rend) {
        run = a.sruns[ri];
        fetch(run, 0);
        commit(run_is_dense(run.len));
    }
    own_split = ri < rend && run_is_dense(run.len);
    ko.load(krow, LOG2E, own_split);
    vo.load(vrow, 1.0f, own_split);
    __syncthreads();
    settle(ko.r);
    settle(vo.r);
    const int troff = tr_lane_offset(lane);

    while (ri < rend) {
        const int len = run.len;
        if (run_is_dense(len) != own_split) {
            own_split = run_is_dense(len);
            ko.load(krow, LOG2E, own_split);
            vo.load(vrow, 1.0f, own_split);
        }
        int nri = ri, npos = pos + run_stride(len);
        Run nrun = run;
        if (run_done(len, npos)) {
            nri++;
            npos = 0;
            if (nri < rend) nrun = a.sruns[nri];
        }
        const bool more = nri < rend;
        if (more) fetch(nrun, npos);

        const float *qq = Qs + j * MLK + 4 * half;
        const float *gq = Gs + j * MLK + 4 * half;
        if (run_is_dense(len)) {
            const int r0 = pos;
            f16v sc, gc;
#pragma unroll
            for (int v = 0; v < 16; v++) {
                sc[v] = 0.f;
                gc[v] = 0.f;
            }
            sc = rows_times_regs(Qb + j * SPP + 32 * half, ko.terms(), sc);
            gc = rows_times_regs(Gb + j * SPP + 32 * half, vo.terms(), gc);
            const bool edge = (r0 < MT - 1) || (r0 + MT - 1 >= len);
#pragma unroll
            for (int g = 0; g < 4; g++) {
                const float4 l4 = *reinterpret_cast<const float4 *>(Ls + 8 * g + 4 * half);
                const float4 i4 = *reinterpret_cast<const float4 *>(Is + 8 * g + 4 * half);
                const float lv[4] = {l4.x, l4.y, l4.z, l4.w};
                const float iv[4] = {i4.x, i4.y, i4.z, i4.w};
#pragma unroll
                for (int e = 0; e < 4; e++) {
                    const int v = 4 * g + e;
                    float p = fast_exp2(sc[v] - lv[e]) * w;
                    if (edge) {
                        const int t = r0 + kappa(v, half) - j;
                        p = (t >= 0 && t < len) ? p : 0.f;
                    }
                    sc[v] = p;
                    gc[v] = p * (gc[v] - iv[e]);
                }
            }
            {
                Terms3 cs;
                split_regs(cs, gc);
                dkt = cols_times_regs(Qb, troff, cs, dkt);
            }
            {
                Terms3 ps;
                split_regs(ps, sc);
                dvt = cols_times_regs(Gb, troff, ps, dvt);
            }
        } else {
            const int L = min(VC, len - pos);
            float kb[16], vb[16];
            ko.floats(kb);
            vo.floats(vb);
#pragma unroll
            for (int i = 0; i < VC; i++) {
                if (i < L) {
                    float4 xq[4], xg[4];
                    read_row(xq, qq + i * MLK);
                    read_row(xg, gq + i * MLK);
                    const float s = xor32_sum(dot16(kb, xq));
                    const float gd = xor32_sum(dot16(vb, xg));
                    const float p = fast_exp2(s - Ls[j + i]) * w;
                    const float coef = p * (gd - Is[j + i]);
#pragma unroll
                    for (int g = 0; g < 4; g++) {
                        dkt[4 * g] = fmaf(coef, xq[g].x, dkt[4 * g]);
                        dkt[4 * g + 1] = fmaf(coef, xq[g].y, dkt[4 * g + 1]);
                        dkt[4 * g + 2] = fmaf(coef, xq[g].z, dkt[4 * g + 2]);
                        dkt[4 * g + 3] = fmaf(coef, xq[g].w, dkt[4 * g + 3]);
                        dvt[4 * g] = fmaf(p, xg[g].x, dvt[4 * g]);
                        dvt[4 * g + 1] = fmaf(p, xg[g].y, dvt[4 * g + 1]);
                        dvt[4 * g + 2] = fmaf(p, xg[g].z, dvt[4 * g + 2]);
                        dvt[4 * g + 3] = fmaf(p, xg[g].w, dvt[4 * g + 3]);
                    }
                }
            }
        }

        __syncthreads();
        if (more) commit(run_is_dense(nrun.len));
        __syncthreads();
        ri = nri;
        pos = npos;
        run = nrun;
    }

    if (mine) {
        T *dk = static_cast<T *>(a.dk) + pt * a.lddk + (size_t)h * 32 + 4 * half;
        T *dv = static_cast<T *>(a.dv) + pt * a.lddv + (size_t)h * 32 + 4 * half;
#pragma unroll
        for (int g = 0; g < 4; g++) {
            store4(dk + 8 * g, make_float4(dkt[4 * g], dkt[4 * g + 1], dkt[4 * g + 2], dkt[4 * g + 3]));
            store4(dv + 8 * g, make_float4(dvt[4 * g], dvt[4 * g + 1], dvt[4 * g + 2], dvt[4 * g + 3]));
        }
    }
}

#include "s2attn_h16.hpp"
#include "s2attn_m32.hpp"

// ---------------------------------------------------------------------------------
// layout permutes: batched 2-D transpose [R, S] -> [S, R] through a 64x65 LDS tile
// ---------------------------------------------------------------------------------
// The grid is one-dimensional (a grid's y and z extents stop at 65535, and H*W/64 passes that on fine grids): workgroup
// id = (batch * gy + row tile) * gx + column tile.
template <typename E> __global__ __launch_bounds__(256) void transpose_kernel(const E *__restrict__ src, E *__restrict__ dst, long R, long S, unsigned gx, unsigned gy)
{
    __shared__ E tile[64][65];
    const unsigned bx = blockIdx.x % gx, rest = blockIdx.x / gx;
    const long bofs = (long)(rest / gy) * R * S;
    const long s0 = (long)bx * 64, r0 = (long)(rest % gy) * 64;
    const int tx = threadIdx.x & 63, ty = threadIdx.x >> 6;
    for (int i = ty; i < 64; i += 4) {
        const long r = r0 + i, s = s0 + tx;
        if (r < R && s < S) tile[i][tx] = src[bofs + r * S + s];
    }
    __syncthreads();
    for (int i = ty; i < 64; i += 4) {
        const long s = s0 + i, r = r0 + tx;
        if (r < R && s < S) dst[bofs + s * R + r] = tile[tx][i];
    }
}

} // namespace s2

// ---------------------------------------------------------------------------------
// launchers of the two 16-longitude matrix-core families: declared everywhere, defined (and instantiated for every
// shape the dispatch below names) in their own compilation of this file
// ---------------------------------------------------------------------------------
namespace s2 {

enum Which { FWD, DQ, DKDV };

template <typename T, int D, bool PAD> int launch_h16(Which which, const Args &a0, hipStream_t stream);
template <int D, int NS> int launch_m32(Which which, const Args &a0, hipStream_t stream);
template <int D, int MODE, typename T> int launch_ring_m32(const Args &a0, hipStream_t stream);
template <int D, bool WRITE, typename T> int launch_ring_pass2_m32(const Args &a0, hipStream_t stream);

#if S2_PART == 0 || S2_PART == 2
// 16-bit matrix-core kernels: bf16 / fp16 storage, head dim D, equal longitude counts, 16-byte aligned tensors.  The
// dq pass exists only in the form that takes the forward's y and lse.
template <typename T, int D, bool PAD> int launch_h16(Which which, const Args &a0, hipStream_t stream)
{
    if constexpr (std::is_same<T, float>::value) {
        return s2attn_fail(S2ATTN_E_UNSUPPORTED, "16-bit kernels asked for fp32 storage");
    } else {
        Args a = a0;
        a.row_first = 0;
        void (*kern)(const Args) = nullptr;
        long nblocks = 0;
        const int lds = h16_lds_bytes<D>();
        if (which == FWD) {
            kern = fwd_h16_kernel<T, D, PAD>;
            nblocks = (long)a.Ho * ((a.Wo + WQ - 1) / WQ) * a.B * a.nh;
        } else if (which == DQ) {
            kern = dq_h16_kernel<T, D, PAD>;
            nblocks = (long)a.Ho * ((a.Wo + WQ - 1) / WQ) * a.B * a.nh;
        } else {
            kern = dkdv_h16_kernel<T, D, PAD>;
            nblocks = (long)a.Hi * ((a.Wi + WQ - 1) / WQ) * a.B * a.nh;
        }
        if (nblocks > 0x7fffffffL) return s2attn_fail(S2ATTN_E_UNSUPPORTED, "problem needs %ld workgroups, more than one grid holds", nblocks);
        if (lds > 48 * 1024) {
            const hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, lds);
            if (e != hipSuccess) return s2attn_fail(S2ATTN_E_LAUNCH, "hipFuncSetAttribute: %s", hipGetErrorString(e));
        }
        hipLaunchKernelGGL(kern, dim3((unsigned)nblocks), dim3(64 * NW), lds, stream, a);
        const hipError_t e = hipGetLastError();
        if (e != hipSuccess) return s2attn_fail(S2ATTN_E_LAUNCH, "kernel launch: %s", hipGetErrorString(e));
        return S2ATTN_OK;
    }
}
#endif
#if S2_PART == 2
#define S2_H16_INSTANCES(T)                                                      \
    template int launch_h16<T, 32, false>(Which, const Args &, hipStream_t);    \
    template int launch_h16<T, 64, false>(Which, const Args &, hipStream_t);    \
    template int launch_h16<T, 128, false>(Which, const Args &, hipStream_t);   \
    template int launch_h16<T, 32, true>(Which, const Args &, hipStream_t);     \
    template int launch_h16<T, 64, true>(Which, const Args &, hipStream_t);     \
    template int launch_h16<T, 128, true>(Which, const Args &, hipStream_t);    \
    template int launch_h16<T, 256, true>(Which, const Args &, hipStream_t);
S2_H16_INSTANCES(bf16_t)
S2_H16_INSTANCES(f16_t)
S2_H16_INSTANCES(float) // never reached (fp32 storage takes the other families); only its error return is compiled
#undef S2_H16_INSTANCES
#endif

#if S2_PART == 0 || S2_PART == 3
// fp32 16-longitude matrix-core kernels, tiles of 16, 32, 64 or 128 channels: same launch geometry and the same conditions as the 16-bit family.
template <int D, int NS> int launch_m32(Which which, const Args &a0, hipStream_t stream)
{
    Args a = a0;
    a.row_first = 0;
    void (*kern)(const Args) = nullptr;
    long nblocks = 0;
    int lds = NS > 1 ? m32_lds_bytes<D, NS>(false) : 0; // one wavefront per workgroup: static LDS
    if (which == FWD) {
        kern = fwd_m32_kernel<D, NS>;
        nblocks = (long)a.Ho * ((a.Wo + HQ - 1) / HQ) * a.B * a.nh;
    } else if (which == DQ) {
        kern = dq_m32_kernel<D, NS>;
        nblocks = (long)a.Ho * ((a.Wo + HQ - 1) / HQ) * a.B * a.nh;
    } else {
        kern = dkdv_m32_kernel<D, NS>;
        nblocks = (long)a.Hi * ((a.Wi + HQ - 1) / HQ) * a.B * a.nh;
        lds = NS > 1 ? m32_lds_bytes<D, NS>(true) : 0;
    }
    if (nblocks > 0x7fffffffL) return s2attn_fail(S2ATTN_E_UNSUPPORTED, "problem needs %ld workgroups, more than one grid holds", nblocks);
    if (lds > 48 * 1024) {
        const hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, lds);
        if (e != hipSuccess) return s2attn_fail(S2ATTN_E_LAUNCH, "hipFuncSetAttribute: %s", hipGetErrorString(e));
    }
    hipLaunchKernelGGL(kern, dim3((unsigned)nblocks), dim3(64 * NS), lds, stream, a);
    const hipError_t e = hipGetLastError();
    if (e != hipSuccess) return s2attn_fail(S2ATTN_E_LAUNCH, "kernel launch: %s", hipGetErrorString(e));
    return S2ATTN_OK;
}
#endif
#if S2_PART == 0 || S2_PART == 3 || S2_PART == 4
// one ring step (forward, or pass 1 of the backward) on the fp32 16-longitude kernels, tensors of storage type T: one wavefront per 16 local output longitudes
template <int D, int MODE, typename T> int launch_ring_m32(const Args &a0, hipStream_t stream)
{
    Args a = a0;
    a.row_first = 0;
    const long nblocks = (long)a.Ho * ((a.Wo + HQ - 1) / HQ) * a.B * a.nh;
    if (nblocks > 0x7fffffffL) return s2attn_fail(S2ATTN_E_UNSUPPORTED, "problem needs %ld workgroups, more than one grid holds", nblocks);
    hipLaunchKernelGGL((ring_m32_kernel<D, MODE, T>), dim3((unsigned)nblocks), dim3(64), 0, stream, a);
    const hipError_t e = hipGetLastError();
    if (e != hipSuccess) return s2attn_fail(S2ATTN_E_LAUNCH, "kernel launch: %s", hipGetErrorString(e));
    return S2ATTN_OK;
}
// pass 2 of a ring step: one wavefront per 16 virtual columns of a column class of a chunk latitude
template <int D, bool WRITE, typename T> int launch_ring_pass2_m32(const Args &a, hipStream_t stream)
{
    const int ntile = (a.r_nkx / a.kps + 1 + HQ - 1) / HQ + 1; // as in the kernel
    const long nblocks = (long)a.Hi * ntile * a.B;
    if (nblocks > 0x7fffffffL) return s2attn_fail(S2ATTN_E_UNSUPPORTED, "problem needs %ld workgroups, more than one grid holds", nblocks);
    hipLaunchKernelGGL((ring_pass2_m32_kernel<D, WRITE, T>), dim3((unsigned)nblocks), dim3(64), 0, stream, a);
    const hipError_t e = hipGetLastError();
    if (e != hipSuccess) return s2attn_fail(S2ATTN_E_LAUNCH, "kernel launch: %s", hipGetErrorString(e));
    return S2ATTN_OK;
}
#endif
#if S2_PART == 3
template int launch_ring_pass2_m32<16, false, float>(const Args &, hipStream_t);
template int launch_ring_pass2_m32<16, true, float>(const Args &, hipStream_t);
template int launch_ring_m32<16, 0, float>(const Args &, hipStream_t);
template int launch_ring_m32<16, 1, float>(const Args &, hipStream_t);
template int launch_ring_m32<16, 2, float>(const Args &, hipStream_t);
template int launch_ring_pass2_m32<32, false, float>(const Args &, hipStream_t);
template int launch_ring_pass2_m32<32, true, float>(const Args &, hipStream_t);
template int launch_ring_m32<32, 0, float>(const Args &, hipStream_t);
template int launch_ring_m32<32, 1, float>(const Args &, hipStream_t);
template int launch_ring_m32<32, 2, float>(const Args &, hipStream_t);
template int launch_ring_pass2_m32<64, false, float>(const Args &, hipStream_t);
template int launch_ring_pass2_m32<64, true, float>(const Args &, hipStream_t);
template int launch_ring_m32<64, 0, float>(const Args &, hipStream_t);
template int launch_ring_m32<64, 1, float>(const Args &, hipStream_t);
template int launch_ring_m32<64, 2, float>(const Args &, hipStream_t);
template int launch_ring_pass2_m32<128, false, float>(const Args &, hipStream_t);
template int launch_ring_pass2_m32<128, true, float>(const Args &, hipStream_t);
template int launch_ring_m32<128, 0, float>(const Args &, hipStream_t);
template int launch_ring_m32<128, 1, float>(const Args &, hipStream_t);
template int launch_ring_m32<128, 2, float>(const Args &, hipStream_t);
template int launch_m32<16, 1>(Which, const Args &, hipStream_t);
template int launch_m32<32, 1>(Which, const Args &, hipStream_t);
template int launch_m32<64, 1>(Which, const Args &, hipStream_t);
template int launch_m32<128, 1>(Which, const Args &, hipStream_t);
template int launch_m32<128, 2>(Which, const Args &, hipStream_t);
template int launch_m32<128, 3>(Which, const Args &, hipStream_t);
template int launch_m32<128, 4>(Which, const Args &, hipStream_t);
#endif
#if S2_PART == 4
template int launch_ring_pass2_m32<16, false, bf16_t>(const Args &, hipStream_t);
template int launch_ring_pass2_m32<16, true, bf16_t>(const Args &, hipStream_t);
template int launch_ring_m32<16, 0, bf16_t>(const Args &, hipStream_t);
template int launch_ring_m32<16, 1, bf16_t>(const Args &, hipStream_t);
template int launch_ring_m32<16, 2, bf16_t>(const Args &, hipStream_t);
template int launch_ring_pass2_m32<32, false, bf16_t>(const Args &, hipStream_t);
template int launch_ring_pass2_m32<32, true, bf16_t>(const Args &, hipStream_t);
template int launch_ring_m32<32, 0, bf16_t>(const Args &, hipStream_t);
template int launch_ring_m32<32, 1, bf16_t>(const Args &, hipStream_t);
template int launch_ring_m32<32, 2, bf16_t>(const Args &, hipStream_t);
template int launch_ring_pass2_m32<64, false, bf16_t>(const Args &, hipStream_t);
template int launch_ring_pass2_m32<64, true, bf16_t>(const Args &, hipStream_t);
template int launch_ring_m32<64, 0, bf16_t>(const Args &, hipStream_t);
template int launch_ring_m32<64, 1, bf16_t>(const Args &, hipStream_t);
template int launch_ring_m32<64, 2, bf16_t>(const Args &, hipStream_t);
template int launch_ring_pass2_m32<128, false, bf16_t>(const Args &, hipStream_t);
template int launch_ring_pass2_m32<128, true, bf16_t>(const Args &, hipStream_t);
template int launch_ring_m32<128, 0, bf16_t>(const Args &, hipStream_t);
template int launch_ring_m32<128, 1, bf16_t>(const Args &, hipStream_t);
template int launch_ring_m32<128, 2, bf16_t>(const Args &, hipStream_t);
template int launch_ring_pass2_m32<16, false, f16_t>(const Args &, hipStream_t);
template int launch_ring_pass2_m32<16, true, f16_t>(const Args &, hipStream_t);
template int launch_ring_m32<16, 0, f16_t>(const Args &, hipStream_t);
template int launch_ring_m32<16, 1, f16_t>(const Args &, hipStream_t);
template int launch_ring_m32<16, 2, f16_t>(const Args &, hipStream_t);
template int launch_ring_pass2_m32<32, false, f16_t>(const Args &, hipStream_t);
template int launch_ring_pass2_m32<32, true, f16_t>(const Args &, hipStream_t);
template int launch_ring_m32<32, 0, f16_t>(const Args &, hipStream_t);
template int launch_ring_m32<32, 1, f16_t>(const Args &, hipStream_t);
template int launch_ring_m32<32, 2, f16_t>(const Args &, hipStream_t);
template int launch_ring_pass2_m32<64, false, f16_t>(const Args &, hipStream_t);
template int launch_ring_pass2_m32<64, true, f16_t>(const Args &, hipStream_t);
template int launch_ring_m32<64, 0, f16_t>(const Args &, hipStream_t);
template int launch_ring_m32<64, 1, f16_t>(const Args &, hipStream_t);
template int launch_ring_m32<64, 2, f16_t>(const Args &, hipStream_t);
template int launch_ring_pass2_m32<128, false, f16_t>(const Args &, hipStream_t);
template int launch_ring_pass2_m32<128, true, f16_t>(const Args &, hipStream_t);
template int launch_ring_m32<128, 0, f16_t>(const Args &, hipStream_t);
template int launch_ring_m32<128, 1, f16_t>(const Args &, hipStream_t);
template int launch_ring_m32<128, 2, f16_t>(const Args &, hipStream_t);
#endif

} // namespace s2

#if S2_PART <= 1
// ---------------------------------------------------------------------------------
// host side
// ---------------------------------------------------------------------------------
namespace {

using namespace s2;

int check_shape(const s2attn_shape *sh)
{
    if (!sh) return s2attn_fail(S2ATTN_E_INVALID, "shape is null");
    if (sh->batch < 1 || sh->nlat_in < 1 || sh->nlon_in < 1 || sh->nlat_out < 1 || sh->nlon_out < 1)
        return s2attn_fail(S2ATTN_E_INVALID, "batch and grid extents must be positive");
    if (sh->num_heads < 1) return s2attn_fail(S2ATTN_E_INVALID, "num_heads must be positive, got %d", sh->num_heads);
    if (sh->ck < 1 || sh->cv < 1) return s2attn_fail(S2ATTN_E_INVALID, "per-head channel counts must be positive");
    if (sh->nlon_in % sh->nlon_out != 0 && sh->nlon_out % sh->nlon_in != 0)
        return s2attn_fail(S2ATTN_E_INVALID, "nlon_in (%d) must be an integer multiple of nlon_out (%d), or the other way round", sh->nlon_in, sh->nlon_out);
    if (sh->dtype != S2ATTN_F32 && sh->dtype != S2ATTN_BF16 && sh->dtype != S2ATTN_F16)
        return s2attn_fail(S2ATTN_E_INVALID, "unknown dtype code %d", sh->dtype);
    {
        const int pk = sh->num_heads * sh->ck, pv = sh->num_heads * sh->cv;
        const int lds[8] = {sh->ld_k, sh->ld_q, sh->ld_dk, sh->ld_dq, sh->ld_v, sh->ld_y, sh->ld_dy, sh->ld_dv};
        for (int i = 0; i < 8; i++)
            if (lds[i] != 0 && (lds[i] < (i < 4 ? pk : pv) || lds[i] % 4 != 0))
                return s2attn_fail(S2ATTN_E_INVALID, "point stride %d is smaller than the packed row (%d) or not a multiple of 4", lds[i], i < 4 ? pk : pv);
    }
    if (sh->ck > 512 || sh->cv > 512)
        return s2attn_fail(S2ATTN_E_UNSUPPORTED, "per-head channels above 512 are not instantiated (ck=%d, cv=%d)", sh->ck, sh->cv);
    // the kernels form offsets inside one latitude of one batch entry in 32 bits
    const long long wmax = sh->nlon_in > sh->nlon_out ? sh->nlon_in : sh->nlon_out, cmax = sh->ck > sh->cv ? sh->ck : sh->cv;
    long long ldmax = 0;
    for (int ld : {sh->ld_k, sh->ld_q, sh->ld_dk, sh->ld_dq, sh->ld_v, sh->ld_y, sh->ld_dy, sh->ld_dv}) ldmax = ld > ldmax ? ld : ldmax;
    if (wmax * ldmax * 4 >= (1LL << 31)) return s2attn_fail(S2ATTN_E_UNSUPPORTED, "one latitude row of a strided tensor (%lld points x %lld elements) exceeds 2 GiB", wmax, ldmax);
    if (wmax * sh->num_heads * cmax * 4 >= (1LL << 31))
        return s2attn_fail(S2ATTN_E_UNSUPPORTED, "one latitude row of a tensor (%lld points x %d heads x %lld channels) exceeds 2 GiB", wmax, sh->num_heads, cmax);
    return S2ATTN_OK;
}

int esize(int dtype) { return dtype == S2ATTN_F32 ? 4 : 2; }

bool aligned(const void *p, size_t n) { return (reinterpret_cast<uintptr_t>(p) % n) == 0; }

template <typename T, int P, bool VEC> int launch_one(Which which, const Args &a0, int row_first, int row_count, hipStream_t stream)
{
    Args a = a0;
    a.row_first = row_first;
    if (row_count <= 0) return S2ATTN_OK;
    const int BH = a.B * a.nh;
    constexpr int LS = P + 4;
    void (*kern)(const Args) = nullptr;
    long nblocks = 0;
    size_t lds = 0;
    // fast path: 16-byte loads, equal longitude counts, and a grid at least as wide as one staged band
    constexpr int FAST_ROWS = Band<T, P>::NIT * Band<T, P>::RPI;
    const bool fast = VEC && a.Wi >= FAST_ROWS && a.dk_ == P && a.dv_ == P;
    if (fast) a.tile_rows = FAST_ROWS;
    if (which == FWD) {
        kern = fast ? fwd_fast_kernel<T, P> : fwd_kernel<T, P, VEC>;
        nblocks = (long)row_count * ((a.Wo + TQ - 1) / TQ) * BH;
        lds = (size_t)2 * a.tile_rows * LS * sizeof(float);
    } else if (which == DQ) {
        kern = fast ? dq_fast_kernel<T, P> : dq_kernel<T, P, VEC>;
        nblocks = (long)row_count * ((a.Wo + TQ - 1) / TQ) * BH;
        lds = (size_t)2 * a.tile_rows * LS * sizeof(float);
    } else {
        kern = fast ? dkdv_fast_kernel<T, P> : dkdv_kernel<T, P, VEC>;
        nblocks = (long)row_count * ((a.Wi + TQ - 1) / TQ) * BH;
        lds = (size_t)2 * a.tile_rows * LS * sizeof(float) + (size_t)a.tile_rows * sizeof(float2);
    }
    if (nblocks > 0x7fffffffL) return s2attn_fail(S2ATTN_E_UNSUPPORTED, "problem needs %ld workgroups, more than one grid holds", nblocks);
    if (lds > 160 * 1024) return s2attn_fail(S2ATTN_E_UNSUPPORTED, "the staged band needs %zu bytes of LDS per workgroup", lds);
    if (lds > 48 * 1024) {
        const hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        if (e != hipSuccess) return s2attn_fail(S2ATTN_E_LAUNCH, "hipFuncSetAttribute: %s", hipGetErrorString(e));
    }
    hipLaunchKernelGGL(kern, dim3((unsigned)nblocks), dim3(TQ), lds, stream, a);
    const hipError_t e = hipGetLastError();
    if (e != hipSuccess) return s2attn_fail(S2ATTN_E_LAUNCH, "kernel launch: %s", hipGetErrorString(e));
    return S2ATTN_OK;
}

template <typename T, int LPQ, bool VEC> int launch_wide(Which which, const Args &a0, int row_first, int row_count, hipStream_t stream)
{
    if (row_count <= 0) return S2ATTN_OK;
    Args a = a0;
    a.row_first = row_first;
    constexpr int TQW = TQ / LPQ, LS = 32 * LPQ + 4, TSW = WideCfg<LPQ>::TSW;
    const int BH = a.B * a.nh;
    void (*kern)(const Args) = nullptr;
    long nblocks = 0;
    a.tile_rows = TQW - 1 + TSW; // a band: the tile's grid points slid over one chunk of neighbors
    size_t lds = (size_t)2 * a.tile_rows * LS * sizeof(float);
    // the tiles double as the exchange buffer when the wavefronts merge their states: 34 / 67 / 64 floats per lane
    static_assert((size_t)2 * (TQW - 1 + TSW) * LS >= (size_t)67 * TQ, "band tiles too small for the state merge");
    static_assert((size_t)(TQW - 1 + TSW) * LS >= (size_t)34 * TQ, "band tile too small for the forward state merge");
    if (which == DKDV) {
        kern = dkdv_wide_kernel<T, LPQ, VEC>;
        nblocks = (long)row_count * ((a.Wi + TQW - 1) / TQW) * BH;
        lds += (size_t)a.tile_rows * sizeof(float2);
    } else {
        kern = which == FWD ? fwd_wide_kernel<T, LPQ, VEC> : dq_wide_kernel<T, LPQ, VEC>;
        nblocks = (long)row_count * ((a.Wo + TQW - 1) / TQW) * BH;
    }
    if (nblocks > 0x7fffffffL) return s2attn_fail(S2ATTN_E_UNSUPPORTED, "problem needs %ld workgroups, more than one grid holds", nblocks);
    if (lds > 160 * 1024) return s2attn_fail(S2ATTN_E_UNSUPPORTED, "the staged band needs %zu bytes of LDS per workgroup", lds);
    if (lds > 48 * 1024) {
        const hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        if (e != hipSuccess) return s2attn_fail(S2ATTN_E_LAUNCH, "hipFuncSetAttribute: %s", hipGetErrorString(e));
    }
    hipLaunchKernelGGL(kern, dim3((unsigned)nblocks), dim3(WNT), lds, stream, a);
    const hipError_t e = hipGetLastError();
    if (e != hipSuccess) return s2attn_fail(S2ATTN_E_LAUNCH, "kernel launch: %s", hipGetErrorString(e));
    return S2ATTN_OK;
}

template <typename T, bool VEC> int launch_p(Which which, const Args &a, int row_first, int row_count, hipStream_t stream)
{
    const int d = a.dk_ > a.dv_ ? a.dk_ : a.dv_;
    if (d > 256) return launch_wide<T, 16, VEC>(which, a, row_first, row_count, stream);
    if (d > 128) return launch_wide<T, 8, VEC>(which, a, row_first, row_count, stream);
    if (d > 64) return launch_wide<T, 4, VEC>(which, a, row_first, row_count, stream);
    if (d > 32) return launch_wide<T, 2, VEC>(which, a, row_first, row_count, stream);
    if (d <= 4) return launch_one<T, 4, VEC>(which, a, row_first, row_count, stream);
    if (d <= 8) return launch_one<T, 8, VEC>(which, a, row_first, row_count, stream);
    if (d <= 16) return launch_one<T, 16, VEC>(which, a, row_first, row_count, stream);
    return launch_one<T, 32, VEC>(which, a, row_first, row_count, stream);
}

// hybrid kernels: head dim 32, vector-aligned rows, at least 64 columns per virtual latitude.  One workgroup row per item
// of the plan's work list (a long-run latitude, a single short-run latitude or a pair of adjacent short-run latitudes;
// long-run and short-run units interleaved: matrix-core-heavy and vector-heavy workgroups side by side).  The dq pass
// exists only in the form that takes the forward's y and lse.
template <typename T> int launch_dense(Which which, const Args &a0, hipStream_t stream)
{
    Args a = a0;
    a.row_first = 0;
    void (*kern)(const Args) = nullptr;
    long nblocks = 0;
    if (which == FWD) {
        kern = fwd_mfma_kernel<T>;
        nblocks = (long)a.n_gitems * ((a.Wo + MT - 1) / MT) * a.B * a.nh;
    } else if (which == DQ) {
        kern = dq_saved_mfma_kernel<T>;
        nblocks = (long)a.Ho * ((a.Wo + MT - 1) / MT) * a.B * a.nh;
    } else {
        kern = dkdv_mfma_kernel<T>;
        nblocks = (long)a.n_sitems * ((a.Wi + MT - 1) / MT) * a.B * a.nh;
    }
    if (nblocks <= 0) return S2ATTN_OK;
    if (nblocks > 0x7fffffffL) return s2attn_fail(S2ATTN_E_UNSUPPORTED, "problem needs %ld workgroups, more than one grid holds", nblocks);
    hipLaunchKernelGGL(kern, dim3((unsigned)nblocks), dim3(64), 0, stream, a);
    const hipError_t e = hipGetLastError();
    if (e != hipSuccess) return s2attn_fail(S2ATTN_E_LAUNCH, "kernel launch: %s", hipGetErrorString(e));
    return S2ATTN_OK;
}

// Head widths: any multiple of 8 from 16 to 256, staged in a tile of 32, 64, 128 or 256 channels (zeros past the head).
bool h16_width(int ck, int cv) { return ck == cv && ck % 8 == 0 && ck >= 16 && ck <= 256; }

template <typename T> bool h16_ok(Which which, const Args &a)
{
    if (std::is_same<T, float>::value) return false;
    if (!h16_width(a.dk_, a.dv_) || a.Wi < HK) return false;
    if (which == DQ && !(a.ysaved && a.lse)) return false;
    const void *ptrs[] = {a.k, a.v, a.q, a.dy, a.y, a.dk, a.dv, a.dq, a.ysaved};
    for (const void *p : ptrs)
        if (p && !aligned(p, 16)) return false;
    return true;
}

// Head widths: any multiple of 4 from 16 to 512, staged in a tile of 16, 32, 64 or 128 channels (zeros past the head), or in
// two to four channel groups of 128 worked on by as many wavefronts.
bool m32_width(int ck, int cv) { return ck == cv && ck % 4 == 0 && ck >= 16 && ck <= 512; }

template <typename T> bool m32_ok(Which which, const Args &a)
{
    if (!std::is_same<T, float>::value) return false;
    if (!m32_width(a.dk_, a.dv_) || a.Wi < HK) return false;
    if (which == DQ && !(a.ysaved && a.lse)) return false;
    const void *ptrs[] = {a.k, a.v, a.q, a.dy, a.y, a.dk, a.dv, a.dq, a.ysaved};
    for (const void *p : ptrs)
        if (p && !aligned(p, 16)) return false;
    return true;
}

bool dense_ok(Which which, const Args &a, bool vec)
{
    if (which == DQ && !(a.ysaved && a.lse)) return false;
    return vec && a.dk_ == 32 && a.dv_ == 32 && a.Wi >= 64;
}

template <typename T> int launch_t(Which which, const Args &a, bool vec, int ndense, hipStream_t stream)
{
    const int nrows = which == DKDV ? a.Hi : a.Ho;
    int first = 0;
    if (a.unpacked) { // column blocks of a wider buffer: only the hybrid kernels address every tensor by its own point stride
        if (!dense_ok(which, a, vec))
            return s2attn_fail(S2ATTN_E_UNSUPPORTED, "tensors with a point stride need the hybrid kernels: ck = cv = 32, 16-byte aligned, at least 64 longitudes%s",
                               which == DQ ? ", backward from saved statistics" : "");
        return launch_dense<T>(which, a, stream);
    }
    if (h16_ok<T>(which, a)) {
        if (a.dk_ == 32) return launch_h16<T, 32, false>(which, a, stream);
        if (a.dk_ == 64) return launch_h16<T, 64, false>(which, a, stream);
        if (a.dk_ == 128) return launch_h16<T, 128, false>(which, a, stream);
        if (a.dk_ < 32) return launch_h16<T, 32, true>(which, a, stream);
        if (a.dk_ < 64) return launch_h16<T, 64, true>(which, a, stream);
        if (a.dk_ < 128) return launch_h16<T, 128, true>(which, a, stream);
        return launch_h16<T, 256, true>(which, a, stream);
    }
    if (dense_ok(which, a, vec)) {
        // head dim 32 on at least 64 columns: the hybrid kernels handle short runs themselves (vector path inside), so
        // they take every latitude; measured ahead of the 16-longitude family there (cfg3 13.5 against 16.4 ms)
        (void)ndense;
        return launch_dense<T>(which, a, stream);
    }
    if (m32_ok<T>(which, a)) {
        if (a.dk_ <= 16) return launch_m32<16, 1>(which, a, stream);
        if (a.dk_ <= 32) return launch_m32<32, 1>(which, a, stream);
        if (a.dk_ <= 64) return launch_m32<64, 1>(which, a, stream);
        if (a.dk_ <= 128) return launch_m32<128, 1>(which, a, stream);
        if (a.dk_ <= 256) return launch_m32<128, 2>(which, a, stream);
        return a.dk_ <= 384 ? launch_m32<128, 3>(which, a, stream) : launch_m32<128, 4>(which, a, stream);
    }
    return vec ? launch_p<T, true>(which, a, first, nrows - first, stream) : launch_p<T, false>(which, a, first, nrows - first, stream);
}

int launch(Which which, const Args &a, int dtype, bool vec, int ndense, hipStream_t stream)
{
    if (dtype == S2ATTN_F32) return launch_t<float>(which, a, vec, ndense, stream);
    if (dtype == S2ATTN_BF16) return launch_t<bf16_t>(which, a, vec, ndense, stream);
    return launch_t<f16_t>(which, a, vec, ndense, stream);
}

// The plan must be the blob s2attn_plan_build made for exactly these grid extents.
int check_plan(const s2attn_plan *plan, const s2attn_shape *sh)
{
    if (!plan || !plan->data) return s2attn_fail(S2ATTN_E_INVALID, "plan is null");
    const int32_t *h = plan->header;
    if (h[S2ATTN_PH_MAGIC] != S2ATTN_PLAN_MAGIC) return s2attn_fail(S2ATTN_E_INVALID, "plan header does not carry this library's plan format");
    if (h[S2ATTN_PH_NLAT_IN] != sh->nlat_in || h[S2ATTN_PH_NLON_IN] != sh->nlon_in || h[S2ATTN_PH_NLAT_OUT] != sh->nlat_out || h[S2ATTN_PH_NLON_OUT] != sh->nlon_out)
        return s2attn_fail(S2ATTN_E_INVALID, "plan was built for grids %dx%d -> %dx%d, the call is for %dx%d -> %dx%d", h[S2ATTN_PH_NLAT_IN], h[S2ATTN_PH_NLON_IN],
                           h[S2ATTN_PH_NLAT_OUT], h[S2ATTN_PH_NLON_OUT], sh->nlat_in, sh->nlon_in, sh->nlat_out, sh->nlon_out);
    const int32_t total = h[S2ATTN_PH_TOTAL];
    for (int i = S2ATTN_PH_GATHER_OFF; i <= S2ATTN_PH_GATHER_SPAN; i++) {
        if (i == S2ATTN_PH_GATHER_NITEMS || i == S2ATTN_PH_GATHER_NPAIRS || i == S2ATTN_PH_SCATTER_NITEMS || i == S2ATTN_PH_SCATTER_NPAIRS) continue;
        if (h[i] < S2ATTN_PLAN_HEADER_INTS || h[i] > total) return s2attn_fail(S2ATTN_E_INVALID, "plan header: offset %d of array %d lies outside the plan", h[i], i);
    }
    return S2ATTN_OK;
}

void fill_args(Args &a, const s2attn_plan *plan, const s2attn_shape *sh, const float *quad_w)
{
    const int32_t *h = plan->header, *d = plan->data;
    a.quad_w = quad_w;
    a.goff = d + h[S2ATTN_PH_GATHER_OFF];
    a.gruns = reinterpret_cast<const Run *>(d + h[S2ATTN_PH_GATHER_RUNS]);
    a.gorder = d + h[S2ATTN_PH_GATHER_ORDER];
    a.gorder_mixed = d + h[S2ATTN_PH_GATHER_ORDER_MIXED];
    a.soff = d + h[S2ATTN_PH_SCATTER_OFF];
    a.sruns = reinterpret_cast<const Run *>(d + h[S2ATTN_PH_SCATTER_RUNS]);
    a.sorder = d + h[S2ATTN_PH_SCATTER_ORDER];
    a.sorder_mixed = d + h[S2ATTN_PH_SCATTER_ORDER_MIXED];
    a.gitems = d + h[S2ATTN_PH_GATHER_ITEMS];
    a.gpoff = d + h[S2ATTN_PH_GATHER_PAIR_OFF];
    a.gpruns = reinterpret_cast<const PRun *>(d + h[S2ATTN_PH_GATHER_PAIR_RUNS]);
    a.n_gitems = h[S2ATTN_PH_GATHER_NITEMS];
    a.sitems = d + h[S2ATTN_PH_SCATTER_ITEMS];
    a.spoff = d + h[S2ATTN_PH_SCATTER_PAIR_OFF];
    a.spruns = reinterpret_cast<const PRun *>(d + h[S2ATTN_PH_SCATTER_PAIR_RUNS]);
    a.n_sitems = h[S2ATTN_PH_SCATTER_NITEMS];
    a.B = sh->batch;
    a.nh = sh->num_heads;
    const bool up = sh->nlon_out % sh->nlon_in == 0 && sh->nlon_out != sh->nlon_in;
    a.kps = up ? 1 : sh->nlon_in / sh->nlon_out;
    a.qps = up ? sh->nlon_out / sh->nlon_in : 1;
    a.Hi = sh->nlat_in * a.kps;  // virtual input latitudes, see key_point()
    a.Ho = sh->nlat_out * a.qps; // virtual output latitudes, see query_point()
    a.Wi = a.Wo = up ? sh->nlon_in : sh->nlon_out; // columns of a virtual latitude
    a.dk_ = sh->ck;
    a.dv_ = sh->cv;
    const unsigned pk = (unsigned)sh->num_heads * sh->ck, pv = (unsigned)sh->num_heads * sh->cv;
    a.ldk = sh->ld_k ? sh->ld_k : pk, a.ldq = sh->ld_q ? sh->ld_q : pk, a.lddk = sh->ld_dk ? sh->ld_dk : pk, a.lddq = sh->ld_dq ? sh->ld_dq : pk;
    a.ldv = sh->ld_v ? sh->ld_v : pv, a.ldy = sh->ld_y ? sh->ld_y : pv, a.ldg = sh->ld_dy ? sh->ld_dy : pv, a.lddv = sh->ld_dv ? sh->ld_dv : pv;
    a.unpacked = a.ldk != pk || a.ldq != pk || a.lddk != pk || a.lddq != pk || a.ldv != pv || a.ldy != pv || a.ldg != pv || a.lddv != pv;
}



} // namespace

extern "C" int s2attn_forward_lse(const void *k, const void *v, const void *q, const float *quad_weights, void *y, float *lse,
                                  const s2attn_plan *plan, const s2attn_shape *shape, void *stream);

extern "C" int s2attn_forward(const void *k, const void *v, const void *q, const float *quad_weights, void *y,
                              const s2attn_plan *plan, const s2attn_shape *shape, void *stream)
{
    return s2attn_forward_lse(k, v, q, quad_weights, y, nullptr, plan, shape, stream);
}

extern "C" int s2attn_forward_lse(const void *k, const void *v, const void *q, const float *quad_weights, void *y, float *lse,
                                  const s2attn_plan *plan, const s2attn_shape *shape, void *stream)
{
    int rc = check_shape(shape);
    if (rc != S2ATTN_OK) return rc;
    if (!k || !v || !q || !y || !quad_weights) return s2attn_fail(S2ATTN_E_INVALID, "null tensor pointer");
    rc = check_plan(plan, shape);
    if (rc != S2ATTN_OK) return rc;
    Args a = {};
    fill_args(a, plan, shape, quad_weights);
    a.k = k, a.v = v, a.q = q, a.y = y;
    a.lse = lse;
    a.tile_rows = TQ - 1 + TL;
    const size_t al = 4 * (size_t)esize(shape->dtype);
    const bool vec = shape->ck % 4 == 0 && shape->cv % 4 == 0 && aligned(k, al) && aligned(v, al) && aligned(q, al) && aligned(y, al);
    return launch(FWD, a, shape->dtype, vec, plan->header[S2ATTN_PH_GATHER_NDENSE], static_cast<hipStream_t>(stream));
}

// Ring steps on the band-staged kernels (ring_m32_kernel, ring_pass2_m32_kernel): checks and kernel arguments shared by the
// six entry points.  The two directions differ in what the plan's latitudes mean: gather direction - input latitudes global
// (the chunk holds r_lat0 .. + r_nlat of them), output longitudes nlon_in / pscale on the circle, of which nlon_out are
// local; up-sampling direction - input latitudes are the chunk's rows as they stand, the plan's output latitudes are
// virtual (nlat_out * pscale_out of them, nlon_in columns each).
namespace {
struct RingGeo {
    int batch, nlat_halo, nlon_kx, nlat_out, nlon_out, ck, cv, dtype, lon_lo_kx, lat_halo_start;
    int nlon_in, kps, qps; // global input longitudes; nlon_in / nlon_out_global and its inverse, one of them 1
};
int ring_plan_args(Args &a, const void *k, const void *v, const void *q, const void *dy, const float *quad_weights, const s2attn_plan *plan, const RingGeo &g)
{
    if (g.batch < 1 || g.nlat_halo < 1 || g.nlon_kx < 1 || g.nlat_out < 1 || g.nlon_out < 1 || g.nlon_in < 1)
        return s2attn_fail(S2ATTN_E_INVALID, "batch and grid extents must be positive");
    if (g.lon_lo_kx < 0 || g.lon_lo_kx + g.nlon_kx > g.nlon_in)
        return s2attn_fail(S2ATTN_E_INVALID, "chunk [%d, %d) leaves the input grid of %d longitudes", g.lon_lo_kx, g.lon_lo_kx + g.nlon_kx, g.nlon_in);
    const int W = g.nlon_in / g.kps;                    // columns of a (virtual) latitude of the plan
    const int wout = g.qps > 1 ? g.nlon_in * g.qps : W; // global output longitudes
    if (g.nlon_out > wout) return s2attn_fail(S2ATTN_E_INVALID, "%d local output longitudes on a grid of %d", g.nlon_out, wout);
    if (!k || !v || !q || !quad_weights) return s2attn_fail(S2ATTN_E_INVALID, "null tensor pointer");
    if (!plan || !plan->data) return s2attn_fail(S2ATTN_E_INVALID, "plan is null");
    const int32_t *h = plan->header;
    if (h[S2ATTN_PH_MAGIC] != S2ATTN_PLAN_MAGIC) return s2attn_fail(S2ATTN_E_INVALID, "plan header does not carry this library's plan format");
    if (h[S2ATTN_PH_NLON_IN] != g.nlon_in || h[S2ATTN_PH_NLAT_OUT] != g.nlat_out || h[S2ATTN_PH_NLON_OUT] != wout || (g.qps > 1 && h[S2ATTN_PH_NLAT_IN] != g.nlat_halo))
        return s2attn_fail(S2ATTN_E_INVALID, "plan was built for grids %dx%d -> %dx%d, the step needs %s x%d -> %dx%d (local latitudes, global longitudes)",
                           h[S2ATTN_PH_NLAT_IN], h[S2ATTN_PH_NLON_IN], h[S2ATTN_PH_NLAT_OUT], h[S2ATTN_PH_NLON_OUT], g.qps > 1 ? "the chunk's latitudes" : "all input latitudes",
                           g.nlon_in, g.nlat_out, wout);
    if (g.dtype != S2ATTN_F32 && g.dtype != S2ATTN_BF16 && g.dtype != S2ATTN_F16) return s2attn_fail(S2ATTN_E_INVALID, "unknown dtype code %d", g.dtype);
    if (!m32_width(g.ck, g.cv) || g.ck > 128 || W < HK)
        return s2attn_fail(S2ATTN_E_UNSUPPORTED, "the band-staged ring steps take tensors with ck = cv a multiple of 4 from 16 to 128 on at least %d longitudes", HK);
    const void *ptrs[] = {k, v, q, dy};
    const int need = g.dtype == S2ATTN_F32 ? 16 : 8; // four channels are loaded at a time
    for (const void *p : ptrs)
        if (p && !aligned(p, need)) return s2attn_fail(S2ATTN_E_UNSUPPORTED, "the band-staged ring steps take tensors aligned to four channels (%d bytes)", need);
    for (int i : {S2ATTN_PH_GATHER_OFF, S2ATTN_PH_GATHER_RUNS, S2ATTN_PH_GATHER_ORDER, S2ATTN_PH_GATHER_SPAN, S2ATTN_PH_SCATTER_OFF, S2ATTN_PH_SCATTER_RUNS, S2ATTN_PH_SCATTER_ORDER})
        if (h[i] < S2ATTN_PLAN_HEADER_INTS || h[i] > h[S2ATTN_PH_TOTAL]) return s2attn_fail(S2ATTN_E_INVALID, "plan header: offset %d of array %d lies outside the plan", h[i], i);
    const int32_t *d = plan->data;
    a.quad_w = quad_weights;
    a.goff = d + h[S2ATTN_PH_GATHER_OFF];
    a.gruns = reinterpret_cast<const Run *>(d + h[S2ATTN_PH_GATHER_RUNS]);
    a.gorder = d + h[S2ATTN_PH_GATHER_ORDER];
    a.gspan = reinterpret_cast<const int2 *>(d + h[S2ATTN_PH_GATHER_SPAN]);
    a.soff = d + h[S2ATTN_PH_SCATTER_OFF];
    a.sruns = reinterpret_cast<const Run *>(d + h[S2ATTN_PH_SCATTER_RUNS]);
    a.sorder = d + h[S2ATTN_PH_SCATTER_ORDER];
    a.k = k, a.v = v, a.q = q, a.dy = dy;
    a.B = g.batch, a.nh = 1, a.kps = g.kps, a.qps = 1;
    a.Hi = h[S2ATTN_PH_NLAT_IN] * g.kps, a.Wi = W;
    a.Ho = g.nlat_out * g.qps;                   // (virtual) output latitudes of the plan
    a.Wo = (g.nlon_out + g.qps - 1) / g.qps;     // columns of one of them that can be local: the tiles' domain
    a.r_qps = g.qps, a.r_wo = g.nlon_out;
    a.dk_ = a.dv_ = g.ck;
    a.r_lon_lo = g.lon_lo_kx, a.r_nkx = g.nlon_kx, a.r_nlat = g.nlat_halo;
    a.r_lat0 = g.qps > 1 ? 0 : g.lat_halo_start;   // the plan's input latitude of the chunk's row 0
    a.r_wlat0 = g.qps > 1 ? g.lat_halo_start : 0;  // the plan's input latitude -> index of its quadrature weight
    return S2ATTN_OK;
}
int ring_geo(RingGeo &g, const s2attn_ring_shape *sh)
{
    if (!sh) return s2attn_fail(S2ATTN_E_INVALID, "ring shape is null");
    if (sh->pscale < 1 || sh->nlon_in < 1 || sh->nlon_in % sh->pscale != 0)
        return s2attn_fail(S2ATTN_E_INVALID, "pscale must be a positive divisor of nlon_in = %d, got %d", sh->nlon_in, sh->pscale);
    g = RingGeo{sh->batch, sh->nlat_halo, sh->nlon_kx, sh->nlat_out, sh->nlon_out, sh->ck, sh->cv, sh->dtype, sh->lon_lo_kx, sh->lat_halo_start, sh->nlon_in, sh->pscale, 1};
    return S2ATTN_OK;
}
int ring_geo(RingGeo &g, const s2attn_ring_up_shape *sh)
{
    if (!sh) return s2attn_fail(S2ATTN_E_INVALID, "ring shape is null");
    if (sh->pscale_out < 1 || sh->nlon_out_global < 1 || sh->nlon_out_global % sh->pscale_out != 0)
        return s2attn_fail(S2ATTN_E_INVALID, "pscale_out must be a positive divisor of nlon_out_global = %d, got %d", sh->nlon_out_global, sh->pscale_out);
    g = RingGeo{sh->batch, sh->nlat_halo, sh->nlon_kx, sh->nlat_out, sh->nlon_out, sh->ck, sh->cv, sh->dtype, sh->lon_lo_kx, sh->lat_halo_start,
                sh->nlon_out_global / sh->pscale_out, 1, sh->pscale_out};
    return S2ATTN_OK;
}
template <int MODE, typename T> int launch_ring_plan_t(const Args &a, hipStream_t st)
{
    if (a.dk_ <= 16) return launch_ring_m32<16, MODE, T>(a, st);
    if (a.dk_ <= 32) return launch_ring_m32<32, MODE, T>(a, st);
    if (a.dk_ <= 64) return launch_ring_m32<64, MODE, T>(a, st);
    return launch_ring_m32<128, MODE, T>(a, st);
}
template <int MODE> int launch_ring_plan(const Args &a, int dtype, hipStream_t st)
{
    if (dtype == S2ATTN_BF16) return launch_ring_plan_t<MODE, bf16_t>(a, st);
    if (dtype == S2ATTN_F16) return launch_ring_plan_t<MODE, f16_t>(a, st);
    return launch_ring_plan_t<MODE, float>(a, st);
}
template <bool WRITE, typename T> int launch_ring_pass2_plan_t(const Args &a, hipStream_t st)
{
    if (a.dk_ <= 16) return launch_ring_pass2_m32<16, WRITE, T>(a, st);
    if (a.dk_ <= 32) return launch_ring_pass2_m32<32, WRITE, T>(a, st);
    if (a.dk_ <= 64) return launch_ring_pass2_m32<64, WRITE, T>(a, st);
    return launch_ring_pass2_m32<128, WRITE, T>(a, st);
}
template <bool WRITE> int launch_ring_pass2_plan(const Args &a, int dtype, hipStream_t st)
{
    if (dtype == S2ATTN_BF16) return launch_ring_pass2_plan_t<WRITE, bf16_t>(a, st);
    if (dtype == S2ATTN_F16) return launch_ring_pass2_plan_t<WRITE, f16_t>(a, st);
    return launch_ring_pass2_plan_t<WRITE, float>(a, st);
}
template <typename SHAPE>
int ring_forward_plan(const void *k, const void *v, const void *q, float *y_acc, float *alpha_sum, float *qdotk_max, const float *quad_weights,
                      const s2attn_plan *plan, const SHAPE *sh, void *stream)
{
    Args a = {};
    RingGeo g;
    int rc = ring_geo(g, sh);
    if (rc == S2ATTN_OK) rc = ring_plan_args(a, k, v, q, nullptr, quad_weights, plan, g);
    if (rc != S2ATTN_OK) return rc;
    if (!y_acc || !alpha_sum || !qdotk_max) return s2attn_fail(S2ATTN_E_INVALID, "null tensor pointer");
    if (!aligned(y_acc, 16)) return s2attn_fail(S2ATTN_E_UNSUPPORTED, "the band-staged ring steps take 16-byte aligned tensors");
    a.r_yacc = y_acc, a.r_asum = alpha_sum, a.r_qmax = qdotk_max;
    return launch_ring_plan<0>(a, g.dtype, static_cast<hipStream_t>(stream));
}
template <typename SHAPE, bool WRITE>
int ring_pass2_plan(const void *k, const void *v, const void *q, const void *dy, const float *alpha_sum, const float *qdotk_max, const float *integral_norm,
                    float *dk, float *dv, const float *quad_weights, const s2attn_plan *plan, const SHAPE *sh, void *stream)
{
    Args a = {};
    RingGeo g;
    int rc = ring_geo(g, sh);
    if (rc == S2ATTN_OK) rc = ring_plan_args(a, k, v, q, dy, quad_weights, plan, g);
    if (rc != S2ATTN_OK) return rc;
    if (!dy || !alpha_sum || !qdotk_max || !integral_norm || !dk || !dv) return s2attn_fail(S2ATTN_E_INVALID, "null tensor pointer");
    if (!aligned(dk, 16) || !aligned(dv, 16)) return s2attn_fail(S2ATTN_E_UNSUPPORTED, "the band-staged ring steps take 16-byte aligned tensors");
    a.r_asum = const_cast<float *>(alpha_sum), a.r_qmax = const_cast<float *>(qdotk_max), a.r_integral = const_cast<float *>(integral_norm);
    a.dk = dk, a.dv = dv;
    return launch_ring_pass2_plan<WRITE>(a, g.dtype, static_cast<hipStream_t>(stream));
}
} // namespace

extern "C" int s2attn_ring_forward_step_plan(const void *k, const void *v, const void *q, float *y_acc, float *alpha_sum, float *qdotk_max,
                                             const float *quad_weights, const s2attn_plan *plan, const s2attn_ring_shape *sh, void *stream)
{
    return ring_forward_plan(k, v, q, y_acc, alpha_sum, qdotk_max, quad_weights, plan, sh, stream);
}

extern "C" int s2attn_ring_forward_step_upsample_plan(const void *k, const void *v, const void *q, float *y_acc, float *alpha_sum, float *qdotk_max,
                                                      const float *quad_weights, const s2attn_plan *plan, const s2attn_ring_up_shape *sh, void *stream)
{
    return ring_forward_plan(k, v, q, y_acc, alpha_sum, qdotk_max, quad_weights, plan, sh, stream);
}

extern "C" int s2attn_ring_backward_pass2_plan(const void *k, const void *v, const void *q, const void *dy, const float *alpha_sum,
                                               const float *qdotk_max, const float *integral_norm, float *dk, float *dv,
                                               const float *quad_weights, const s2attn_plan *plan, const s2attn_ring_shape *sh, void *stream)
{
    return ring_pass2_plan<s2attn_ring_shape, false>(k, v, q, dy, alpha_sum, qdotk_max, integral_norm, dk, dv, quad_weights, plan, sh, stream);
}

extern "C" int s2attn_ring_backward_pass2_upsample_plan(const void *k, const void *v, const void *q, const void *dy, const float *alpha_sum,
                                                        const float *qdotk_max, const float *integral_norm, float *dk, float *dv,
                                                        const float *quad_weights, const s2attn_plan *plan, const s2attn_ring_up_shape *sh, void *stream)
{
    return ring_pass2_plan<s2attn_ring_up_shape, true>(k, v, q, dy, alpha_sum, qdotk_max, integral_norm, dk, dv, quad_weights, plan, sh, stream);
}

extern "C" int s2attn_ring_backward_pass1_plan(const void *k, const void *v, const void *q, const void *dy, float *alpha_sum, float *qdotk_max,
                                               float *integral, float *alpha_k, float *alpha_kvw, const float *quad_weights,
                                               const s2attn_plan *plan, const s2attn_ring_shape *sh, void *stream)
{
    Args a = {};
    RingGeo g;
    int rc = ring_geo(g, sh);
    if (rc == S2ATTN_OK) rc = ring_plan_args(a, k, v, q, dy, quad_weights, plan, g);
    if (rc != S2ATTN_OK) return rc;
    if (!dy || !alpha_sum || !qdotk_max || !integral || !alpha_k || !alpha_kvw) return s2attn_fail(S2ATTN_E_INVALID, "null tensor pointer");
    if (!aligned(alpha_k, 16) || !aligned(alpha_kvw, 16)) return s2attn_fail(S2ATTN_E_UNSUPPORTED, "the band-staged ring steps take 16-byte aligned tensors");
    a.r_asum = alpha_sum, a.r_qmax = qdotk_max, a.r_integral = integral, a.r_ak = alpha_k, a.r_akvw = alpha_kvw;
    return launch_ring_plan<1>(a, g.dtype, static_cast<hipStream_t>(stream));
}

extern "C" int s2attn_ring_backward_pass1_upsample_plan(const void *k, const void *v, const void *q, const void *dy, const float *qdotk_max,
                                                        float *integral, float *alpha_k, float *alpha_kvw, const float *quad_weights,
                                                        const s2attn_plan *plan, const s2attn_ring_up_shape *sh, void *stream)
{
    Args a = {};
    RingGeo g;
    int rc = ring_geo(g, sh);
    if (rc == S2ATTN_OK) rc = ring_plan_args(a, k, v, q, dy, quad_weights, plan, g);
    if (rc != S2ATTN_OK) return rc;
    if (!dy || !qdotk_max || !integral || !alpha_k || !alpha_kvw) return s2attn_fail(S2ATTN_E_INVALID, "null tensor pointer");
    if (!aligned(alpha_k, 16) || !aligned(alpha_kvw, 16)) return s2attn_fail(S2ATTN_E_UNSUPPORTED, "the band-staged ring steps take 16-byte aligned tensors");
    a.r_qmax = const_cast<float *>(qdotk_max), a.r_integral = integral, a.r_ak = alpha_k, a.r_akvw = alpha_kvw;
    return launch_ring_plan<2>(a, g.dtype, static_cast<hipStream_t>(stream));
}

namespace {
// Shapes of the matrix-core kernel families (16-bit, fp32 16-longitude, hybrid).  Their dq pass consumes the forward's output and normaliser; a backward
// that is not handed them (s2attn_backward, s2attn_backward_dq) first recomputes both into the tail of the workspace.
bool h16_shape(const s2attn_shape *sh)
{
    const int w = sh->nlon_out < sh->nlon_in ? sh->nlon_out : sh->nlon_in; // columns of a virtual latitude
    if (sh->ck != sh->cv || w < HK) return false;
    if (sh->dtype == S2ATTN_F32) return m32_width(sh->ck, sh->cv); // the fp32 16-longitude family and the hybrid kernels work the same way
    return h16_width(sh->ck, sh->cv);
}
int64_t stat_points(const s2attn_shape *sh) { return (int64_t)sh->batch * sh->num_heads * sh->nlat_out * sh->nlon_out; }
int64_t round16(int64_t n) { return (n + 15) / 16 * 16; }
} // namespace

extern "C" int64_t s2attn_backward_saved_workspace_bytes(const s2attn_shape *shape)
{
    const int rc = check_shape(shape);
    if (rc != S2ATTN_OK) return rc;
    return round16(stat_points(shape) * (int64_t)sizeof(float2));
}

extern "C" int64_t s2attn_backward_workspace_bytes(const s2attn_shape *shape)
{
    const int rc = check_shape(shape);
    if (rc != S2ATTN_OK) return rc;
    const int64_t n = stat_points(shape);
    int64_t bytes = round16(n * (int64_t)sizeof(float2));
    if (h16_shape(shape)) bytes += round16(n * 4) + n * shape->cv * esize(shape->dtype); // lse, y
    return bytes;
}

namespace {
int backward_args(Args &a, bool &vec, const void *k, const void *v, const void *q, const void *dy, const float *quad_weights, const void *workspace,
                  const s2attn_plan *plan, const s2attn_shape *shape)
{
    const int rc = check_shape(shape);
    if (rc != S2ATTN_OK) return rc;
    if (!k || !v || !q || !dy || !quad_weights || !workspace) return s2attn_fail(S2ATTN_E_INVALID, "null tensor pointer");
    const int rcp = check_plan(plan, shape);
    if (rcp != S2ATTN_OK) return rcp;
    if (!aligned(workspace, sizeof(float2))) return s2attn_fail(S2ATTN_E_INVALID, "workspace must be 8-byte aligned");
    fill_args(a, plan, shape, quad_weights);
    a.k = k, a.v = v, a.q = q, a.dy = dy;
    a.stats = static_cast<float2 *>(const_cast<void *>(workspace));
    const size_t al = 4 * (size_t)esize(shape->dtype);
    vec = shape->ck % 4 == 0 && shape->cv % 4 == 0 && aligned(k, al) && aligned(v, al) && aligned(q, al) && aligned(dy, al);
    return S2ATTN_OK;
}
} // namespace

extern "C" int s2attn_backward_dq(const void *k, const void *v, const void *q, const void *dy, const float *quad_weights, void *dq,
                                  void *workspace, const s2attn_plan *plan, const s2attn_shape *shape, void *stream)
{
    Args a = {};
    bool vec = false;
    const int rc = backward_args(a, vec, k, v, q, dy, quad_weights, workspace, plan, shape);
    if (rc != S2ATTN_OK) return rc;
    if (!dq) return s2attn_fail(S2ATTN_E_INVALID, "null tensor pointer");
    a.dq = dq;
    vec = vec && aligned(dq, 4 * (size_t)esize(shape->dtype));
    a.tile_rows = TQ - 1 + TL;
    if (h16_shape(shape) && aligned(workspace, 16)) {
        const int64_t n = stat_points(shape);
        char *ws = static_cast<char *>(workspace);
        float *lse = reinterpret_cast<float *>(ws + round16(n * (int64_t)sizeof(float2)));
        void *y = ws + round16(n * (int64_t)sizeof(float2)) + round16(n * 4);
        Args f = a;
        f.y = y, f.lse = lse, f.dq = nullptr, f.dy = nullptr;
        f.ldy = (unsigned)shape->num_heads * shape->cv; // the recomputed output in the workspace is packed
        a.ldy = f.ldy;
        const int rc2 = launch(FWD, f, shape->dtype, vec, plan->header[S2ATTN_PH_GATHER_NDENSE], static_cast<hipStream_t>(stream));
        if (rc2 != S2ATTN_OK) return rc2;
        a.ysaved = y, a.lse = lse;
    }
    return launch(DQ, a, shape->dtype, vec, plan->header[S2ATTN_PH_GATHER_NDENSE], static_cast<hipStream_t>(stream));
}

extern "C" int s2attn_backward_dq_saved(const void *k, const void *v, const void *q, const void *dy, const void *y, const float *lse,
                                        const float *quad_weights, void *dq, void *workspace, const s2attn_plan *plan,
                                        const s2attn_shape *shape, void *stream)
{
    Args a = {};
    bool vec = false;
    const int rc = backward_args(a, vec, k, v, q, dy, quad_weights, workspace, plan, shape);
    if (rc != S2ATTN_OK) return rc;
    if (!dq || !y || !lse) return s2attn_fail(S2ATTN_E_INVALID, "null tensor pointer");
    a.dq = dq;
    a.ysaved = y;
    a.lse = const_cast<float *>(lse);
    const size_t al = 4 * (size_t)esize(shape->dtype);
    vec = vec && aligned(dq, al) && aligned(y, al);
    a.tile_rows = TQ - 1 + TL;
    return launch(DQ, a, shape->dtype, vec, plan->header[S2ATTN_PH_GATHER_NDENSE], static_cast<hipStream_t>(stream));
}

extern "C" int s2attn_backward_dkdv(const void *k, const void *v, const void *q, const void *dy, const float *quad_weights,
                                    void *dk, void *dv, const void *workspace, const s2attn_plan *plan,
                                    const s2attn_shape *shape, void *stream)
{
    Args a = {};
    bool vec = false;
    const int rc = backward_args(a, vec, k, v, q, dy, quad_weights, workspace, plan, shape);
    if (rc != S2ATTN_OK) return rc;
    if (!dk || !dv) return s2attn_fail(S2ATTN_E_INVALID, "null tensor pointer");
    a.dk = dk, a.dv = dv;
    const size_t al = 4 * (size_t)esize(shape->dtype);
    vec = vec && aligned(dk, al) && aligned(dv, al);
    a.tile_rows = TQ + TL;
    if (a.tile_rows < TQ) a.tile_rows = TQ; // the tile also stages the lane-owned k/v and dk/dv rows
    return launch(DKDV, a, shape->dtype, vec, plan->header[S2ATTN_PH_SCATTER_NDENSE], static_cast<hipStream_t>(stream));
}

extern "C" int s2attn_backward_saved(const void *k, const void *v, const void *q, const void *dy, const void *y, const float *lse,
                                     const float *quad_weights, void *dk, void *dv, void *dq, void *workspace, const s2attn_plan *plan,
                                     const s2attn_shape *shape, void *stream)
{
    if (!dk || !dv || !dq) return s2attn_fail(S2ATTN_E_INVALID, "null tensor pointer");
    const int rc = s2attn_backward_dq_saved(k, v, q, dy, y, lse, quad_weights, dq, workspace, plan, shape, stream);
    if (rc != S2ATTN_OK) return rc;
    return s2attn_backward_dkdv(k, v, q, dy, quad_weights, dk, dv, workspace, plan, shape, stream);
}

extern "C" int s2attn_backward(const void *k, const void *v, const void *q, const void *dy, const float *quad_weights,
                               void *dk, void *dv, void *dq, void *workspace, const s2attn_plan *plan,
                               const s2attn_shape *shape, void *stream)
{
    if (!dk || !dv || !dq) return s2attn_fail(S2ATTN_E_INVALID, "null tensor pointer");
    const int rc = s2attn_backward_dq(k, v, q, dy, quad_weights, dq, workspace, plan, shape, stream);
    if (rc != S2ATTN_OK) return rc;
    return s2attn_backward_dkdv(k, v, q, dy, quad_weights, dk, dv, workspace, plan, shape, stream);
}

// ---------------------------------------------------------------------------------
// backward from saved statistics for callers that cannot allocate: the workspace is a device array of this library
// ---------------------------------------------------------------------------------
static __device__ __align__(256) unsigned char scratch[S2ATTN_NOALLOC_SCRATCH_BYTES];

namespace {
constexpr int MAX_DEVICES = 64;
std::mutex g_scratch_mutex;
void *g_scratch_ptr[MAX_DEVICES] = {}; // address of `scratch` on each device, looked up once per device
} // namespace

extern "C" int s2attn_backward_saved_noalloc(const void *k, const void *v, const void *q, const void *dy, const void *y, const float *lse,
                                             const float *quad_weights, void *dk, void *dv, void *dq, const s2attn_plan *plan,
                                             const s2attn_shape *shape, void *stream)
{
    const int64_t need = s2attn_backward_saved_workspace_bytes(shape);
    if (need < 0) return (int)need;
    if (need > (int64_t)S2ATTN_NOALLOC_SCRATCH_BYTES)
        return s2attn_fail(S2ATTN_E_UNSUPPORTED, "this shape needs %lld bytes of backward workspace, the built-in scratch array holds %lld; use s2attn_backward_saved with a caller-allocated workspace",
                           (long long)need, (long long)S2ATTN_NOALLOC_SCRATCH_BYTES);
    int dev = -1;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return s2attn_fail(S2ATTN_E_LAUNCH, "hipGetDevice: %s", hipGetErrorString(e));
    if (dev < 0 || dev >= MAX_DEVICES) return s2attn_fail(S2ATTN_E_UNSUPPORTED, "device ordinal %d is outside the %d this library keeps a scratch address for", dev, MAX_DEVICES);
    void *ws = nullptr;
    {
        std::lock_guard<std::mutex> lock(g_scratch_mutex);
        if (!g_scratch_ptr[dev]) { // every device holds its own copy of the array at its own address
            void *p = nullptr;
            e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
            if (e != hipSuccess || !p) return s2attn_fail(S2ATTN_E_LAUNCH, "hipGetSymbolAddress(scratch): %s", hipGetErrorString(e));
            g_scratch_ptr[dev] = p;
        }
        ws = g_scratch_ptr[dev];
    }
    // the dq pass writes both statistics of every (batch, head, output point) before the dk/dv pass reads them, so
    // nothing of a previous call's contents is ever read and nothing needs clearing
    return s2attn_backward_saved(k, v, q, dy, y, lse, quad_weights, dk, dv, dq, ws, plan, shape, stream);
}

namespace {
template <typename E> int launch_transpose(const void *src, void *dst, long nb, long R, long S, hipStream_t stream)
{
    if (nb == 0 || R == 0 || S == 0) return S2ATTN_OK;
    const long gx = (S + 63) / 64, gy = (R + 63) / 64;
    if (gx > 0x7fffffffL || gy > 0x7fffffffL || nb > 0x7fffffffL || gx * gy > 0x7fffffffL || gx * gy * nb > 0x7fffffffL)
        return s2attn_fail(S2ATTN_E_UNSUPPORTED, "permute needs %ld x %ld x %ld workgroups, more than one grid holds", gx, gy, nb);
    hipLaunchKernelGGL(s2::transpose_kernel<E>, dim3((unsigned)(gx * gy * nb)), dim3(256), 0, stream, static_cast<const E *>(src),
                       static_cast<E *>(dst), R, S, (unsigned)gx, (unsigned)gy);
    const hipError_t e = hipGetLastError();
    if (e != hipSuccess) return s2attn_fail(S2ATTN_E_LAUNCH, "kernel launch: %s", hipGetErrorString(e));
    return S2ATTN_OK;
}

int permute(const void *src, void *dst, long nb, long R, long S, int elem_size, void *stream)
{
    if (nb < 0 || R < 0 || S < 0) return s2attn_fail(S2ATTN_E_INVALID, "negative extent");
    if ((!src || !dst) && nb * R * S > 0) return s2attn_fail(S2ATTN_E_INVALID, "null tensor pointer");
    hipStream_t st = static_cast<hipStream_t>(stream);
    switch (elem_size) {
    case 2: return launch_transpose<unsigned short>(src, dst, nb, R, S, st);
    case 4: return launch_transpose<unsigned int>(src, dst, nb, R, S, st);
    case 8: return launch_transpose<unsigned long long>(src, dst, nb, R, S, st);
    default: return s2attn_fail(S2ATTN_E_INVALID, "element size %d is not 2, 4 or 8 bytes", elem_size);
    }
}
} // namespace

extern "C" int s2attn_permute_to_nhwc(const void *src, void *dst, int64_t B, int64_t C, int64_t H, int64_t W, int elem_size, void *stream)
{
    return permute(src, dst, B, C, H * W, elem_size, stream); // [C, HW] -> [HW, C]
}

extern "C" int s2attn_permute_to_nchw(const void *src, void *dst, int64_t B, int64_t H, int64_t W, int64_t C, int elem_size, void *stream)
{
    return permute(src, dst, B, H * W, C, elem_size, stream); // [HW, C] -> [C, HW]
}
#endif // S2_PART <= 1
