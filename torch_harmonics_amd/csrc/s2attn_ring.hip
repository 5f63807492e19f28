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
constexpr int NCI = MAXC / 64; // channels per lane

struct Args {
    const void *k, *v, *q, *dy;
    float *y_acc, *alpha_sum, *qdotk_max, *integral, *alpha_k, *alpha_kvw; // state (read-only in pass 2 where they are inputs)
    const float *integral_norm;
    float *dk, *dv;
    const float *quad_w;
    const int64_t *col_idx, *row_off;
    const int32_t *row_idx; // launch order of the output latitudes (may be null: natural order)
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

// Forward: folds the chunk into (y_acc, alpha_sum, qdotk_max).  attention_cuda_fwd_ring.cu:66-175.
template <typename T> __global__ __launch_bounds__(256) void fwd_kernel(const Args a)
{
    int b, ho, wo, lane;
    if (!locate(a, b, ho, wo, lane)) return;
    const long out = ((long)b * a.Ho + ho) * a.Wo + wo;
    const T *q = static_cast<const T *>(a.q) + out * a.ck;
    const T *kx = static_cast<const T *>(a.k) + (long)b * a.nlat_halo * a.nlon_kx * a.ck;
    const T *vx = static_cast<const T *>(a.v) + (long)b * a.nlat_halo * a.nlon_kx * a.cv;
    float qr[NCI], y[NCI];
#pragma unroll
    for (int i = 0; i < NCI; i++) {
        const int c = lane + 64 * i;
        qr[i] = c < a.ck ? ld(q + c) : 0.f;
        y[i] = c < a.cv ? a.y_acc[out * a.cv + c] : 0.f;
    }
    float S = a.alpha_sum[out], m = a.qdotk_max[out];
    for (int64_t z = a.row_off[ho]; z < a.row_off[ho + 1]; z++) {
        int hi;
        const long pt = chunk_point(a, a.col_idx[z], wo, hi);
        if (pt < 0) continue;
        const T *kr = kx + pt * a.ck, *vr = vx + pt * a.cv;
        float s = 0.f;
#pragma unroll
        for (int i = 0; i < NCI; i++) {
            const int c = lane + 64 * i;
            if (c < a.ck) s = fmaf(qr[i], ld(kr + c), s);
        }
        s = wave_sum(s);
        const float mn = fmaxf(m, s);
        const float alpha = __expf(s - mn) * a.quad_w[hi];
        const float corr = __expf(m - mn); // m = -inf on the first neighbor: 0
        S = alpha + S * corr;
#pragma unroll
        for (int i = 0; i < NCI; i++) {
            const int c = lane + 64 * i;
            if (c < a.cv) y[i] = fmaf(alpha, ld(vr + c), y[i] * corr);
        }
        m = mn;
    }
    if (lane == 0) {
        a.alpha_sum[out] = S;
        a.qdotk_max[out] = m;
    }
#pragma unroll
    for (int i = 0; i < NCI; i++) {
        const int c = lane + 64 * i;
        if (c < a.cv) a.y_acc[out * a.cv + c] = y[i];
    }
}

// Backward pass 1: folds the chunk into (alpha_sum, qdotk_max, integral = sum alpha <dy, v>, alpha_k = sum alpha k,
// alpha_kvw = sum alpha <dy, v> k).  attention_cuda_bwd_ring.cu:78-205.
template <typename T> __global__ __launch_bounds__(256) void pass1_kernel(const Args a)
{
    int b, ho, wo, lane;
    if (!locate(a, b, ho, wo, lane)) return;
    const long out = ((long)b * a.Ho + ho) * a.Wo + wo;
    const T *q = static_cast<const T *>(a.q) + out * a.ck;
    const T *g = static_cast<const T *>(a.dy) + out * a.cv;
    const T *kx = static_cast<const T *>(a.k) + (long)b * a.nlat_halo * a.nlon_kx * a.ck;
    const T *vx = static_cast<const T *>(a.v) + (long)b * a.nlat_halo * a.nlon_kx * a.cv;
    float qr[NCI], gr[NCI], ak[NCI], akg[NCI];
#pragma unroll
    for (int i = 0; i < NCI; i++) {
        const int c = lane + 64 * i;
        qr[i] = c < a.ck ? ld(q + c) : 0.f;
        gr[i] = c < a.cv ? ld(g + c) : 0.f;
        ak[i] = c < a.ck ? a.alpha_k[out * a.ck + c] : 0.f;
        akg[i] = c < a.ck ? a.alpha_kvw[out * a.ck + c] : 0.f;
    }
    float S = a.alpha_sum[out], m = a.qdotk_max[out], I = a.integral[out];
    for (int64_t z = a.row_off[ho]; z < a.row_off[ho + 1]; z++) {
        int hi;
        const long pt = chunk_point(a, a.col_idx[z], wo, hi);
        if (pt < 0) continue;
        const T *kr = kx + pt * a.ck, *vr = vx + pt * a.cv;
        float s = 0.f, gv = 0.f, kv[NCI];
#pragma unroll
        for (int i = 0; i < NCI; i++) {
            const int c = lane + 64 * i;
            kv[i] = c < a.ck ? ld(kr + c) : 0.f;
            s = fmaf(qr[i], kv[i], s);
            if (c < a.cv) gv = fmaf(gr[i], ld(vr + c), gv);
        }
        s = wave_sum(s);
        gv = wave_sum(gv);
        const float mn = fmaxf(m, s);
        const float alpha = __expf(s - mn) * a.quad_w[hi];
        const float corr = __expf(m - mn);
        S = S * corr + alpha;
        I = I * corr + alpha * gv;
        const float ag = alpha * gv;
#pragma unroll
        for (int i = 0; i < NCI; i++) {
            ak[i] = fmaf(alpha, kv[i], ak[i] * corr);
            akg[i] = fmaf(ag, kv[i], akg[i] * corr);
        }
        m = mn;
    }
    if (lane == 0) {
        a.alpha_sum[out] = S;
        a.qdotk_max[out] = m;
        a.integral[out] = I;
    }
#pragma unroll
    for (int i = 0; i < NCI; i++) {
        const int c = lane + 64 * i;
        if (c < a.ck) {
            a.alpha_k[out * a.ck + c] = ak[i];
            a.alpha_kvw[out * a.ck + c] = akg[i];
        }
    }
}

// Backward pass 2: with the final statistics, adds this chunk's dk and dv (fp32, atomically: several output points
// see the same input point).  attention_cuda_bwd_ring.cu:1312-1440.
template <typename T> __global__ __launch_bounds__(256) void pass2_kernel(const Args a)
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

enum Step { FWD, PASS1, PASS2 };

template <typename T> int launch_t(Step step, const Args &a, hipStream_t stream)
{
    const long npts = (long)a.B * a.Ho * a.Wo;
    const long nblocks = (npts + 3) / 4;
    if (nblocks > 0x7fffffffL) return s2attn_fail(S2ATTN_E_UNSUPPORTED, "problem needs %ld workgroups, more than one grid holds", nblocks);
    void (*kern)(const Args) = step == FWD ? fwd_kernel<T> : step == PASS1 ? pass1_kernel<T> : pass2_kernel<T>;
    hipLaunchKernelGGL(kern, dim3((unsigned)nblocks), dim3(256), 0, stream, a);
    const hipError_t e = hipGetLastError();
    if (e != hipSuccess) return s2attn_fail(S2ATTN_E_LAUNCH, "kernel launch: %s", hipGetErrorString(e));
    return S2ATTN_OK;
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
