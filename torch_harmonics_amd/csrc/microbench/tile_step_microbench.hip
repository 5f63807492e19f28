// Cost of one matrix-core tile step of the forward (32 queries x 32 band positions, 32 channels), two ways (gfx950):
//
//   F32     what the hybrid kernels run today: S^T = K Q^T and Y^T += V^T P^T as 16 + 16 v_mfma_f32_32x32x2_f32, operands from an
//           fp32 LDS tile (row pitch 144 B), staged rows written as they are.
//   BF16    the same products on v_mfma_f32_32x32x16_bf16 with fp32 operands split into bf16 terms (round-to-nearest, x = h + m + l
//           to 2^-25): with three terms per value a product is the six term products with i + j <= 4, with two terms three.
//           K and V are split when a staged row is committed to LDS (planes [row][term][32 channels], channel order so that a
//           lane's operand is one 16-byte read); P is split in registers; V^T comes from transposing LDS reads.  Variants:
//           KT terms for K and q (the scores), PT terms for P and V (the output sums).
//
// Each wave loops over tile steps exactly as the kernels do (prefetch of the next tile from global memory into registers,
// products, softmax with a running maximum, barrier, commit, barrier).  The program first checks both variants against a
// float64 evaluation on the host, then times them at 1, 2 and 3 waves per SIMD.
//
// Build and run:  make -C torch_harmonics_amd/csrc microbench && torch_harmonics_amd/csrc/build/tile_step_microbench
#include <hip/hip_runtime.h>
#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <vector>

#define CHECK(x)                                                                       \
    do {                                                                               \
        hipError_t e_ = (x);                                                           \
        if (e_ != hipSuccess) {                                                        \
            fprintf(stderr, "%s:%d: %s\n", __FILE__, __LINE__, hipGetErrorString(e_)); \
            exit(1);                                                                   \
        }                                                                              \
    } while (0)

typedef float f16v __attribute__((ext_vector_type(16)));
typedef float f2v __attribute__((ext_vector_type(2)));
typedef float f4v __attribute__((ext_vector_type(4)));
typedef unsigned u4v __attribute__((ext_vector_type(4)));
typedef unsigned u2v __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef short s16x4 __attribute__((ext_vector_type(4)));

constexpr int MT = 32;
constexpr int MLK = 36;          // fp32 tile: floats per row
constexpr int P3 = 208;          // bf16 tile with three terms: bytes per row (3 x 64 + 16)
constexpr int NROWS = 4096;      // rows of the synthetic K and V (wraps)
constexpr float NEG_BIG = -1e30f;

__device__ inline int kappa(int v, int half) { return 8 * (v / 4) + 4 * half + (v % 4); }
__device__ inline float xor32(float x) { return __shfl_xor(x, 32); }
__device__ inline float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }
__device__ inline unsigned pk_bf16(float a, float b)
{
    f2v x = {a, b};
    return __builtin_bit_cast(unsigned, __builtin_convertvector(x, bf16x2));
}
__device__ inline float lo_f32(unsigned p) { return __uint_as_float(p << 16); }
__device__ inline float hi_f32(unsigned p) { return __uint_as_float(p & 0xffff0000u); }
// two floats -> three (two) packed bf16 terms, round to nearest, each term the rounding of what the earlier ones left
__device__ inline void split3(float a, float b, unsigned &h, unsigned &m, unsigned &l)
{
    h = pk_bf16(a, b);
    const float ra = a - lo_f32(h), rb = b - hi_f32(h);
    m = pk_bf16(ra, rb);
    l = pk_bf16(ra - lo_f32(m), rb - hi_f32(m));
}
__device__ inline void split2(float a, float b, unsigned &h, unsigned &m)
{
    h = pk_bf16(a, b);
    m = pk_bf16(a - lo_f32(h), b - hi_f32(h));
}
__device__ inline bf16x8 as_bf16x8(u4v x) { return __builtin_bit_cast(bf16x8, x); }

struct Out {
    float *y;   // [waves][32 queries][32 channels] un-normalised sums
    float *s;   // [waves][32 queries] normaliser
    float *m;   // [waves][32 queries] running maximum
};

// ---- F32 ---------------------------------------------------------------------------------------------------------------------
__global__ __launch_bounds__(64) void tile_f32(const float *__restrict__ K, const float *__restrict__ V, const float *__restrict__ Q, Out out, int steps)
{
    __shared__ __attribute__((aligned(16))) float Ks[MT * MLK];
    __shared__ __attribute__((aligned(16))) float Vs[MT * MLK];
    const int lane = threadIdx.x, j = lane & 31, half = lane >> 5;
    const int wave = blockIdx.x;
    float qb[16];
    for (int g = 0; g < 4; g++)
        for (int e = 0; e < 4; e++) qb[4 * g + e] = Q[j * 32 + 8 * g + 4 * half + e];
    f16v acc;
    for (int v = 0; v < 16; v++) acc[v] = 0.f;
    float m = NEG_BIG, S = 0.f;
    const float w = 1.0f;
    f4v kraw[4], vraw[4];
    const int r0 = lane >> 3, cb = 4 * (lane & 7);
    int base = (wave * 37) % NROWS;
    auto fetch = [&](int row0) {
        for (int it = 0; it < 4; it++) {
            const int r = (row0 + r0 + 8 * it) % NROWS;
            kraw[it] = *reinterpret_cast<const f4v *>(K + (size_t)r * 32 + cb);
            vraw[it] = *reinterpret_cast<const f4v *>(V + (size_t)r * 32 + cb);
        }
    };
    auto commit = [&]() {
        for (int it = 0; it < 4; it++) {
            *reinterpret_cast<f4v *>(Ks + (r0 + 8 * it) * MLK + cb) = kraw[it];
            *reinterpret_cast<f4v *>(Vs + (r0 + 8 * it) * MLK + cb) = vraw[it];
        }
    };
    fetch(base);
    commit();
    __syncthreads();
    for (int st = 0; st < steps; st++) {
        if (st + 1 < steps) fetch(base + 32 * (st + 1));
        const float *kq = Ks + j * MLK + 4 * half;
        f16v sc;
        for (int v = 0; v < 16; v++) sc[v] = 0.f;
#pragma unroll
        for (int g = 0; g < 4; g++) {
            const f4v x = *reinterpret_cast<const f4v *>(kq + 8 * g);
            sc = __builtin_amdgcn_mfma_f32_32x32x2f32(x[0], qb[4 * g + 0], sc, 0, 0, 0);
            sc = __builtin_amdgcn_mfma_f32_32x32x2f32(x[1], qb[4 * g + 1], sc, 0, 0, 0);
            sc = __builtin_amdgcn_mfma_f32_32x32x2f32(x[2], qb[4 * g + 2], sc, 0, 0, 0);
            sc = __builtin_amdgcn_mfma_f32_32x32x2f32(x[3], qb[4 * g + 3], sc, 0, 0, 0);
        }
        float mx = sc[0];
#pragma unroll
        for (int v = 1; v < 16; v++) mx = fmaxf(mx, sc[v]);
        mx = fmaxf(mx, xor32(mx));
        const float mn = fmaxf(m, mx);
        if (__any(mn > m)) {
            const float corr = fast_exp2(m - mn);
            S *= corr;
#pragma unroll
            for (int v = 0; v < 16; v++) acc[v] *= corr;
        }
        m = mn;
        float rs = 0.f;
#pragma unroll
        for (int v = 0; v < 16; v++) {
            const float p = fast_exp2(sc[v] - mn) * w;
            sc[v] = p;
            rs += p;
        }
        rs += xor32(rs);
        S += rs;
#pragma unroll
        for (int v = 0; v < 16; v++) {
            const float x = Vs[kappa(v, half) * MLK + j];
            acc = __builtin_amdgcn_mfma_f32_32x32x2f32(x, sc[v], acc, 0, 0, 0);
        }
        __syncthreads();
        if (st + 1 < steps) commit();
        __syncthreads();
    }
    for (int g = 0; g < 4; g++)
        for (int e = 0; e < 4; e++) out.y[((size_t)wave * 32 + j) * 32 + 8 * g + 4 * half + e] = acc[4 * g + e];
    if (half == 0) {
        out.s[wave * 32 + j] = S;
        out.m[wave * 32 + j] = m;
    }
}

// ---- BF16x3 -------------------------------------------------------------------------------------------------------------------
// LDS row of a split tile: term t of channel c at byte 64 t + 2 (16 hh + 4 g + e), c = 8 g + 4 hh + e: the 16 channels a lane
// (row, hh) feeds to the two matrix instructions of a product are 32 contiguous bytes.
template <int KTERMS, int PTERMS> __global__ __launch_bounds__(64) void tile_bf16(const float *__restrict__ K, const float *__restrict__ V, const float *__restrict__ Q, Out out, int steps)
{
    __shared__ __attribute__((aligned(16))) char Ks[MT * P3];
    __shared__ __attribute__((aligned(16))) char Vs[MT * P3];
    typedef s16x4 __attribute__((address_space(3))) * tr_ptr;
    const int lane = threadIdx.x, j = lane & 31, half = lane >> 5;
    const int wave = blockIdx.x;
    // q: channels 8 g + 4 half + e as three packed terms; qh[n] is the B operand of matrix instruction n (channels g = 2n, 2n + 1)
    u4v qh[2], qm[2], ql[2];
    for (int n = 0; n < 2; n++)
        for (int i = 0; i < 4; i++) {
            const int g = 2 * n + i / 2, e = 2 * (i % 2);
            unsigned h_, m_, l_;
            split3(Q[j * 32 + 8 * g + 4 * half + e], Q[j * 32 + 8 * g + 4 * half + e + 1], h_, m_, l_);
            qh[n][i] = h_, qm[n][i] = m_, ql[n][i] = l_;
        }
    f16v acc;
    for (int v = 0; v < 16; v++) acc[v] = 0.f;
    float m = NEG_BIG, S = 0.f;
    const float w = 1.0f;
    f4v kraw[4], vraw[4];
    const int r0 = lane >> 3, c8 = lane & 7, cb = 4 * c8;
    const int woff = 32 * (c8 & 1) + 8 * (c8 >> 1); // byte offset of this lane's four channels inside a term of a row
    int base = (wave * 37) % NROWS;
    auto fetch = [&](int row0) {
        for (int it = 0; it < 4; it++) {
            const int r = (row0 + r0 + 8 * it) % NROWS;
            kraw[it] = *reinterpret_cast<const f4v *>(K + (size_t)r * 32 + cb);
            vraw[it] = *reinterpret_cast<const f4v *>(V + (size_t)r * 32 + cb);
        }
    };
    auto commit = [&]() {
        for (int it = 0; it < 4; it++) {
            unsigned h0, m0, l0, h1, m1, l1;
            split3(kraw[it][0], kraw[it][1], h0, m0, l0);
            split3(kraw[it][2], kraw[it][3], h1, m1, l1);
            char *kr = Ks + (r0 + 8 * it) * P3 + woff;
            *reinterpret_cast<u2v *>(kr) = u2v{h0, h1};
            *reinterpret_cast<u2v *>(kr + 64) = u2v{m0, m1};
            if (KTERMS == 3) *reinterpret_cast<u2v *>(kr + 128) = u2v{l0, l1};
            if (PTERMS == 3) {
                split3(vraw[it][0], vraw[it][1], h0, m0, l0);
                split3(vraw[it][2], vraw[it][3], h1, m1, l1);
            } else {
                split2(vraw[it][0], vraw[it][1], h0, m0);
                split2(vraw[it][2], vraw[it][3], h1, m1);
            }
            char *vr = Vs + (r0 + 8 * it) * P3 + woff;
            *reinterpret_cast<u2v *>(vr) = u2v{h0, h1};
            *reinterpret_cast<u2v *>(vr + 64) = u2v{m0, m1};
            if (PTERMS == 3) *reinterpret_cast<u2v *>(vr + 128) = u2v{l0, l1};
        }
    };
    // transposing read of V^T: source lane s of 16-lane group G addresses row 4 (G / 2) + (s % 16) / 4 (+ 8 a + 16 n), channels
    // 4 (4 (G % 2) + s % 4) .. + 3; the lane receives its own channel (lane % 32) of four rows
    const int G = lane >> 4, es = (lane & 15) >> 2, t = lane & 3;
    const int cbs = 4 * (G & 1) + t;
    const int troff = (4 * (G >> 1) + es) * P3 + 32 * (cbs & 1) + 8 * (cbs >> 1);

    fetch(base);
    commit();
    __syncthreads();
    for (int st = 0; st < steps; st++) {
        if (st + 1 < steps) fetch(base + 32 * (st + 1));
        // ---- S^T = K Q^T: low-order products first ----
        const char *kq = Ks + j * P3 + 32 * half;
        f16v sc;
        for (int v = 0; v < 16; v++) sc[v] = 0.f;
        u4v kh[2], km[2], kl[2];
#pragma unroll
        for (int n = 0; n < 2; n++) {
            kh[n] = *reinterpret_cast<const u4v *>(kq + 16 * n);
            km[n] = *reinterpret_cast<const u4v *>(kq + 64 + 16 * n);
            if (KTERMS == 3) kl[n] = *reinterpret_cast<const u4v *>(kq + 128 + 16 * n);
        }
#pragma unroll
        for (int n = 0; n < 2; n++) {
            if (KTERMS == 3) {
                sc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(as_bf16x8(kl[n]), as_bf16x8(qh[n]), sc, 0, 0, 0);
                sc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(as_bf16x8(kh[n]), as_bf16x8(ql[n]), sc, 0, 0, 0);
                sc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(as_bf16x8(km[n]), as_bf16x8(qm[n]), sc, 0, 0, 0);
            }
            sc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(as_bf16x8(km[n]), as_bf16x8(qh[n]), sc, 0, 0, 0);
            sc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(as_bf16x8(kh[n]), as_bf16x8(qm[n]), sc, 0, 0, 0);
        }
#pragma unroll
        for (int n = 0; n < 2; n++) sc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(as_bf16x8(kh[n]), as_bf16x8(qh[n]), sc, 0, 0, 0);
        float mx = sc[0];
#pragma unroll
        for (int v = 1; v < 16; v++) mx = fmaxf(mx, sc[v]);
        mx = fmaxf(mx, xor32(mx));
        const float mn = fmaxf(m, mx);
        if (__any(mn > m)) {
            const float corr = fast_exp2(m - mn);
            S *= corr;
#pragma unroll
            for (int v = 0; v < 16; v++) acc[v] *= corr;
        }
        m = mn;
        float rs = 0.f;
        u4v ph[2], pm[2], pl[2];
#pragma unroll
        for (int v = 0; v < 16; v += 2) {
            const float p0 = fast_exp2(sc[v] - mn) * w, p1 = fast_exp2(sc[v + 1] - mn) * w;
            rs += p0 + p1;
            unsigned h_, m_, l_ = 0;
            if (PTERMS == 3)
                split3(p0, p1, h_, m_, l_);
            else
                split2(p0, p1, h_, m_);
            ph[v / 8][(v % 8) / 2] = h_;
            pm[v / 8][(v % 8) / 2] = m_;
            pl[v / 8][(v % 8) / 2] = l_;
        }
        rs += xor32(rs);
        S += rs;
        // ---- Y^T += V^T P^T ----
#pragma unroll
        for (int n = 0; n < 2; n++) {
            u4v vh, vm, vl;
#pragma unroll
            for (int a = 0; a < 2; a++) {
                const char *p = Vs + troff + (16 * n + 8 * a) * P3;
                const s16x4 x = __builtin_amdgcn_ds_read_tr16_b64_v4i16((tr_ptr)(p));
                const s16x4 y = __builtin_amdgcn_ds_read_tr16_b64_v4i16((tr_ptr)(p + 64));
                const u2v xu = __builtin_bit_cast(u2v, x), yu = __builtin_bit_cast(u2v, y);
                vh[2 * a] = xu[0], vh[2 * a + 1] = xu[1];
                vm[2 * a] = yu[0], vm[2 * a + 1] = yu[1];
                if (PTERMS == 3) {
                    const u2v zu = __builtin_bit_cast(u2v, __builtin_amdgcn_ds_read_tr16_b64_v4i16((tr_ptr)(p + 128)));
                    vl[2 * a] = zu[0], vl[2 * a + 1] = zu[1];
                }
            }
            if (PTERMS == 3) {
                acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(as_bf16x8(vl), as_bf16x8(ph[n]), acc, 0, 0, 0);
                acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(as_bf16x8(vh), as_bf16x8(pl[n]), acc, 0, 0, 0);
                acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(as_bf16x8(vm), as_bf16x8(pm[n]), acc, 0, 0, 0);
            }
            acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(as_bf16x8(vm), as_bf16x8(ph[n]), acc, 0, 0, 0);
            acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(as_bf16x8(vh), as_bf16x8(pm[n]), acc, 0, 0, 0);
            acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(as_bf16x8(vh), as_bf16x8(ph[n]), acc, 0, 0, 0);
        }
        __syncthreads();
        if (st + 1 < steps) commit();
        __syncthreads();
    }
    for (int g = 0; g < 4; g++)
        for (int e = 0; e < 4; e++) out.y[((size_t)wave * 32 + j) * 32 + 8 * g + 4 * half + e] = acc[4 * g + e];
    if (half == 0) {
        out.s[wave * 32 + j] = S;
        out.m[wave * 32 + j] = m;
    }
}

template <typename F> float time_kernel(F launch)
{
    hipEvent_t e0, e1;
    CHECK(hipEventCreate(&e0));
    CHECK(hipEventCreate(&e1));
    launch();
    CHECK(hipEventRecord(e0));
    launch();
    CHECK(hipEventRecord(e1));
    CHECK(hipEventSynchronize(e1));
    float ms = 0;
    CHECK(hipEventElapsedTime(&ms, e0, e1));
    CHECK(hipEventDestroy(e0));
    CHECK(hipEventDestroy(e1));
    return ms;
}

int main()
{
    const int maxwaves = 256 * 4 * 3;
    std::vector<float> hK((size_t)NROWS * 32), hV((size_t)NROWS * 32), hQ(32 * 32);
    srand(333);
    auto rnd = []() { float u = 0; for (int i = 0; i < 12; i++) u += rand() / (float)RAND_MAX; return u - 6.0f; }; // ~N(0,1)
    for (auto &x : hK) x = rnd();
    for (auto &x : hV) x = rnd();
    for (auto &x : hQ) x = rnd() * 1.4426950408889634f / sqrtf(32.f);
    float *K, *V, *Q;
    Out out;
    CHECK(hipMalloc(&K, hK.size() * 4));
    CHECK(hipMalloc(&V, hV.size() * 4));
    CHECK(hipMalloc(&Q, hQ.size() * 4));
    CHECK(hipMalloc(&out.y, (size_t)maxwaves * 32 * 32 * 4));
    CHECK(hipMalloc(&out.s, (size_t)maxwaves * 32 * 4));
    CHECK(hipMalloc(&out.m, (size_t)maxwaves * 32 * 4));
    CHECK(hipMemcpy(K, hK.data(), hK.size() * 4, hipMemcpyHostToDevice));
    CHECK(hipMemcpy(V, hV.data(), hV.size() * 4, hipMemcpyHostToDevice));
    CHECK(hipMemcpy(Q, hQ.data(), hQ.size() * 4, hipMemcpyHostToDevice));

    // ---- numerics: wave 0, `csteps` tile steps, against float64 ----
    const int csteps = 24; // 768 keys per query
    std::vector<double> ry(32 * 32), rs(32);
    for (int q = 0; q < 32; q++) {
        std::vector<double> s(csteps * 32);
        double mx = -1e300;
        for (int r = 0; r < csteps * 32; r++) {
            double a = 0;
            for (int c = 0; c < 32; c++) a += (double)hQ[q * 32 + c] * hK[(size_t)r * 32 + c];
            s[r] = a;
            mx = std::max(mx, a);
        }
        double S = 0;
        std::vector<double> y(32, 0.0);
        for (int r = 0; r < csteps * 32; r++) {
            const double p = std::exp2(s[r] - mx);
            S += p;
            for (int c = 0; c < 32; c++) y[c] += p * hV[(size_t)r * 32 + c];
        }
        for (int c = 0; c < 32; c++) ry[q * 32 + c] = y[c] / S;
        rs[q] = mx + std::log2(S);
    }
    auto check = [&](const char *name) {
        std::vector<float> y(32 * 32), s(32), m(32);
        CHECK(hipMemcpy(y.data(), out.y, y.size() * 4, hipMemcpyDeviceToHost));
        CHECK(hipMemcpy(s.data(), out.s, s.size() * 4, hipMemcpyDeviceToHost));
        CHECK(hipMemcpy(m.data(), out.m, m.size() * 4, hipMemcpyDeviceToHost));
        double ey = 0, el = 0;
        for (int q = 0; q < 32; q++) {
            for (int c = 0; c < 32; c++) ey = std::max(ey, std::fabs(y[q * 32 + c] / s[q] - ry[q * 32 + c]));
            el = std::max(el, std::fabs(m[q] + std::log2((double)s[q]) - rs[q]));
        }
        printf("  %-22s max |y - y64| = %.3e   max |lse - lse64| = %.3e   (y of size 0.1-1, %d keys per query)\n", name, ey, el, csteps * 32);
    };
    printf("numerics of one wave against float64:\n");
    hipLaunchKernelGGL(tile_f32, dim3(1), dim3(64), 0, 0, K, V, Q, out, csteps);
    CHECK(hipDeviceSynchronize());
    check("F32");
    hipLaunchKernelGGL((tile_bf16<3, 3>), dim3(1), dim3(64), 0, 0, K, V, Q, out, csteps);
    CHECK(hipDeviceSynchronize());
    check("BF16 KT=3 PT=3");
    hipLaunchKernelGGL((tile_bf16<3, 2>), dim3(1), dim3(64), 0, 0, K, V, Q, out, csteps);
    CHECK(hipDeviceSynchronize());
    check("BF16 KT=3 PT=2");
    hipLaunchKernelGGL((tile_bf16<2, 2>), dim3(1), dim3(64), 0, 0, K, V, Q, out, csteps);
    CHECK(hipDeviceSynchronize());
    check("BF16 KT=2 PT=2");

    // ---- time per tile step ----
    const int steps = 400;
    printf("\ntime per tile step (32 queries x 32 positions x 32 channels, forward), ns of SIMD time = launch time / steps / waves per SIMD:\n");
    printf("  %-10s %-12s %-16s %-16s %-16s\n", "waves/SIMD", "F32", "BF16 KT=3 PT=3", "BF16 KT=3 PT=2", "BF16 KT=2 PT=2");
    for (int wps : {1, 2, 3}) {
        const int blocks = 256 * 4 * wps;
        const float a = time_kernel([&] { hipLaunchKernelGGL(tile_f32, dim3(blocks), dim3(64), 0, 0, K, V, Q, out, steps); });
        const float b = time_kernel([&] { hipLaunchKernelGGL((tile_bf16<3, 3>), dim3(blocks), dim3(64), 0, 0, K, V, Q, out, steps); });
        const float c = time_kernel([&] { hipLaunchKernelGGL((tile_bf16<3, 2>), dim3(blocks), dim3(64), 0, 0, K, V, Q, out, steps); });
        const float d = time_kernel([&] { hipLaunchKernelGGL((tile_bf16<2, 2>), dim3(blocks), dim3(64), 0, 0, K, V, Q, out, steps); });
        printf("  %-10d %-12.1f %-16.1f %-16.1f %-16.1f\n", wps, a * 1e6 / steps / wps, b * 1e6 / steps / wps, c * 1e6 / steps / wps, d * 1e6 / steps / wps);
    }
    return 0;
}
