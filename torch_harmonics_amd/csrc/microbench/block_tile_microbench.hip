// What a short-run latitude of the dq pass would cost if a workgroup staged the K and V rows of several adjacent output latitudes
// ONCE and every wavefront then walked all its runs from LDS (gfx950) - against the hybrid kernel's one staging per run.
//
// Workgroup = NW wavefronts; wavefront w owns output latitude ho0 + w, longitudes w0 .. w0 + 31 (two lanes per query, sixteen
// channels per lane).  The equatorial neighborhood of a 721 x 1440 grid with a cutoff of three spacings is used: seven input
// latitudes ho - 3 .. ho + 3 with runs of 1, 5, 5, 7, 5, 5, 1 longitudes centred on the query (29 neighbors).  The workgroup stages
// input latitudes ho0 - 3 .. ho0 + NW + 2, columns w0 - 4 .. w0 + 35 (40 rows of 144 B per latitude and tensor) - NW = 8 fills a
// CU's LDS (157.5 KB) - then every wavefront does its 29 row steps (row_step_microbench.hip) without further staging or barriers.
// Tensors have the layout of the benchmark configuration: 8 heads of 32 fp32 channels packed per grid point (1 KB per point).
//
// Build and run:  make -C torch_harmonics_amd/csrc microbench && torch_harmonics_amd/csrc/build/block_tile_microbench
#include <hip/hip_runtime.h>
#include <cstdio>
#include <cstdlib>

#define CHECK(x)                                                                       \
    do {                                                                               \
        hipError_t e_ = (x);                                                           \
        if (e_ != hipSuccess) {                                                        \
            fprintf(stderr, "%s:%d: %s\n", __FILE__, __LINE__, hipGetErrorString(e_)); \
            exit(1);                                                                   \
        }                                                                              \
    } while (0)

constexpr int MLK = 36;  // floats per staged row
constexpr int NCOL = 40; // staged columns per latitude
constexpr int HALO = 3;
constexpr int W = 1440, LD = 256; // longitudes, floats per grid point (8 heads x 32 channels)

extern __shared__ float4 smem[];

__device__ inline float xor32_sum(float x)
{
    const auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
    return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}
__device__ inline void read_row(float (&x)[16], const float *row)
{
#pragma unroll
    for (int g = 0; g < 4; g++) {
        const float4 t = *reinterpret_cast<const float4 *>(row + 8 * g);
        x[4 * g + 0] = t.x, x[4 * g + 1] = t.y, x[4 * g + 2] = t.z, x[4 * g + 3] = t.w;
    }
}
__device__ inline float dot16(const float (&a)[16], const float (&b)[16])
{
    float c[4];
#pragma unroll
    for (int g = 0; g < 4; g++) {
        c[g] = a[4 * g] * b[4 * g];
#pragma unroll
        for (int e = 1; e < 4; e++) c[g] = fmaf(a[4 * g + e], b[4 * g + e], c[g]);
    }
    return (c[0] + c[1]) + (c[2] + c[3]);
}

template <int LEN> __device__ inline void run_steps(float (&dq)[16], const float (&q)[16], const float (&dy)[16], const float *kq, const float *vq, float lse, float I, float w)
{
#pragma unroll
    for (int t = 0; t < LEN; t++) {
        float k[16], v[16];
        read_row(k, kq + t * MLK);
        read_row(v, vq + t * MLK);
        const float s = xor32_sum(dot16(q, k));
        const float g = xor32_sum(dot16(dy, v));
        const float c = (g - I) * (__builtin_amdgcn_exp2f(s - lse) * w);
#pragma unroll
        for (int i = 0; i < 16; i++) dq[i] = fmaf(c, k[i], dq[i]);
    }
}

// K, V, Q, DY: [nlat][W][LD]; head h of the launch is channels 32 h .. of a point
template <int NW> __global__ __launch_bounds__(64 * NW) void block_dq(const float *__restrict__ K, const float *__restrict__ V, const float *__restrict__ Q, const float *__restrict__ DY,
                                                                    float *__restrict__ DQ, int ngroups, int ntiles)
{
    constexpr int NLAT = NW + 2 * HALO, ROWS = NLAT * NCOL;
    float *Ks = reinterpret_cast<float *>(smem), *Vs = Ks + ROWS * MLK;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    int id = blockIdx.x;
    const int h = id % 8;
    id /= 8;
    const int tile = id % ntiles, grp = id / ntiles;
    if (grp >= ngroups) return;
    const int ho0 = HALO + grp * NW, w0 = 32 * tile;
    // ---- stage once: ROWS rows of 8 sixteen-byte pieces per tensor; all loads in flight before the first LDS write ----
    {
        constexpr int NIT = (ROWS * 8 + 64 * NW - 1) / (64 * NW);
        float4 kx[NIT], vx[NIT];
#pragma unroll
        for (int it = 0; it < NIT; it++) {
            const int p = tid + it * 64 * NW;
            kx[it] = vx[it] = make_float4(0.f, 0.f, 0.f, 0.f);
            if (p < ROWS * 8) {
                const int r = p >> 3, piece = p & 7;
                const int lat = ho0 - HALO + r / NCOL;
                int col = w0 - 4 + r % NCOL;
                col += col < 0 ? W : 0;
                col -= col >= W ? W : 0;
                const size_t g = ((size_t)lat * W + col) * LD + 32 * h + 4 * piece;
                kx[it] = *reinterpret_cast<const float4 *>(K + g);
                vx[it] = *reinterpret_cast<const float4 *>(V + g);
            }
        }
#pragma unroll
        for (int it = 0; it < NIT; it++) {
            const int p = tid + it * 64 * NW;
            if (p < ROWS * 8) {
                const int r = p >> 3, piece = p & 7;
                *reinterpret_cast<float4 *>(Ks + r * MLK + 4 * piece) = kx[it];
                *reinterpret_cast<float4 *>(Vs + r * MLK + 4 * piece) = vx[it];
            }
        }
    }
    const int j = lane & 31, half = lane >> 5;
    float q[16], dy[16], dq[16];
    {
        const size_t g = ((size_t)(ho0 + wave) * W + w0 + j) * LD + 32 * h + 4 * half;
#pragma unroll
        for (int gg = 0; gg < 4; gg++) {
            const float4 x = *reinterpret_cast<const float4 *>(Q + g + 8 * gg), z = *reinterpret_cast<const float4 *>(DY + g + 8 * gg);
            q[4 * gg] = x.x, q[4 * gg + 1] = x.y, q[4 * gg + 2] = x.z, q[4 * gg + 3] = x.w;
            dy[4 * gg] = z.x, dy[4 * gg + 1] = z.y, dy[4 * gg + 2] = z.z, dy[4 * gg + 3] = z.w;
        }
    }
#pragma unroll
    for (int i = 0; i < 16; i++) dq[i] = 0.f;
    const float lse = 0.3f, I = 0.1f, w = 0.5f;
    __syncthreads();
    // ---- seven runs, all from LDS: run of input latitude ho + dl starts at column w0 + j - (len - 1) / 2 = staged column 4 + j - (len - 1) / 2 ----
    const float *kb = Ks + (wave * NCOL + j) * MLK + 4 * half, *vb = Vs + (wave * NCOL + j) * MLK + 4 * half;
    run_steps<1>(dq, q, dy, kb + (0 * NCOL + 4) * MLK, vb + (0 * NCOL + 4) * MLK, lse, I, w);
    run_steps<5>(dq, q, dy, kb + (1 * NCOL + 2) * MLK, vb + (1 * NCOL + 2) * MLK, lse, I, w);
    run_steps<5>(dq, q, dy, kb + (2 * NCOL + 2) * MLK, vb + (2 * NCOL + 2) * MLK, lse, I, w);
    run_steps<7>(dq, q, dy, kb + (3 * NCOL + 1) * MLK, vb + (3 * NCOL + 1) * MLK, lse, I, w);
    run_steps<5>(dq, q, dy, kb + (4 * NCOL + 2) * MLK, vb + (4 * NCOL + 2) * MLK, lse, I, w);
    run_steps<5>(dq, q, dy, kb + (5 * NCOL + 2) * MLK, vb + (5 * NCOL + 2) * MLK, lse, I, w);
    run_steps<1>(dq, q, dy, kb + (6 * NCOL + 4) * MLK, vb + (6 * NCOL + 4) * MLK, lse, I, w);
    {
        const size_t g = ((size_t)(ho0 + wave) * W + w0 + j) * LD + 32 * h + 4 * half;
#pragma unroll
        for (int gg = 0; gg < 4; gg++) *reinterpret_cast<float4 *>(DQ + g + 8 * gg) = make_float4(dq[4 * gg], dq[4 * gg + 1], dq[4 * gg + 2], dq[4 * gg + 3]);
    }
}

template <int NW> void run(const float *K, const float *V, const float *Q, const float *DY, float *DQ, int nlat, int ncu)
{
    const int ngroups = (nlat - 2 * HALO) / NW, ntiles = W / 32;
    const int lds = 2 * (NW + 2 * HALO) * NCOL * MLK * 4;
    CHECK(hipFuncSetAttribute(reinterpret_cast<const void *>(block_dq<NW>), hipFuncAttributeMaxDynamicSharedMemorySize, lds));
    const int nblocks = ngroups * ntiles * 8;
    hipEvent_t e0, e1;
    CHECK(hipEventCreate(&e0));
    CHECK(hipEventCreate(&e1));
    hipLaunchKernelGGL(block_dq<NW>, dim3(nblocks), dim3(64 * NW), lds, 0, K, V, Q, DY, DQ, ngroups, ntiles);
    CHECK(hipDeviceSynchronize());
    CHECK(hipEventRecord(e0));
    for (int r = 0; r < 3; r++) hipLaunchKernelGGL(block_dq<NW>, dim3(nblocks), dim3(64 * NW), lds, 0, K, V, Q, DY, DQ, ngroups, ntiles);
    CHECK(hipEventRecord(e1));
    CHECK(hipEventSynchronize(e1));
    float ms = 0.f;
    CHECK(hipEventElapsedTime(&ms, e0, e1));
    ms /= 3;
    const double tiles = (double)ngroups * NW * ntiles * 8, pairs = tiles * 32 * 29;
    printf("  NW = %d (LDS %6.1f KB per workgroup): %7.3f ms for %d latitudes x 45 tiles x 8 heads = %.3f G pairs -> %.2f us of CU time per tile, %.1f G pairs/s\n", NW, lds / 1024.0, ms,
           ngroups * NW, pairs / 1e9, ms * 1e3 * ncu / tiles, pairs / ms / 1e6);
}

int main()
{
    hipDeviceProp_t prop;
    CHECK(hipGetDeviceProperties(&prop, 0));
    const int nlat = 486; // 480 output latitudes + halo
    const size_t n = (size_t)nlat * W * LD;
    float *K, *V, *Q, *DY, *DQ;
    CHECK(hipMalloc(&K, n * 4));
    CHECK(hipMalloc(&V, n * 4));
    CHECK(hipMalloc(&Q, n * 4));
    CHECK(hipMalloc(&DY, n * 4));
    CHECK(hipMalloc(&DQ, n * 4));
    CHECK(hipMemset(K, 0, n * 4));
    CHECK(hipMemset(V, 0, n * 4));
    CHECK(hipMemset(Q, 0, n * 4));
    CHECK(hipMemset(DY, 0, n * 4));
    printf("device: %s, %d CUs; dq pass of 480 equatorial latitudes of a 1440-longitude grid, 8 heads of 32 channels, 29 neighbors per query\n", prop.gcnArchName, prop.multiProcessorCount);
    run<8>(K, V, Q, DY, DQ, nlat, prop.multiProcessorCount);
    run<6>(K, V, Q, DY, DQ, nlat, prop.multiProcessorCount);
    run<4>(K, V, Q, DY, DQ, nlat, prop.multiProcessorCount);
    run<2>(K, V, Q, DY, DQ, nlat, prop.multiProcessorCount);
    return 0;
}
