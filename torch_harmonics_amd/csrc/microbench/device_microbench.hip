// Device microbenchmarks behind the design decisions of the attention kernels (gfx950).  Stand-alone: no library code, no torch.
//
//   part 1  Do matrix-core and vector instructions execute at the same time on one SIMD?
//           Per iteration a wave issues NM matrix instructions (four independent accumulators) and/or 256 vector FMAs (sixteen
//           independent chains), as separate phases of one stream, interleaved in one stream, or split over different waves of
//           the same SIMD (waves w and w + 4 of a 512-thread workgroup share a SIMD; the kernel records HW_ID to show it).
//   part 2  LDS and vector-L1 bytes per clock per CU for the access shapes the kernels use.
//
// Build and run:  make -C torch_harmonics_amd/csrc microbench && torch_harmonics_amd/csrc/build/device_microbench
#include <hip/hip_runtime.h>
#include <cstdio>
#include <cstdlib>
#include <vector>

#define CHECK(x)                                                                                   \
    do {                                                                                           \
        hipError_t e_ = (x);                                                                       \
        if (e_ != hipSuccess) {                                                                    \
            fprintf(stderr, "%s:%d: %s\n", __FILE__, __LINE__, hipGetErrorString(e_));             \
            exit(1);                                                                               \
        }                                                                                          \
    } while (0)

typedef float f16v __attribute__((ext_vector_type(16)));
typedef float f4v __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef unsigned u4v __attribute__((ext_vector_type(4)));
typedef short s16x4_t __attribute__((ext_vector_type(4)));

constexpr int NV = 256; // vector FMAs per iteration

// KIND 0: v_mfma_f32_32x32x2_f32, 1: v_mfma_f32_32x32x16_bf16, 2: v_mfma_f32_16x16x32_bf16, 3: v_mfma_f32_16x16x4_f32
template <int KIND> struct Mat;
template <> struct Mat<0> {
    typedef f16v acc_t;
    static constexpr const char *name = "v_mfma_f32_32x32x2_f32";
    static constexpr int NM = 16;
    __device__ static inline acc_t op(float a, float b, bf16x8, bf16x8, acc_t c) { return __builtin_amdgcn_mfma_f32_32x32x2f32(a, b, c, 0, 0, 0); }
};
template <> struct Mat<1> {
    typedef f16v acc_t;
    static constexpr const char *name = "v_mfma_f32_32x32x16_bf16";
    static constexpr int NM = 16;
    __device__ static inline acc_t op(float, float, bf16x8 a, bf16x8 b, acc_t c) { return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0); }
};
template <> struct Mat<2> {
    typedef f4v acc_t;
    static constexpr const char *name = "v_mfma_f32_16x16x32_bf16";
    static constexpr int NM = 32;
    __device__ static inline acc_t op(float, float, bf16x8 a, bf16x8 b, acc_t c) { return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0); }
};
template <> struct Mat<3> {
    typedef f4v acc_t;
    static constexpr const char *name = "v_mfma_f32_16x16x4_f32";
    static constexpr int NM = 32;
    __device__ static inline acc_t op(float a, float b, bf16x8, bf16x8, acc_t c) { return __builtin_amdgcn_mfma_f32_16x16x4f32(a, b, c, 0, 0, 0); }
};

__device__ inline unsigned hw_id()
{
    unsigned v;
    asm volatile("s_getreg_b32 %0, hwreg(HW_REG_HW_ID)" : "=s"(v));
    return v;
}

// MODE 0: matrix only, 1: vector only, 2: phases in one wave, 3: interleaved in one wave, 4: matrix waves and vector waves side by side
template <int KIND, int MODE> __global__ __launch_bounds__(512) void coexec_kernel(float *out, unsigned *ids, long long *clk, int iters)
{
    typedef Mat<KIND> M;
    constexpr int NM = M::NM;
    typename M::acc_t acc[4];
    for (int c = 0; c < 4; c++)
        for (unsigned v = 0; v < sizeof(acc[c]) / 4; v++) acc[c][v] = 0.f;
    const float a = threadIdx.x * 1e-3f, b = 1.0001f;
    bf16x8 av, bv;
    for (int i = 0; i < 8; i++) {
        av[i] = (__bf16)(a + i);
        bv[i] = (__bf16)(b - i);
    }
    float x[16];
    for (int i = 0; i < 16; i++) x[i] = a + i;
    const int wave = threadIdx.x >> 6;
    const bool do_m = MODE == 0 || MODE == 2 || (MODE == 4 && wave < 4);
    const bool do_v = MODE == 1 || MODE == 2 || (MODE == 4 && wave >= 4);
    const long long t0 = clock64(), r0 = wall_clock64();
    for (int it = 0; it < iters; it++) {
        if (MODE == 3) {
#pragma unroll
            for (int m = 0; m < NM; m++) {
                acc[m & 3] = M::op(a, b, av, bv, acc[m & 3]);
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int n = 0; n < NV / NM; n++) x[(m * (NV / NM) + n) & 15] = fmaf(x[(m * (NV / NM) + n) & 15], b, a);
                __builtin_amdgcn_sched_barrier(0);
            }
        } else {
            if (do_m) {
#pragma unroll
                for (int m = 0; m < NM; m++) acc[m & 3] = M::op(a, b, av, bv, acc[m & 3]);
            }
            __builtin_amdgcn_sched_barrier(0);
            if (do_v) {
#pragma unroll
                for (int n = 0; n < NV; n++) x[n & 15] = fmaf(x[n & 15], b, a);
            }
            __builtin_amdgcn_sched_barrier(0);
        }
    }
    const long long t1 = clock64(), r1 = wall_clock64();
    float s = 0.f;
    for (int c = 0; c < 4; c++)
        for (unsigned v = 0; v < sizeof(acc[c]) / 4; v++) s += acc[c][v];
    for (int i = 0; i < 16; i++) s += x[i];
    out[(size_t)blockIdx.x * blockDim.x + threadIdx.x] = s;
    if ((threadIdx.x & 63) == 0) ids[blockIdx.x * (blockDim.x >> 6) + wave] = (hw_id() << 1) | (do_m ? 1u : 0u);
    if (blockIdx.x == 0 && threadIdx.x == 0) {
        clk[0] = t1 - t0;
        clk[1] = r1 - r0;
    }
}

struct Res {
    double us_per_iter; // wall time of the launch / iterations
    double shader_clk_per_iter, ghz;
};

template <int KIND, int MODE> Res run_coexec(float *out, unsigned *ids, long long *clk, int waves_per_simd, int iters, bool check_ids)
{
    // 256 CUs x 4 SIMDs; 512 threads = 8 waves = 2 per SIMD of one CU (1 wave per SIMD: 256 threads)
    const int threads = waves_per_simd == 1 ? 256 : 512;
    const int blocks = 256 * 4 * waves_per_simd * 64 / threads;
    hipEvent_t e0, e1;
    CHECK(hipEventCreate(&e0));
    CHECK(hipEventCreate(&e1));
    hipLaunchKernelGGL((coexec_kernel<KIND, MODE>), dim3(blocks), dim3(threads), 0, 0, out, ids, clk, 10);
    CHECK(hipEventRecord(e0));
    hipLaunchKernelGGL((coexec_kernel<KIND, MODE>), dim3(blocks), dim3(threads), 0, 0, out, ids, clk, iters);
    CHECK(hipEventRecord(e1));
    CHECK(hipEventSynchronize(e1));
    float ms = 0;
    CHECK(hipEventElapsedTime(&ms, e0, e1));
    long long c[2];
    CHECK(hipMemcpy(c, clk, sizeof(c), hipMemcpyDeviceToHost));
    Res r;
    r.us_per_iter = ms * 1e3 / iters;
    r.shader_clk_per_iter = (double)c[0] / iters;
    r.ghz = c[1] > 0 ? (double)c[0] / ((double)c[1] * 10.0) : 0.0; // wall_clock64 ticks at 100 MHz
    if (check_ids) {
        // every SIMD that got waves must have got as many matrix waves as vector waves
        const int nw = blocks * (threads / 64);
        std::vector<unsigned> h(nw);
        CHECK(hipMemcpy(h.data(), ids, nw * 4, hipMemcpyDeviceToHost));
        // a workgroup's waves w and w + 4 must sit on the same SIMD (HW_ID bits 5:4) of the same CU
        int bad = 0;
        for (int g = 0; g < blocks; g++)
            for (int w = 0; w < 4; w++) {
                const unsigned i0 = h[g * 8 + w] >> 1, i1 = h[g * 8 + w + 4] >> 1;
                const unsigned simd0 = (i0 >> 4) & 3, simd1 = (i1 >> 4) & 3, cu0 = (i0 >> 8) & 0xff, cu1 = (i1 >> 8) & 0xff;
                if (simd0 != simd1 || cu0 != cu1) bad++;
            }
        if (bad) printf("    (note: %d of %d matrix/vector wave pairs did NOT share a SIMD)\n", bad, blocks * 4);
    }
    CHECK(hipEventDestroy(e0));
    CHECK(hipEventDestroy(e1));
    return r;
}

template <int KIND> void coexec_table(float *out, unsigned *ids, long long *clk)
{
    const int iters = 2000;
    printf("\n%s: %d per iteration (4 independent accumulators) against %d v_fma_f32 (16 independent chains)\n", Mat<KIND>::name, Mat<KIND>::NM, NV);
    printf("  SIMD time per wave-iteration = launch time / iterations / waves per SIMD, in ns and (in parentheses) in shader clocks at the measured clock.\n");
    printf("  'side by side': half of the waves of each SIMD issue only the matrix work, the other half only the vector work; SIMD time per (matrix + vector) pair of iterations.\n");
    printf("  %-10s %-16s %-16s %-16s %-16s %-16s %s\n", "waves/SIMD", "matrix only", "vector only", "phases", "interleaved", "side by side", "clock GHz");
    for (int w : {1, 2, 4, 8}) {
        const Res m = run_coexec<KIND, 0>(out, ids, clk, w, iters, false);
        const Res v = run_coexec<KIND, 1>(out, ids, clk, w, iters, false);
        const Res p = run_coexec<KIND, 2>(out, ids, clk, w, iters, false);
        const Res i = run_coexec<KIND, 3>(out, ids, clk, w, iters, false);
        const double ghz = p.ghz;
        auto cell = [&](double us_per_iter, int div) {
            const double ns = us_per_iter * 1e3 / div;
            printf("%7.1f (%5.0f)  ", ns, ns * ghz);
        };
        printf("  %-10d ", w);
        cell(m.us_per_iter, w);
        cell(v.us_per_iter, w);
        cell(p.us_per_iter, w);
        cell(i.us_per_iter, w);
        if (w >= 2) {
            const Res s = run_coexec<KIND, 4>(out, ids, clk, w, iters, true);
            cell(s.us_per_iter, w / 2);
        } else
            printf("%-16s ", "-");
        printf("%.2f\n", ghz);
    }
}

// ---- part 2: LDS and L1 ----
constexpr int PITCH = 160;
// MODE 0: 8 ds_read_b128 (row pieces at pitch 160 B); 1: 8 ds_write_b128; 2: 8 ds_read_b64_tr_b16; 3: 8 ds_read_b64; 4: 16 ds_write_b64; 5: 32 ds_write_b32;
//      6: 8 global_load_lds of 16 B per lane; 7: 8 global loads of 16 B per lane into registers (L1-resident lines)
template <int MODE> __global__ __launch_bounds__(64) void lds_kernel(float *out, const char *src, int iters)
{
    __shared__ __attribute__((aligned(16))) char T[2 * 32 * PITCH];
    const int lane = threadIdx.x, c = lane & 15, qd = lane >> 4;
    for (int i = lane; i < 2 * 32 * PITCH / 4; i += 64) reinterpret_cast<unsigned *>(T)[i] = i;
    __syncthreads();
    u4v acc = {(unsigned)lane, 1, 2, 3};
    const char *rowp = T + c * PITCH + 16 * qd;
    char *wp = T + (lane / 8) * PITCH + 16 * (lane % 8);
    typedef s16x4_t __attribute__((address_space(3))) * lds_ptr;
    const char *tp = T + (4 * qd + (c >> 2)) * PITCH + 8 * (c & 3);
    const char *g = src + (size_t)(blockIdx.x % 64) * 8192 + lane * 16;
    for (int it = 0; it < iters; it++) {
        if (MODE == 0) {
#pragma unroll
            for (int j = 0; j < 8; j++) {
                u4v r = *reinterpret_cast<const u4v *>(rowp + (j & 1) * 16 * PITCH + (j >> 1) * 64 + ((j >> 2) * 32 * PITCH));
                asm volatile("" : "+v"(r));
                acc ^= r;
            }
        }
        if (MODE == 1) {
#pragma unroll
            for (int j = 0; j < 8; j++) {
                u4v w = acc;
                w.x += j;
                *reinterpret_cast<u4v *>(wp + (j & 3) * 8 * PITCH + (j >> 2) * 32 * PITCH) = w;
            }
        }
        if (MODE == 2) {
#pragma unroll
            for (int j = 0; j < 8; j++) {
                s16x4_t r = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_ptr)(tp + (j & 1) * 16 * PITCH + (j >> 1) * 32));
                asm volatile("" : "+v"(r));
                acc.x ^= (unsigned)r[0];
            }
        }
        if (MODE == 3) {
#pragma unroll
            for (int j = 0; j < 8; j++) {
                uint2 r = *reinterpret_cast<const uint2 *>(tp + (j & 1) * 16 * PITCH + (j >> 1) * 32);
                asm volatile("" : "+v"(r.x), "+v"(r.y));
                acc.x ^= r.x;
            }
        }
        if (MODE == 4) {
            char *w8 = T + (lane / 16) * PITCH + 8 * (lane % 16);
#pragma unroll
            for (int j = 0; j < 16; j++) *reinterpret_cast<uint2 *>(w8 + j * 4 * PITCH) = make_uint2(acc.x + j, acc.y);
        }
        if (MODE == 5) {
            char *w4 = T + (lane / 32) * PITCH + 4 * (lane % 32);
#pragma unroll
            for (int j = 0; j < 32; j++) *reinterpret_cast<unsigned *>(w4 + j * 2 * PITCH) = acc.x + j;
        }
        if (MODE == 6) {
#pragma unroll
            for (int j = 0; j < 8; j++)
                __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void *)(g + j * 1024), (__attribute__((address_space(3))) void *)(T + j * 1024), 16, 0, 0);
            asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        }
        if (MODE == 7) {
#pragma unroll
            for (int j = 0; j < 8; j++) {
                u4v r = *reinterpret_cast<const u4v *>(g + j * 1024);
                asm volatile("" : "+v"(r));
                acc ^= r;
            }
        }
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    }
    __syncthreads();
    out[(size_t)blockIdx.x * 64 + lane] = acc.x + acc.y + acc.z + acc.w + reinterpret_cast<unsigned *>(T)[lane];
}

template <int MODE> double run_lds(float *out, const char *src, int w, int iters)
{
    hipEvent_t e0, e1;
    CHECK(hipEventCreate(&e0));
    CHECK(hipEventCreate(&e1));
    hipLaunchKernelGGL((lds_kernel<MODE>), dim3(256 * 4 * w), dim3(64), 0, 0, out, src, 10);
    CHECK(hipEventRecord(e0));
    hipLaunchKernelGGL((lds_kernel<MODE>), dim3(256 * 4 * w), dim3(64), 0, 0, out, src, iters);
    CHECK(hipEventRecord(e1));
    CHECK(hipEventSynchronize(e1));
    float ms = 0;
    CHECK(hipEventElapsedTime(&ms, e0, e1));
    CHECK(hipEventDestroy(e0));
    CHECK(hipEventDestroy(e1));
    return ms * 1e-3 / iters / (4 * w); // seconds of CU time per wave-iteration
}

int main()
{
    float *out;
    unsigned *ids;
    long long *clk;
    char *src;
    CHECK(hipMalloc(&out, (size_t)256 * 4 * 8 * 64 * 4));
    CHECK(hipMalloc(&ids, (size_t)256 * 4 * 8 * 4));
    CHECK(hipMalloc(&clk, 16));
    CHECK(hipMalloc(&src, 64 * 8192 + 65536));
    CHECK(hipMemset(src, 1, 64 * 8192 + 65536));
    hipDeviceProp_t prop;
    CHECK(hipGetDeviceProperties(&prop, 0));
    printf("device: %s, %d CUs, clock %.0f MHz\n", prop.gcnArchName, prop.multiProcessorCount, prop.clockRate / 1e3);

    printf("\n== part 1: matrix-core and vector instructions on one SIMD ==\n");
    coexec_table<0>(out, ids, clk);
    coexec_table<3>(out, ids, clk);
    coexec_table<1>(out, ids, clk);
    coexec_table<2>(out, ids, clk);

    printf("\n== part 2: LDS and vector-L1 throughput per CU (one wave per workgroup; bytes per CU clock at the clock part 1 reports) ==\n");
    const double kb[8] = {8, 8, 4, 4, 8, 8, 8, 8};
    const char *names[8] = {"ds_read_b128", "ds_write_b128", "ds_read_b64_tr_b16", "ds_read_b64", "ds_write_b64", "ds_write_b32", "global_load_lds 16B", "global_load 16B (L1 hit)"};
    for (int w : {1, 2, 4}) {
        const int iters = 4000;
        const double t[8] = {run_lds<0>(out, src, w, iters), run_lds<1>(out, src, w, iters), run_lds<2>(out, src, w, iters), run_lds<3>(out, src, w, iters),
                             run_lds<4>(out, src, w, iters), run_lds<5>(out, src, w, iters), run_lds<6>(out, src, w, iters), run_lds<7>(out, src, w, iters)};
        printf("  waves/SIMD %d:\n", w);
        for (int i = 0; i < 8; i++) printf("    %-26s %7.1f ns per %g KB  = %6.1f B/ns per CU\n", names[i], t[i] * 1e9, kb[i], kb[i] * 1024 / (t[i] * 1e9));
    }
    return 0;
}
