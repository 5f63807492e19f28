// Cost of one "row step" of the vector path of the hybrid kernels' dq pass (gfx950): 32 queries (two lanes each, sixteen channels
// per lane) each take ONE neighbor: K and V half-rows from a 40-row LDS tile (row pitch 144 B, 4 + 4 16-byte reads per lane),
// s = q.k and g = dy.v as four multiply-add chains each, one v_permlane32_swap per dot product, p = exp2(s - lse) w,
// dq += p (g - I) k.  48 of the ~66 vector instructions are the multiply-adds of the three products.
//
// Variants, timed at 1 .. 4 single-wavefront workgroups per SIMD (occupancy set by the LDS a workgroup asks for):
//   lds+alu      as the kernel's loop has it: reads of a row, wait, arithmetic
//   alu only     the same arithmetic on operands that stay in registers (no LDS instruction in the loop)
//   lds only     the reads alone (their values are summed so that they stay)
//   pipelined    the reads of the next row are issued before the arithmetic of the current one
//   2 rows       two neighbors per loop turn, their reads issued together (twice the operand registers)
//   dpp          no LDS: K and V rows stay in the registers of the lane that loaded them and neighbor t of a query is taken from
//                the lane t places up its row of sixteen lanes (v_fmac_f32_dpp row_shl:t), eight neighbors per loaded row
// Figures: SIMD time per row step = launch time / row steps per wave / waves per SIMD, in shader clocks at the measured clock.
//
// Build and run:  make -C torch_harmonics_amd/csrc microbench && torch_harmonics_amd/csrc/build/row_step_microbench
#include <hip/hip_runtime.h>
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

constexpr int MLK = 36;   // floats per tile row
constexpr int ROWS = 40;  // rows per tile
constexpr int NB = 8;     // neighbors per chunk: rows j .. j + 7 of the tile for query j

extern __shared__ float4 smem[];

__device__ inline float xor32_sum(float x)
{
    const auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
    return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}
__device__ inline float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

typedef float f4v __attribute__((ext_vector_type(4)));
// The reads are written as instructions so that every variant issues exactly these and waits where it says (the compiler does not
// count them, so each variant places its own s_waitcnt).  addr = LDS byte address of the lane's half of row j.
struct Row {
    f4v x[4];
};
template <int ROW> __device__ inline void read_row(Row &r, unsigned addr)
{
    asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(r.x[0]) : "v"(addr), "n"(ROW * MLK * 4));
    asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(r.x[1]) : "v"(addr), "n"(ROW * MLK * 4 + 32));
    asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(r.x[2]) : "v"(addr), "n"(ROW * MLK * 4 + 64));
    asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(r.x[3]) : "v"(addr), "n"(ROW * MLK * 4 + 96));
}
template <int N> __device__ inline void wait_lds() { asm volatile("s_waitcnt lgkmcnt(%0)" ::"n"(N) : "memory"); }
__device__ inline void settle(Row &r) { asm volatile("" : "+v"(r.x[0]), "+v"(r.x[1]), "+v"(r.x[2]), "+v"(r.x[3])); } // the values are here from now on
__device__ inline void unpack(float (&o)[16], const Row &r)
{
#pragma unroll
    for (int g = 0; g < 4; g++)
#pragma unroll
        for (int e = 0; e < 4; e++) o[4 * g + e] = r.x[g][e];
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
__device__ inline void step(float (&dq)[16], const float (&q)[16], const float (&dy)[16], const float (&k)[16], const float (&v)[16], float lse, float I, float w)
{
    const float s = xor32_sum(dot16(q, k));
    const float g = xor32_sum(dot16(dy, v));
    const float c = (g - I) * (fast_exp2(s - lse) * w);
#pragma unroll
    for (int i = 0; i < 16; i++) dq[i] = fmaf(c, k[i], dq[i]);
}

// The same step with K and V taken from the registers of the lane T places up its row of sixteen (DPP row_shl as an operand
// modifier of the multiply-adds: no LDS, no extra instruction); out-of-row lanes read zeros.
template <int T> __device__ inline void fmac_shl(float &acc, float x, float y)
{
    if constexpr (T == 0)
        acc = fmaf(x, y, acc);
    else
        asm("v_fmac_f32_dpp %0, %1, %2 row_shl:%3 row_mask:0xf bank_mask:0xf bound_ctrl:1" : "+v"(acc) : "v"(x), "v"(y), "n"(T));
}
template <int T> __device__ inline float mul_shl(float x, float y)
{
    float r;
    if constexpr (T == 0)
        r = x * y;
    else
        asm("v_mul_f32_dpp %0, %1, %2 row_shl:%3 row_mask:0xf bank_mask:0xf bound_ctrl:1" : "=v"(r) : "v"(x), "v"(y), "n"(T));
    return r;
}
template <int T> __device__ inline float dot16_shl(const float (&a)[16], const float (&b)[16]) // sum_c a_c (this lane) b_c (lane + T)
{
    float c[4];
#pragma unroll
    for (int g = 0; g < 4; g++) {
        c[g] = mul_shl<T>(b[4 * g], a[4 * g]);
#pragma unroll
        for (int e = 1; e < 4; e++) fmac_shl<T>(c[g], b[4 * g + e], a[4 * g + e]);
    }
    return (c[0] + c[1]) + (c[2] + c[3]);
}
template <int T> __device__ inline void step_shl(float (&dq)[16], const float (&q)[16], const float (&dy)[16], const float (&k)[16], const float (&v)[16], float lse, float I, float w)
{
    const float s = xor32_sum(dot16_shl<T>(q, k));
    const float g = xor32_sum(dot16_shl<T>(dy, v));
    const float c = (g - I) * (fast_exp2(s - lse) * w);
#pragma unroll
    for (int i = 0; i < 16; i++) fmac_shl<T>(dq[i], k[i], c);
}

// fills the tiles; returns the LDS byte addresses of this lane's half of row j of the K and of the V tile (the dynamic
// allocation is the kernel's only LDS, so it starts at address 0)
__device__ inline void fill_tiles(int lane, bool overlap, unsigned &kaddr, unsigned &vaddr)
{
    float *Ks = reinterpret_cast<float *>(smem), *Vs = overlap ? Ks : Ks + ROWS * MLK;
    for (int i = lane; i < ROWS * MLK; i += 64) {
        Ks[i] = 0.001f * (float)((i * 7) % 97) - 0.05f;
        Vs[i] = 0.002f * (float)((i * 5) % 89) - 0.09f;
    }
    __syncthreads();
    const int j = lane & 31, half = lane >> 5;
    kaddr = (unsigned)(j * MLK + 4 * half) * 4u;
    vaddr = kaddr + (overlap ? 0u : (unsigned)(ROWS * MLK * 4));
}

template <int MODE, int N> struct Turn {
    static __device__ inline void run(float (&dq)[16], const float (&q)[16], const float (&dy)[16], Row &kr, Row &vr, Row &k2, Row &v2, unsigned ka, unsigned va, float lse, float I, float w)
    {
        float k[16], v[16];
        if constexpr (MODE == 0) { // reads of a row, wait, arithmetic
            read_row<N>(kr, ka);
            read_row<N>(vr, va);
            wait_lds<0>();
            settle(kr), settle(vr);
            unpack(k, kr), unpack(v, vr);
            step(dq, q, dy, k, v, lse, I, w);
        } else if constexpr (MODE == 1) { // operands stay in registers
            settle(kr), settle(vr);
            unpack(k, kr), unpack(v, vr);
            step(dq, q, dy, k, v, lse, I, w);
        } else if constexpr (MODE == 2) { // the reads alone
            read_row<N>(kr, ka);
            read_row<N>(vr, va);
            wait_lds<0>();
            settle(kr), settle(vr);
        } else if constexpr (MODE == 3) { // the next row's reads fly during this row's arithmetic
            unpack(k, kr), unpack(v, vr);
            read_row<(N + 1) % NB>(k2, ka);
            read_row<(N + 1) % NB>(v2, va);
            __builtin_amdgcn_sched_barrier(0);
            step(dq, q, dy, k, v, lse, I, w);
            __builtin_amdgcn_sched_barrier(0);
            wait_lds<0>();
            settle(k2), settle(v2);
            kr = k2, vr = v2;
        } else if constexpr (MODE == 5) { // operands stay in registers and are taken from the lane N places up the row
            if constexpr (N == 0) settle(kr), settle(vr);
            unpack(k, kr), unpack(v, vr);
            step_shl<N>(dq, q, dy, k, v, lse, I, w);
        } else if constexpr (N % 2 == 0) { // two rows per turn, their reads issued together
            read_row<N>(kr, ka);
            read_row<N>(vr, va);
            read_row<N + 1>(k2, ka);
            read_row<N + 1>(v2, va);
            wait_lds<8>();
            settle(kr), settle(vr);
            unpack(k, kr), unpack(v, vr);
            step(dq, q, dy, k, v, lse, I, w);
            wait_lds<0>();
            settle(k2), settle(v2);
            unpack(k, k2), unpack(v, v2);
            step(dq, q, dy, k, v, lse, I, w);
        }
        if constexpr (N + 1 < NB) Turn<MODE, N + 1>::run(dq, q, dy, kr, vr, k2, v2, ka, va, lse, I, w);
    }
};

template <int MODE> __global__ __launch_bounds__(64) void row_steps(float *out, int turns, int overlap)
{
    const int lane = threadIdx.x;
    unsigned ka, va;
    fill_tiles(lane, overlap != 0, ka, va);
    float q[16], dy[16], dq[16];
#pragma unroll
    for (int i = 0; i < 16; i++) q[i] = 0.01f * (float)(lane + i), dy[i] = 0.02f * (float)(lane - i), dq[i] = 0.f;
    const float lse = 0.3f, I = 0.1f, w = 0.5f;
    Row kr, vr, k2, v2;
    read_row<0>(kr, ka);
    read_row<0>(vr, va);
    wait_lds<0>();
    settle(kr), settle(vr);
    k2 = kr, v2 = vr;
    for (int it = 0; it < turns; it++) {
        Turn<MODE, 0>::run(dq, q, dy, kr, vr, k2, v2, ka, va, lse, I, w);
        asm volatile("" : "+v"(ka), "+v"(va));
    }
    float s = 0.f;
#pragma unroll
    for (int i = 0; i < 16; i++) s += dq[i];
    if constexpr (MODE == 2) s += kr.x[0][0] + vr.x[3][3];
    out[(size_t)blockIdx.x * 64 + lane] = s;
}

__global__ void clock_probe(long long *c)
{
    const long long t0 = clock64(), r0 = wall_clock64();
    float x = (float)threadIdx.x;
    for (int i = 0; i < 200000; i++) x = fmaf(x, 1.0001f, 0.5f);
    const long long t1 = clock64(), r1 = wall_clock64();
    if (threadIdx.x == 0) c[0] = t1 - t0, c[1] = r1 - r0, c[2] = (long long)x;
}

template <int MODE> double run(int waves_per_simd, int ncu, float *out, int turns)
{
    const int wg_per_cu = 4 * waves_per_simd;
    int lds = (160 * 1024 / wg_per_cu) & ~255; // so many workgroups fit a CU and no more
    const int need = 2 * ROWS * MLK * 4;
    const int overlap = lds < need;
    if (lds > 64 * 1024) lds = 64 * 1024;
    CHECK(hipFuncSetAttribute(reinterpret_cast<const void *>(row_steps<MODE>), hipFuncAttributeMaxDynamicSharedMemorySize, lds));
    const int nblocks = ncu * wg_per_cu;
    hipEvent_t e0, e1;
    CHECK(hipEventCreate(&e0));
    CHECK(hipEventCreate(&e1));
    hipLaunchKernelGGL(row_steps<MODE>, dim3(nblocks), dim3(64), lds, 0, out, turns, overlap);
    CHECK(hipDeviceSynchronize());
    CHECK(hipEventRecord(e0));
    hipLaunchKernelGGL(row_steps<MODE>, dim3(nblocks), dim3(64), lds, 0, out, turns, overlap);
    CHECK(hipEventRecord(e1));
    CHECK(hipEventSynchronize(e1));
    float ms = 0.f;
    CHECK(hipEventElapsedTime(&ms, e0, e1));
    return (double)ms * 1e6 / ((double)turns * NB) / waves_per_simd; // ns of SIMD time per row step
}

int main()
{
    hipDeviceProp_t prop;
    CHECK(hipGetDeviceProperties(&prop, 0));
    const int ncu = prop.multiProcessorCount;
    printf("device: %s, %d CUs\n", prop.gcnArchName, ncu);
    float *out;
    CHECK(hipMalloc(&out, (size_t)ncu * 32 * 64 * sizeof(float)));
    long long *c;
    CHECK(hipMalloc(&c, 3 * sizeof(long long)));
    hipLaunchKernelGGL(clock_probe, dim3(1), dim3(64), 0, 0, c);
    long long hc[3];
    CHECK(hipMemcpy(hc, c, sizeof(hc), hipMemcpyDeviceToHost));
    const double ghz = (double)hc[0] / ((double)hc[1] * 10.0);
    printf("shader clock in a short kernel: %.2f GHz (figures below in clocks at this rate)\n", ghz);
    const int turns = 4000;
    printf("\nSIMD clocks per row step (32 queries x 1 neighbor, dq pass), single-wavefront workgroups\n");
    printf("  %-10s %-10s %-10s %-10s %-10s %-10s %-10s\n", "waves/SIMD", "lds+alu", "alu only", "lds only", "pipelined", "2 rows", "dpp");
    for (int w = 1; w <= 4; w++) {
        const double a = run<0>(w, ncu, out, turns), b = run<1>(w, ncu, out, turns), l = run<2>(w, ncu, out, turns), p = run<3>(w, ncu, out, turns),
                     d = run<4>(w, ncu, out, turns), x = run<5>(w, ncu, out, turns);
        printf("  %-10d %-10.0f %-10.0f %-10.0f %-10.0f %-10.0f %-10.0f\n", w, a * ghz, b * ghz, l * ghz, p * ghz, d * ghz, x * ghz);
    }
    CHECK(hipFree(out));
    CHECK(hipFree(c));
    return 0;
}
