// Matrix-core tiles of the hybrid fp32 kernels on bf16 matrix instructions (head dim 32): the dk/dv pass.  Included by
// s2attn_kernels.hip inside namespace s2, after Tile40 and the pair path.
//
// v_mfma_f32_32x32x16_bf16 does sixteen times the work of v_mfma_f32_32x32x2_f32 per clock (a 32x32x32 product: 60 clocks
// against 1,000).  fp32 operands are split into three bf16 terms, x = h + m + l, every term the round-to-nearest bf16 of what
// the earlier ones left (|x - h - m - l| <= 2^-25 |x|), and a product is the sum of the six term products with i + j <= 4
// (relative error 2^-23 per term of the sum; two terms per value were measured and miss rtol 1e-5 where one neighbor
// dominates a sum).  Low-order products are issued first, so the accumulator meets the large terms last.
//
// The split is vector work (11 instructions per two values) and vector and matrix instructions do not overlap on a SIMD, so
// the exchange pays where a tile step has many products per split value: the dk/dv pass (four products, two staged tensors,
// two coefficient sets: 64 fp32 matrix instructions become 48 bf16 ones of half the length each) gains 15 % on the long-run
// latitudes; the forward (two products) gains nothing and the dq pass loses its third resident wavefront per SIMD to the
// extra registers, so both stay on fp32 matrix instructions.
//
// Staged rows are split when they are committed to LDS.  A row of a split tile is [term][32 channels] bf16 (64 B per term)
// with channel c = 8 g + 4 hh + e stored at position 16 hh + 4 g + e: the sixteen channels that lane (row, hh) feeds to the two
// matrix instructions of a product are 32 contiguous bytes, and they are the channels 8 g + 4 half + e that a lane of the
// other operand holds in registers anyway.  Row pitch 208 B: 16-byte row reads, transposing 8-byte reads and the 8-byte
// commit writes are all free of bank conflicts.  The transposed operand (channels x positions) comes from
// ds_read_b64_tr_b16 on the same rows.

typedef unsigned u4v __attribute__((ext_vector_type(4)));
typedef unsigned u2v __attribute__((ext_vector_type(2)));
typedef float f2v __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef short s16x4_t __attribute__((ext_vector_type(4)));

constexpr int SPP = 208;                   // bytes per row of a split tile
constexpr int SPLIT_TILE_BYTES = MT * SPP; // 32 rows

__device__ inline unsigned pk_bf16(float a, float b)
{
    const f2v x = {a, b};
    return __builtin_bit_cast(unsigned, __builtin_convertvector(x, bf16x2_t)); // v_cvt_pk_bf16_f32: a in the low half
}
__device__ inline float pk_lo(unsigned p) { return __uint_as_float(p << 16); }
__device__ inline float pk_hi(unsigned p) { return __uint_as_float(p & 0xffff0000u); }
__device__ inline void split3(float a, float b, unsigned &h, unsigned &m, unsigned &l)
{
    h = pk_bf16(a, b);
    const float ra = a - pk_lo(h), rb = b - pk_hi(h);
    m = pk_bf16(ra, rb);
    l = pk_bf16(ra - pk_lo(m), rb - pk_hi(m));
}
__device__ inline bf16x8_t as_bf16(u4v x) { return __builtin_bit_cast(bf16x8_t, x); }
__device__ inline f16v mma(u4v a, u4v b, f16v c) { return __builtin_amdgcn_mfma_f32_32x32x16_bf16(as_bf16(a), as_bf16(b), c, 0, 0, 0); }

// Sixteen values of a lane (registers 8 n + e are the k slots of matrix instruction n) as packed bf16 terms.
struct Terms3 {
    u4v h[2], m[2], l[2];
};
template <typename A> __device__ inline void split_regs(Terms3 &o, const A &x)
{
#pragma unroll
    for (int n = 0; n < 2; n++)
#pragma unroll
        for (int i = 0; i < 4; i++) {
            unsigned h_, m_, l_;
            split3(x[8 * n + 2 * i], x[8 * n + 2 * i + 1], h_, m_, l_);
            o.h[n][i] = h_, o.m[n][i] = m_, o.l[n][i] = l_;
        }
}

// Commit of a tile prefetched with Tile40::fetch_split (rows 4 (lane / 8) + it, channels 4 (lane & 7) .. + 3 per lane) as a split
// tile of 32 rows.
template <typename T> __device__ inline void commit_split(const Tile40<T> &t, char *dst, int lane)
{
    const int r0 = lane >> 3, c8 = lane & 7;
    char *p = dst + 4 * r0 * SPP + 32 * (c8 & 1) + 8 * (c8 >> 1);
#pragma unroll
    for (int it = 0; it < 4; it++) {
        const float4 x = widen4(t.raw[it], (const T *)nullptr);
        unsigned h0, m0, l0, h1, m1, l1;
        split3(x.x, x.y, h0, m0, l0);
        split3(x.z, x.w, h1, m1, l1);
        *reinterpret_cast<u2v *>(p + it * SPP) = u2v{h0, h1};
        *reinterpret_cast<u2v *>(p + it * SPP + 64) = u2v{m0, m1};
        *reinterpret_cast<u2v *>(p + it * SPP + 128) = u2v{l0, l1};
    }
}

// acc += X W^T: X = staged rows (this lane's row at rowp = tile + row * SPP + 32 * hh), W = the other operand's terms in registers.
__device__ inline f16v rows_times_regs(const char *rowp, const Terms3 &w, f16v acc)
{
    u4v xh[2], xm[2], xl[2];
#pragma unroll
    for (int n = 0; n < 2; n++) {
        xh[n] = *reinterpret_cast<const u4v *>(rowp + 16 * n);
        xm[n] = *reinterpret_cast<const u4v *>(rowp + 64 + 16 * n);
        xl[n] = *reinterpret_cast<const u4v *>(rowp + 128 + 16 * n);
    }
#pragma unroll
    for (int n = 0; n < 2; n++) {
        acc = mma(xl[n], w.h[n], acc);
        acc = mma(xh[n], w.l[n], acc);
        acc = mma(xm[n], w.m[n], acc);
    }
#pragma unroll
    for (int n = 0; n < 2; n++) {
        acc = mma(xm[n], w.h[n], acc);
        acc = mma(xh[n], w.m[n], acc);
    }
#pragma unroll
    for (int n = 0; n < 2; n++) acc = mma(xh[n], w.h[n], acc);
    return acc;
}

// Per-lane byte offset of the transposing reads: source lane s of 16-lane group G addresses row 4 (G / 2) + (s % 16) / 4 and the
// four channels 4 (4 (G % 2) + s % 4) .. + 3; a lane then receives channel lane % 32 of rows 4 (lane / 32) + 0..3 (+ the row
// offset of the read), which are the k slots kappa(v, lane / 32) of its matrix instruction.
__device__ inline int tr_lane_offset(int lane)
{
    const int G = lane >> 4, es = (lane & 15) >> 2, cbs = 4 * (G & 1) + (lane & 3);
    return (4 * (G >> 1) + es) * SPP + 32 * (cbs & 1) + 8 * (cbs >> 1);
}
// term `term` of the transposed operand of matrix instruction n: [channel = lane % 32][k slots of lane / 32]
__device__ inline u4v read_tr(const char *tile, int troff, int n, int term)
{
    typedef s16x4_t __attribute__((address_space(3))) * lds_ptr;
    const char *p = tile + troff + 16 * n * SPP + 64 * term;
    const u2v a = __builtin_bit_cast(u2v, __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_ptr)(p)));
    const u2v b = __builtin_bit_cast(u2v, __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_ptr)(p + 8 * SPP)));
    return u4v{a[0], a[1], b[0], b[1]};
}
// acc += X^T W, X staged, W in registers.
__device__ inline f16v cols_times_regs(const char *tile, int troff, const Terms3 &w, f16v acc)
{
#pragma unroll
    for (int n = 0; n < 2; n++) {
        const u4v xh = read_tr(tile, troff, n, 0), xm = read_tr(tile, troff, n, 1), xl = read_tr(tile, troff, n, 2);
        acc = mma(xl, w.h[n], acc);
        acc = mma(xh, w.l[n], acc);
        acc = mma(xm, w.m[n], acc);
        acc = mma(xm, w.h[n], acc);
        acc = mma(xh, w.m[n], acc);
        acc = mma(xh, w.h[n], acc);
    }
    return acc;
}

// The lane's own operand (k or v: sixteen channels 8 g + 4 half + e) kept in ONE set of registers in the form the current run
// needs: sixteen floats for vector chunks, or three bf16 terms (24 registers) for matrix-core steps.  A latitude changes form at
// most twice, and the change reloads the row (both forms alive at once would cost registers the kernel does not have).
struct OwnRegs {
    unsigned r[24];
    template <typename T> __device__ inline void load(const T *row, float scale, bool split)
    {
        float f[16];
        load_half_row(f, row, scale);
        if (split) {
            Terms3 t;
            split_regs(t, f);
#pragma unroll
            for (int i = 0; i < 8; i++) r[i] = t.h[i / 4][i % 4], r[8 + i] = t.m[i / 4][i % 4], r[16 + i] = t.l[i / 4][i % 4];
        } else {
#pragma unroll
            for (int i = 0; i < 16; i++) r[i] = __float_as_uint(f[i]);
#pragma unroll
            for (int i = 16; i < 24; i++) r[i] = 0u;
        }
    }
    __device__ inline void floats(float (&f)[16]) const
    {
#pragma unroll
        for (int i = 0; i < 16; i++) f[i] = __uint_as_float(r[i]);
    }
    __device__ inline Terms3 terms() const
    {
        Terms3 t;
#pragma unroll
        for (int i = 0; i < 8; i++) t.h[i / 4][i % 4] = r[i], t.m[i / 4][i % 4] = r[8 + i], t.l[i / 4][i % 4] = r[16 + i];
        return t;
    }
};
