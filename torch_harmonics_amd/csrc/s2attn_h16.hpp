// Matrix-core kernels for 16-bit storage (bf16, fp16): forward, dq and dk/dv with v_mfma_f32_16x16x32_{bf16,f16}.
// Included by s2attn_kernels.hip inside namespace s2 (uses its Args, Run and storage types).
//
// Shape domain: ck == cv = dr, a multiple of 8 with dr <= D (the tile is D channels wide, D a multiple of 32; channels
// from dr on are staged as zeros and never stored), at least 32 columns per virtual latitude, 16-byte aligned rows.
//
// One wavefront owns HQ = 16 consecutive longitudes of one latitude for one (batch, head) and walks every run of that
// latitude in steps of HK = 32 band positions (len + 15 positions per run; position u belongs to the neighborhood of
// column c iff 0 <= u - c < len).  Lane l = (c = l % 16, qd = l / 16).  Facts about the instruction used below:
//   A operand: lane supplies A[i = c][k = 8 qd + e], e < 8;   B operand: lane supplies B[k = 8 qd + e][j = c];
//   D: register v of the lane holds D[i = 4 qd + v][j = c].
// Scores are produced transposed (S^T[position][column]) so that a lane holds 8 positions of ITS column per step:
// (block kb < 2, v < 4) <-> position 16 kb + 4 qd + v.  Packed to 16 bit in the order e = 4 kb + v these eight values
// are, unchanged, the B operand of the second product, whose k slot (qd, e) therefore means position 16 kb + 4 qd + v.
// The matching A operand (channels x positions, i.e. a transposed read of a [position][channel] tile) comes from
// ds_read_b64_tr_b16: inside a group of 16 lanes, lane r addresses the 8 bytes of row r / 4, column group r % 4 and
// receives column r of the four rows.
//
// The quadrature weight enters the exponent (score * log2 e + log2 w) so that probabilities handed to the matrix
// cores lie in [0, 1] whatever the weight's magnitude (polar weights are below the fp16 normal range).

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef _Float16 f16x8_t __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
typedef _Float16 f16x2_t __attribute__((ext_vector_type(2)));
typedef short s16x4_t __attribute__((ext_vector_type(4)));
typedef float f4v __attribute__((ext_vector_type(4)));
typedef unsigned u4v __attribute__((ext_vector_type(4)));

constexpr int HQ = 16; // grid points per wavefront
constexpr int HK = 32; // band positions per step
constexpr int HG = 16; // latitudes (in launch order) whose tiles of one longitude range are issued back to back: they run at
                       // the same time on one XCD and fetch the same K/V (Q/dY) rows, so all but the first hit in its L2

template <typename T> struct H16;
template <> struct H16<bf16_t> {
    static __device__ inline f4v mfma(uint4 a, uint4 b, f4v c)
    {
        return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, a), __builtin_bit_cast(bf16x8_t, b), c, 0, 0, 0);
    }
    static __device__ inline unsigned pack2(float lo, float hi)
    {
        bf16x2_t r = {(__bf16)lo, (__bf16)hi};
        return __builtin_bit_cast(unsigned, r);
    }
    static __device__ inline float2 unpack2(unsigned u) { return make_float2(__uint_as_float(u << 16), __uint_as_float(u & 0xffff0000u)); }
};
template <> struct H16<f16_t> {
    static __device__ inline f4v mfma(uint4 a, uint4 b, f4v c)
    {
        return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8_t, a), __builtin_bit_cast(f16x8_t, b), c, 0, 0, 0);
    }
    static __device__ inline unsigned pack2(float lo, float hi)
    {
        f16x2_t r = {(_Float16)lo, (_Float16)hi};
        return __builtin_bit_cast(unsigned, r);
    }
    static __device__ inline float2 unpack2(unsigned u)
    {
        const f16x2_t r = __builtin_bit_cast(f16x2_t, u);
        return make_float2((float)r[0], (float)r[1]);
    }
};

// 32 consecutive longitudes (c0.., wrapping once at W) of one latitude/head as a [32][row] LDS tile: rows of CPR_
// 16-byte pieces, PITCH_ bytes apart.  fetch() keeps the tile in registers (one 16-byte load per lane per iteration) so
// that the loads of the next step fly while the current one is consumed; commit() writes it to LDS.
template <int CPR_, int PITCH_> struct BandTile {
    static constexpr int CPR = CPR_;         // 16-byte pieces per row
    static constexpr int RPI = 64 / CPR;     // rows per iteration
    static constexpr int NIT = HK / RPI;     // iterations
    static constexpr int PITCH = PITCH_;     // bytes
    u4v raw[NIT];
    // Byte offsets of this lane's pieces inside one latitude of one (batch, head) slice; the same for every tensor of
    // a step (k and v, or q and dy).  lane_off = (lane / CPR) * ldb + 16 * (lane % CPR).
    static __device__ inline void offsets(unsigned (&off)[NIT], unsigned lane_off, int lane, int c0, int W, unsigned ldb)
    {
        const int r0 = lane / CPR;
        const int lim = W - c0; // staged rows from lim on wrap around the circle
        const unsigned base = (unsigned)c0 * ldb + lane_off;
#pragma unroll
        for (int it = 0; it < NIT; it++) off[it] = base + (unsigned)(it * RPI) * ldb - ((r0 >= lim - it * RPI) ? (unsigned)W * ldb : 0u);
    }
    __device__ inline void fetch(const char *src, const unsigned (&off)[NIT])
    {
#pragma unroll
        for (int it = 0; it < NIT; it++) raw[it] = *reinterpret_cast<const u4v *>(src + off[it]);
    }
    // the same for a lane that may own a piece beyond the end of the row (a head narrower than the tile): it stages zeros
    __device__ inline void fetch_if(const char *src, const unsigned (&off)[NIT], bool valid)
    {
        if (valid) {
#pragma unroll
            for (int it = 0; it < NIT; it++) raw[it] = *reinterpret_cast<const u4v *>(src + off[it]);
        } else {
#pragma unroll
            for (int it = 0; it < NIT; it++) raw[it] = u4v{0u, 0u, 0u, 0u};
        }
    }
    __device__ inline void commit(char *dst, int lane) const
    {
        const int r0 = lane / CPR, cb = 16 * (lane % CPR);
#pragma unroll
        for (int it = 0; it < NIT; it++) *reinterpret_cast<u4v *>(dst + (r0 + it * RPI) * PITCH + cb) = raw[it];
    }
};

// 16-bit tile of D channels.  Row pitch measured with SQ_LDS_BANK_CONFLICT: pitches of 32 or 96 bytes modulo 128 are free
// of bank conflicts for all three access patterns (16-byte row pieces by lanes (c, qd), transposing 8-byte reads, 16-byte
// writes); 2 D + 16 costs both reads 2x.
template <int D> struct HTile : BandTile<D / 8, 2 * D + 32> {};

// A operand "channels 16 cb + c, positions (kb, v) of this lane's quarter" from a [position][channel] tile
template <int PITCH> __device__ inline uint4 h16_read_transposed(const char *tile, int cb, int c, int qd)
{
    typedef s16x4_t __attribute__((address_space(3))) * lds_ptr;
    const char *p0 = tile + (4 * qd + (c >> 2)) * PITCH + 32 * cb + 8 * (c & 3);
    const s16x4_t r0 = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_ptr)(p0));
    const s16x4_t r1 = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_ptr)(p0 + 16 * PITCH));
    const uint2 u0 = __builtin_bit_cast(uint2, r0), u1 = __builtin_bit_cast(uint2, r1);
    return make_uint4(u0.x, u0.y, u1.x, u1.y);
}

// A operand "row 16 kb + c, channels 32 s + 8 qd .. + 8" (plain 16-byte read)
template <int PITCH> __device__ inline uint4 h16_read_row(const char *tile, int kb, int s, int c, int qd)
{
    return *reinterpret_cast<const uint4 *>(tile + (16 * kb + c) * PITCH + 64 * s + 16 * qd);
}

// one 16-byte piece of a grid point's vector, zeros when the head ends before it
__device__ inline uint4 h16_load_piece(const char *p, bool ok)
{
    uint4 r = make_uint4(0u, 0u, 0u, 0u);
    if (ok) r = *reinterpret_cast<const uint4 *>(p);
    return r;
}

__device__ inline float h16_quarter_max(float x)
{
    return xor32_max(xor16_max(x));
}
__device__ inline float h16_quarter_sum(float x)
{
    return xor32_sum(xor16_sum(x));
}

// Workgroup index -> ((batch, head), index inside it).  The hardware deals consecutive workgroups round-robin to the 8
// XCDs, each with its own L2: when the number of (batch, head) slices is a multiple of 8, slice x + 8 n is worked on
// by XCD x only, one slice at a time, so that the K/V (or Q/dY) latitudes its tiles share stay in that L2.
__device__ inline void xcd_split(int id, int BH, int per_bh, int &bh, int &rest)
{
    if ((BH & 7) == 0) {
        const int r = id >> 3;
        bh = (id & 7) + 8 * (r / per_bh);
        rest = r % per_bh;
    } else {
        bh = id % BH;
        rest = id / BH;
    }
}

#define S2_H16_IDS(W_TILED, NROWS)                                            \
    const int lane = threadIdx.x;                                             \
    const int c = lane & 15, qd = lane >> 4;                                  \
    const int BH = a.B * a.nh;                                                \
    const int ntile = ((W_TILED) + HQ - 1) / HQ;                              \
    int bh, id_;                                                              \
    xcd_split(blockIdx.x, BH, ntile *(NROWS), bh, id_);                       \
    const int grp_ = id_ / (HG * ntile);                                      \
    const int grows_ = min(HG, (NROWS)-grp_ * HG);                            \
    id_ -= grp_ * HG * ntile;                                                 \
    const int wt = id_ / grows_;                                              \
    const int rowsel = grp_ * HG + id_ % grows_;                              \
    const int b = bh / a.nh, h = bh % a.nh;                                   \
    const int w0 = wt * HQ;                                                   \
    const int nvalid = min(HQ, (W_TILED)-w0);

// ---- forward ---------------------------------------------------------------------------------------------------
template <typename T, int D, bool PAD> __global__ __launch_bounds__(64) void fwd_h16_kernel(const Args a)
{
    typedef HTile<D> Tile;
    typedef H16<T> M;
    constexpr int PITCH = Tile::PITCH, NS = D / 32, NCB = D / 16;
    __shared__ __attribute__((aligned(16))) char Ks[HK * PITCH];
    __shared__ __attribute__((aligned(16))) char Vs[HK * PITCH];

    S2_H16_IDS(a.Wo, a.Ho)
    const int ho = a.gorder[a.row_first + rowsel];
    const int dr = PAD ? a.dk_ : D;     // real head width (PAD = false: a compile-time constant, every mask below folds away)
    const unsigned ldb = a.nh * dr * 2; // bytes between two grid points
    const char *kx = static_cast<const char *>(a.k) + ((size_t)b * a.Hi * a.Wi * a.nh + h) * (dr * 2);
    const char *vx = static_cast<const char *>(a.v) + ((size_t)b * a.Hi * a.Wi * a.nh + h) * (dr * 2);
    const bool mine = c < nvalid;
    const size_t pt = (size_t)query_point(a, b, ho, ho / a.qps) + (size_t)(w0 + (mine ? c : 0)) * a.qps;

    uint4 qop[NS]; // B operand of S^T = K Q^T: channels 32 s + 8 qd .. + 8 of column c
    {
        const char *qrow = static_cast<const char *>(a.q) + pt * ldb + (size_t)h * (dr * 2) + 16 * qd;
#pragma unroll
        for (int s = 0; s < NS; s++) qop[s] = h16_load_piece(qrow + 64 * s, 32 * s + 8 * qd < dr);
    }
    f4v acc[NCB]; // Y^T: register v of block cb is channel 16 cb + 4 qd + v of column c
#pragma unroll
    for (int cb = 0; cb < NCB; cb++) acc[cb] = f4v{0.f, 0.f, 0.f, 0.f};
    float m = NEG_BIG, S = 0.f;

    int ri = a.goff[ho];
    const int rend = a.goff[ho + 1];
    int pos = 0;
    Run run = {0, 0, 0, 0};
    Tile kt, vt;
    const unsigned ldbk = ldb * a.kps; // bytes between two columns of a virtual input latitude
    const unsigned lane_off = (unsigned)(lane / Tile::CPR) * ldbk + 16u * (lane % Tile::CPR);
    const bool piece_ok = 8 * (lane % Tile::CPR) < dr; // this lane's 16-byte piece of a staged row exists
    auto fetch = [&](const Run &rn, int p) {
        const int c0 = (rn.ws + w0 + p) % a.Wi;
        unsigned off[Tile::NIT];
        Tile::offsets(off, lane_off, lane, c0, a.Wi, ldbk);
        const size_t lat_off = (size_t)key_row(a, rn.lat, rn.pad) * ldb;
        kt.fetch_if(kx + lat_off, off, piece_ok);
        vt.fetch_if(vx + lat_off, off, piece_ok);
    };
    if (ri < rend) {
        run = a.gruns[ri];
        fetch(run, 0);
        kt.commit(Ks, lane);
        vt.commit(Vs, lane);
    }
    __syncthreads();
    settle(qop);

    while (ri < rend) {
        const float lw = fast_log2(a.quad_w[run.pad]);
        const int len = run.len;
        int nri = ri, npos = pos + HK;
        Run nrun = run;
        if (npos >= len + HQ - 1) {
            nri++;
            npos = 0;
            if (nri < rend) nrun = a.gruns[nri];
        }
        const bool more = nri < rend;
        if (more) fetch(nrun, npos);

        f4v sc[2];
#pragma unroll
        for (int kb = 0; kb < 2; kb++) {
            sc[kb] = f4v{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int s = 0; s < NS; s++) sc[kb] = M::mfma(h16_read_row<PITCH>(Ks, kb, s, c, qd), qop[s], sc[kb]);
        }
        // band mask, running maximum (of score * log2 e + log2 w, common to the four lanes of a column), probabilities
        const int tb = pos + 4 * qd - c; // neighbor index of element (kb, v): tb + 16 kb + v
        float mx = -INFINITY;
        if (pos >= HQ - 1 && pos + HK <= len) { // every element of the step is a neighbor: no band mask (most steps of a long run)
#pragma unroll
            for (int kb = 0; kb < 2; kb++) {
#pragma unroll
                for (int v = 0; v < 4; v++) mx = fmaxf(mx, sc[kb][v]);
            }
        } else {
#pragma unroll
            for (int kb = 0; kb < 2; kb++) {
#pragma unroll
                for (int v = 0; v < 4; v++) {
                    const unsigned t = (unsigned)(tb + 16 * kb + v);
                    sc[kb][v] = (t < (unsigned)len) ? sc[kb][v] : -INFINITY;
                    mx = fmaxf(mx, sc[kb][v]);
                }
            }
        }
        mx = h16_quarter_max(mx);
        const float mn = fmaxf(m, fmaf(mx, LOG2E, lw)); // m starts finite, so mn is finite
        if (__any(mn > m)) {
            const float corr = fast_exp2(m - mn);
            S *= corr;
#pragma unroll
            for (int cb = 0; cb < NCB; cb++) acc[cb] *= corr;
        }
        m = mn;
        const float sh = lw - mn;
#pragma unroll
        for (int kb = 0; kb < 2; kb++) {
#pragma unroll
            for (int v = 0; v < 4; v++) {
                const float p = fast_exp2(fmaf(sc[kb][v], LOG2E, sh)); // masked: exp2(-inf) = 0
                sc[kb][v] = p;
                S += p; // this lane's share; the four lanes of a column are added up at the end
            }
        }
        const uint4 pop = make_uint4(M::pack2(sc[0][0], sc[0][1]), M::pack2(sc[0][2], sc[0][3]), M::pack2(sc[1][0], sc[1][1]), M::pack2(sc[1][2], sc[1][3]));
#pragma unroll
        for (int cb = 0; cb < NCB; cb++) acc[cb] = M::mfma(h16_read_transposed<PITCH>(Vs, cb, c, qd), pop, acc[cb]);

        __syncthreads();
        if (more) {
            kt.commit(Ks, lane);
            vt.commit(Vs, lane);
        }
        __syncthreads();
        ri = nri;
        pos = npos;
        run = nrun;
    }

    S = h16_quarter_sum(S);
    if (mine) {
        if (a.lse && qd == 0) a.lse[((size_t)bh * a.Ho + ho) * a.Wo + w0 + c] = m + fast_log2(S);
        const float inv = 1.0f / S;
        char *y = static_cast<char *>(a.y) + pt * ldb + (size_t)h * (dr * 2) + 8 * qd;
#pragma unroll
        for (int cb = 0; cb < NCB; cb++)
            if (16 * cb + 4 * qd < dr)
                *reinterpret_cast<uint2 *>(y + 32 * cb) = make_uint2(M::pack2(acc[cb][0] * inv, acc[cb][1] * inv), M::pack2(acc[cb][2] * inv, acc[cb][3] * inv));
    }
}

// ---- backward, dq pass (needs the forward's y and lse) -------------------------------------------------------------
// Three products per step:  S^T = K Q^T,  G^T = V dY^T,  dQ^T += K^T dS^T  with dS = P o (G - I),  I = <dy, y>.
template <typename T, int D, bool PAD> __global__ __launch_bounds__(64) void dq_h16_kernel(const Args a)
{
    typedef HTile<D> Tile;
    typedef H16<T> M;
    constexpr int PITCH = Tile::PITCH, NS = D / 32, NCB = D / 16;
    __shared__ __attribute__((aligned(16))) char Ks[HK * PITCH];
    __shared__ __attribute__((aligned(16))) char Vs[HK * PITCH];

    S2_H16_IDS(a.Wo, a.Ho)
    const int ho = a.gorder[a.row_first + rowsel];
    const int dr = PAD ? a.dk_ : D;
    const unsigned ldb = a.nh * dr * 2;
    const char *kx = static_cast<const char *>(a.k) + ((size_t)b * a.Hi * a.Wi * a.nh + h) * (dr * 2);
    const char *vx = static_cast<const char *>(a.v) + ((size_t)b * a.Hi * a.Wi * a.nh + h) * (dr * 2);
    const bool mine = c < nvalid;
    const size_t pt = (size_t)query_point(a, b, ho, ho / a.qps) + (size_t)(w0 + (mine ? c : 0)) * a.qps;
    const size_t sidx = ((size_t)bh * a.Ho + ho) * a.Wo + w0 + (mine ? c : 0);

    uint4 qop[NS], gop[NS];
    float I = 0.f;
    {
        const size_t off = pt * ldb + (size_t)h * (dr * 2) + 16 * qd;
#pragma unroll
        for (int s = 0; s < NS; s++) {
            const bool ok = 32 * s + 8 * qd < dr;
            qop[s] = h16_load_piece(static_cast<const char *>(a.q) + off + 64 * s, ok);
            gop[s] = h16_load_piece(static_cast<const char *>(a.dy) + off + 64 * s, ok);
            const uint4 yv = h16_load_piece(static_cast<const char *>(a.ysaved) + off + 64 * s, ok);
            const unsigned gu[4] = {gop[s].x, gop[s].y, gop[s].z, gop[s].w}, yu[4] = {yv.x, yv.y, yv.z, yv.w};
#pragma unroll
            for (int i = 0; i < 4; i++) {
                const float2 g2 = M::unpack2(gu[i]), y2 = M::unpack2(yu[i]);
                I = fmaf(g2.x, y2.x, I);
                I = fmaf(g2.y, y2.y, I);
            }
        }
    }
    I = h16_quarter_sum(I);
    const float lse = a.lse[sidx];

    f4v acc[NCB];
#pragma unroll
    for (int cb = 0; cb < NCB; cb++) acc[cb] = f4v{0.f, 0.f, 0.f, 0.f};

    int ri = a.goff[ho];
    const int rend = a.goff[ho + 1];
    int pos = 0;
    Run run = {0, 0, 0, 0};
    Tile kt, vt;
    const unsigned ldbk = ldb * a.kps; // bytes between two columns of a virtual input latitude
    const unsigned lane_off = (unsigned)(lane / Tile::CPR) * ldbk + 16u * (lane % Tile::CPR);
    const bool piece_ok = 8 * (lane % Tile::CPR) < dr; // this lane's 16-byte piece of a staged row exists
    auto fetch = [&](const Run &rn, int p) {
        const int c0 = (rn.ws + w0 + p) % a.Wi;
        unsigned off[Tile::NIT];
        Tile::offsets(off, lane_off, lane, c0, a.Wi, ldbk);
        const size_t lat_off = (size_t)key_row(a, rn.lat, rn.pad) * ldb;
        kt.fetch_if(kx + lat_off, off, piece_ok);
        vt.fetch_if(vx + lat_off, off, piece_ok);
    };
    if (ri < rend) {
        run = a.gruns[ri];
        fetch(run, 0);
        kt.commit(Ks, lane);
        vt.commit(Vs, lane);
    }
    __syncthreads();
    settle(qop);
    settle(gop);
    float lse_ = lse;
    settle(lse_);

    while (ri < rend) {
        const float lwl = fast_log2(a.quad_w[run.pad]) - lse_;
        const int len = run.len;
        int nri = ri, npos = pos + HK;
        Run nrun = run;
        if (npos >= len + HQ - 1) {
            nri++;
            npos = 0;
            if (nri < rend) nrun = a.gruns[nri];
        }
        const bool more = nri < rend;
        if (more) fetch(nrun, npos);

        f4v sc[2], gc[2];
#pragma unroll
        for (int kb = 0; kb < 2; kb++) {
            sc[kb] = f4v{0.f, 0.f, 0.f, 0.f};
            gc[kb] = f4v{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int s = 0; s < NS; s++) {
                sc[kb] = M::mfma(h16_read_row<PITCH>(Ks, kb, s, c, qd), qop[s], sc[kb]);
                gc[kb] = M::mfma(h16_read_row<PITCH>(Vs, kb, s, c, qd), gop[s], gc[kb]);
            }
        }
        const int tb = pos + 4 * qd - c;
        if (pos >= HQ - 1 && pos + HK <= len) { // every element of the step is a neighbor: no band mask
#pragma unroll
            for (int kb = 0; kb < 2; kb++) {
#pragma unroll
                for (int v = 0; v < 4; v++) gc[kb][v] = fast_exp2(fmaf(sc[kb][v], LOG2E, lwl)) * (gc[kb][v] - I);
            }
        } else {
#pragma unroll
            for (int kb = 0; kb < 2; kb++) {
#pragma unroll
                for (int v = 0; v < 4; v++) {
                    const unsigned t = (unsigned)(tb + 16 * kb + v);
                    const float p = (t < (unsigned)len) ? fast_exp2(fmaf(sc[kb][v], LOG2E, lwl)) : 0.f;
                    gc[kb][v] = p * (gc[kb][v] - I);
                }
            }
        }
        const uint4 dop = make_uint4(M::pack2(gc[0][0], gc[0][1]), M::pack2(gc[0][2], gc[0][3]), M::pack2(gc[1][0], gc[1][1]), M::pack2(gc[1][2], gc[1][3]));
#pragma unroll
        for (int cb = 0; cb < NCB; cb++) acc[cb] = M::mfma(h16_read_transposed<PITCH>(Ks, cb, c, qd), dop, acc[cb]);

        __syncthreads();
        if (more) {
            kt.commit(Ks, lane);
            vt.commit(Vs, lane);
        }
        __syncthreads();
        ri = nri;
        pos = npos;
        run = nrun;
    }

    // (stored after the walk: a global store ahead of the loop would turn the loop's scalar loads of runs and weights,
    // which the compiler only uses while nothing in the kernel can have written memory, into vector loads with waits)
    if (mine && qd == 0) a.stats[sidx] = make_float2(lse, I);
    if (mine) {
        char *dq = static_cast<char *>(a.dq) + pt * ldb + (size_t)h * (dr * 2) + 8 * qd;
#pragma unroll
        for (int cb = 0; cb < NCB; cb++)
            if (16 * cb + 4 * qd < dr)
                *reinterpret_cast<uint2 *>(dq + 32 * cb) = make_uint2(M::pack2(acc[cb][0], acc[cb][1]), M::pack2(acc[cb][2], acc[cb][3]));
    }
}

// ---- backward, dk/dv pass: transposed gather ---------------------------------------------------------------------
// The wavefront owns 16 INPUT longitudes (column c = key) and walks the runs grouped by input latitude; staged rows
// are queries.  Staged row r of a run (first row = longitude w0 - ws - len + 1) sees key c iff 0 <= r - c < len.
// Four products per step:  S = Q K^T,  G = dY V^T  (rows = queries, columns = keys),  dV^T += dY^T P,  dK^T += Q^T dS.
template <typename T, int D, bool PAD> __global__ __launch_bounds__(64) void dkdv_h16_kernel(const Args a)
{
    typedef HTile<D> Tile;
    typedef H16<T> M;
    constexpr int PITCH = Tile::PITCH, NS = D / 32, NCB = D / 16;
    __shared__ __attribute__((aligned(16))) char Qs[HK * PITCH];
    __shared__ __attribute__((aligned(16))) char Gs[HK * PITCH];
    __shared__ __attribute__((aligned(16))) float Ls[HK];
    __shared__ __attribute__((aligned(16))) float Is[HK];

    S2_H16_IDS(a.Wi, a.Hi)
    const int hi = a.sorder[a.row_first + rowsel];
    const int dr = PAD ? a.dk_ : D;
    const unsigned ldb = a.nh * dr * 2;
    const char *qy = static_cast<const char *>(a.q) + ((size_t)b * a.Ho * a.Wo * a.nh + h) * (dr * 2);
    const char *gy = static_cast<const char *>(a.dy) + ((size_t)b * a.Ho * a.Wo * a.nh + h) * (dr * 2);
    const float2 *stats = a.stats + (size_t)bh * a.Ho * a.Wo;
    const bool mine = c < nvalid;
    const size_t pt = (size_t)key_point(a, b, hi, hi / a.kps) + (size_t)(w0 + (mine ? c : 0)) * a.kps;

    uint4 kop[NS], vop[NS]; // B operands: channels 32 s + 8 qd .. + 8 of key c
    {
        const size_t off = pt * ldb + (size_t)h * (dr * 2) + 16 * qd;
#pragma unroll
        for (int s = 0; s < NS; s++) {
            const bool ok = 32 * s + 8 * qd < dr;
            kop[s] = h16_load_piece(static_cast<const char *>(a.k) + off + 64 * s, ok);
            vop[s] = h16_load_piece(static_cast<const char *>(a.v) + off + 64 * s, ok);
        }
    }
    f4v dkt[NCB], dvt[NCB];
#pragma unroll
    for (int cb = 0; cb < NCB; cb++) {
        dkt[cb] = f4v{0.f, 0.f, 0.f, 0.f};
        dvt[cb] = f4v{0.f, 0.f, 0.f, 0.f};
    }
    const float lw = fast_log2(a.quad_w[hi / a.kps]);

    int ri = a.soff[hi];
    const int rend = a.soff[hi + 1];
    int pos = 0;
    Run run = {0, 0, 0, 0};
    Tile qt, gt;
    float2 st = make_float2(0.f, 0.f);
    const unsigned ldbq = ldb * a.qps; // bytes between two columns of a virtual output latitude
    const unsigned lane_off = (unsigned)(lane / Tile::CPR) * ldbq + 16u * (lane % Tile::CPR);
    const bool piece_ok = 8 * (lane % Tile::CPR) < dr; // this lane's 16-byte piece of a staged row exists
    auto fetch = [&](const Run &rn, int p) {
        int c0 = (w0 - rn.ws - rn.len + 1 + p) % a.Wo; // longitude of staged row 0
        c0 += (c0 < 0) ? a.Wo : 0;
        unsigned off[Tile::NIT];
        Tile::offsets(off, lane_off, lane, c0, a.Wo, ldbq);
        const size_t lat_off = (size_t)query_row(a, rn.lat, rn.pad) * ldb;
        qt.fetch_if(qy + lat_off, off, piece_ok);
        gt.fetch_if(gy + lat_off, off, piece_ok);
        int col = c0 + lane; // lanes 0..31 fetch the statistics of the staged rows
        col -= (col >= a.Wo) ? a.Wo : 0;
        if (lane < HK) st = stats[(size_t)rn.lat * a.Wo + col];
    };
    auto commit = [&]() {
        qt.commit(Qs, lane);
        gt.commit(Gs, lane);
        if (lane < HK) {
            Ls[lane] = st.x;
            Is[lane] = st.y;
        }
    };
    if (ri < rend) {
        run = a.sruns[ri];
        fetch(run, 0);
        commit();
    }
    __syncthreads();
    settle(kop);
    settle(vop);

    while (ri < rend) {
        const int len = run.len;
        int nri = ri, npos = pos + HK;
        Run nrun = run;
        if (npos >= len + HQ - 1) {
            nri++;
            npos = 0;
            if (nri < rend) nrun = a.sruns[nri];
        }
        const bool more = nri < rend;
        if (more) fetch(nrun, npos);

        f4v sc[2], gc[2];
#pragma unroll
        for (int qb = 0; qb < 2; qb++) {
            sc[qb] = f4v{0.f, 0.f, 0.f, 0.f};
            gc[qb] = f4v{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int s = 0; s < NS; s++) {
                sc[qb] = M::mfma(h16_read_row<PITCH>(Qs, qb, s, c, qd), kop[s], sc[qb]);
                gc[qb] = M::mfma(h16_read_row<PITCH>(Gs, qb, s, c, qd), vop[s], gc[qb]);
            }
        }
        const int tb = pos + 4 * qd - c; // r - c of element (qb, v): tb + 16 qb + v
        const bool inner = pos >= HQ - 1 && pos + HK <= len; // every element of the step is a (query, key) pair of the run
#pragma unroll
        for (int qb = 0; qb < 2; qb++) {
            const float4 l4 = *reinterpret_cast<const float4 *>(Ls + 16 * qb + 4 * qd);
            const float4 i4 = *reinterpret_cast<const float4 *>(Is + 16 * qb + 4 * qd);
            const float lv[4] = {l4.x, l4.y, l4.z, l4.w};
            const float iv[4] = {i4.x, i4.y, i4.z, i4.w};
#pragma unroll
            for (int v = 0; v < 4; v++) {
                float p = fast_exp2(fmaf(sc[qb][v], LOG2E, lw - lv[v]));
                if (!inner) p = ((unsigned)(tb + 16 * qb + v) < (unsigned)len) ? p : 0.f; // band mask, first and last steps of a run only
                sc[qb][v] = p;
                gc[qb][v] = p * (gc[qb][v] - iv[v]);
            }
        }
        const uint4 pop = make_uint4(M::pack2(sc[0][0], sc[0][1]), M::pack2(sc[0][2], sc[0][3]), M::pack2(sc[1][0], sc[1][1]), M::pack2(sc[1][2], sc[1][3]));
        const uint4 dop = make_uint4(M::pack2(gc[0][0], gc[0][1]), M::pack2(gc[0][2], gc[0][3]), M::pack2(gc[1][0], gc[1][1]), M::pack2(gc[1][2], gc[1][3]));
#pragma unroll
        for (int cb = 0; cb < NCB; cb++) {
            dvt[cb] = M::mfma(h16_read_transposed<PITCH>(Gs, cb, c, qd), pop, dvt[cb]);
            dkt[cb] = M::mfma(h16_read_transposed<PITCH>(Qs, cb, c, qd), dop, dkt[cb]);
        }

        __syncthreads();
        if (more) commit();
        __syncthreads();
        ri = nri;
        pos = npos;
        run = nrun;
    }

    if (mine) {
        const size_t off = pt * ldb + (size_t)h * (dr * 2) + 8 * qd;
        char *dk = static_cast<char *>(a.dk) + off, *dv = static_cast<char *>(a.dv) + off;
#pragma unroll
        for (int cb = 0; cb < NCB; cb++) {
            if (16 * cb + 4 * qd < dr) {
                *reinterpret_cast<uint2 *>(dk + 32 * cb) = make_uint2(M::pack2(dkt[cb][0], dkt[cb][1]), M::pack2(dkt[cb][2], dkt[cb][3]));
                *reinterpret_cast<uint2 *>(dv + 32 * cb) = make_uint2(M::pack2(dvt[cb][0], dvt[cb][1]), M::pack2(dvt[cb][2], dvt[cb][3]));
            }
        }
    }
}
