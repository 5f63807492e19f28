// Matrix-core kernels for 16-bit storage (bf16, fp16): forward, dq and dk/dv with v_mfma_f32_16x16x32_{bf16,f16}.
// Included by s2attn_kernels.hip inside namespace s2 (uses its Args, Run and storage types).
//
// Shape domain: ck == cv = dr, a multiple of 8 with dr <= D (the tile is D channels wide, D a multiple of 32; channels
// from dr on are staged as zeros and never stored), at least 32 columns per virtual latitude, 16-byte aligned rows.
//
// A workgroup of NW = 4 wavefronts owns 64 consecutive longitudes of one latitude for one (batch, head); wavefront w owns
// HQ = 16 of them and walks every run of that latitude in steps of HK = 32 band positions (len + 15 positions per run;
// position u belongs to the neighborhood of column c iff 0 <= u - c < len).  The four walks read one staged band: band
// row x of a run is the grid point "first longitude of the workgroup + run start + x", wavefront w is at rows
// 16 w + pos .. + 32 in a step, so a run starts with 80 staged rows and every further step adds 32 for the whole
// workgroup (each wavefront alone would stage 32 per step: loads through the vector L1 (64 B/clk per CU) and LDS writes
// (about 75 B/clk per CU measured, against 215 B/clk for 16-byte LDS reads) are what these kernels run out of first).
// The band lives in LDS as a ring of BR = 128 rows: the 32 rows of the next step never overlap the 80 rows in use, so a
// step inside a run needs one barrier; the first step of the next run replaces rows in use and needs two.
// Lane l = (c = l % 16, qd = l / 16).  Facts about the instruction used below:
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

constexpr int HQ = 16;                    // grid points per wavefront
constexpr int HK = 32;                    // band positions per step
constexpr int NW = 4;                     // wavefronts per workgroup
constexpr int WQ = HQ * NW;               // grid points per workgroup
constexpr int FRESH = HK + HQ * (NW - 1); // band rows the first step of a run needs
constexpr int BR = 128;                   // rows of the LDS ring (a power of two, a multiple of 16, at least FRESH + HK)
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

// (Staging of the fp32 family, s2attn_m32.hpp, one band per wavefront.)  32 consecutive longitudes (c0.., wrapping once at W) of one latitude/head as a [32][row] LDS tile: rows of CPR_
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

// The staged band of two tensors that share their addressing (k and v, or q and dy): rows of CPR 16-byte pieces, PITCH
// bytes apart, row x of the run at ring row x % BR.  fetch() loads rows x0 .. x0 + n of the run into registers, one
// 16-byte piece per thread per iteration and tensor (the loads fly while the current step is consumed); commit() writes
// them to LDS.  Row pitch measured with SQ_LDS_BANK_CONFLICT: pitches of 32 or 96 bytes modulo 128 are free of bank
// conflicts for all three access patterns (16-byte row pieces by lanes (c, qd), transposing 8-byte reads, 16-byte
// writes); 2 D + 16 costs both reads 2x.
template <int D> struct WgBand {
    static constexpr int CPR = D / 8;                   // 16-byte pieces per row
    static constexpr int PITCH = 2 * D + 32;            // bytes
    static constexpr int RPI = 64 * NW / CPR;           // rows per iteration of the workgroup
    static constexpr int NIT = (FRESH + RPI - 1) / RPI; // iterations for the first step of a run
    static constexpr int BYTES = BR * PITCH;            // one tensor's ring
    u4v ra[NIT], rb[NIT];

    // cs: longitude of the first of the N rows on the circle of W columns (0 <= cs < W); ldc: bytes between two columns.
    // N (FRESH or HK) is the number of rows; iterations and row tests that N rules out are not compiled.
    template <int N, bool PAD> __device__ inline void fetch(const char *pa, const char *pb, int tid, int cs, int W, unsigned ldc, bool piece_ok)
    {
        const int r0 = tid / CPR;
        const unsigned pc = 16u * (tid % CPR);
#pragma unroll
        for (int it = 0; it < (N + RPI - 1) / RPI; it++) {
            if (PAD) { // a thread may own a piece beyond the end of the row (a head narrower than the tile): it stages zeros
                ra[it] = u4v{0u, 0u, 0u, 0u};
                rb[it] = u4v{0u, 0u, 0u, 0u};
            }
            if (((it + 1) * RPI <= N || it * RPI + r0 < N) && (!PAD || piece_ok)) {
                unsigned col = (unsigned)(cs + r0); // r0 < RPI <= 64 <= 2 W
                col = min(col, col - (unsigned)W);  // col - W wraps to a huge value when col < W
                if (RPI > 32) col = min(col, col - (unsigned)W);
                const unsigned off = col * ldc + pc;
                ra[it] = *reinterpret_cast<const u4v *>(pa + off);
                rb[it] = *reinterpret_cast<const u4v *>(pb + off);
            }
            cs += RPI;
            while (cs >= W) cs -= W;
        }
    }
    template <int N> __device__ inline void commit(char *A, char *B, int tid, int x0) const
    {
        const int r0 = tid / CPR, pc = 16 * (tid % CPR);
#pragma unroll
        for (int it = 0; it < (N + RPI - 1) / RPI; it++) {
            if ((it + 1) * RPI <= N || it * RPI + r0 < N) {
                const int o = ((x0 + it * RPI + r0) & (BR - 1)) * PITCH + pc;
                *reinterpret_cast<u4v *>(A + o) = ra[it];
                *reinterpret_cast<u4v *>(B + o) = rb[it];
            }
        }
    }
};

// start of the 16 ring rows that hold band rows x .. x + 16 (x a multiple of 16)
template <int PITCH> __device__ inline const char *band_block(const char *ring, int x)
{
    return ring + (x & (BR - 1)) * PITCH;
}

// A operand "channels 16 cb + c, positions (kb, v) of this lane's quarter" from the two 16-row blocks of a step
// ([position][channel] rows)
template <int PITCH> __device__ inline uint4 h16_read_transposed(const char *blk0, const char *blk1, int cb, int c, int qd)
{
    typedef s16x4_t __attribute__((address_space(3))) * lds_ptr;
    const int o = (4 * qd + (c >> 2)) * PITCH + 32 * cb + 8 * (c & 3);
    const s16x4_t r0 = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_ptr)(blk0 + o));
    const s16x4_t r1 = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_ptr)(blk1 + o));
    const uint2 u0 = __builtin_bit_cast(uint2, r0), u1 = __builtin_bit_cast(uint2, r1);
    return make_uint4(u0.x, u0.y, u1.x, u1.y);
}

// A operand "row c of the block, channels 32 s + 8 qd .. + 8" (plain 16-byte read)
template <int PITCH> __device__ inline uint4 h16_read_row(const char *blk, int s, int c, int qd)
{
    return *reinterpret_cast<const uint4 *>(blk + c * PITCH + 64 * s + 16 * qd);
}

// one 16-byte piece of a grid point's vector, zeros when the head ends before it
__device__ inline uint4 h16_load_piece(const char *p, bool ok)
{
    uint4 r = make_uint4(0u, 0u, 0u, 0u);
    if (ok) r = *reinterpret_cast<const uint4 *>(p);
    return r;
}

// A 16-byte piece (eight 16-bit values) times log2 e, rounded back to the storage type: the q (or k) operand of the score product
// then yields scores in the log2 domain straight from the matrix cores.  The rounding is one more of the size the storage type
// already made (2^-9 relative for bf16), independent per channel.
template <typename M> __device__ inline uint4 h16_scale_log2e(uint4 x)
{
    unsigned u[4] = {x.x, x.y, x.z, x.w};
#pragma unroll
    for (int i = 0; i < 4; i++) {
        const float2 f = M::unpack2(u[i]);
        u[i] = M::pack2(f.x * LOG2E, f.y * LOG2E);
    }
    return make_uint4(u[0], u[1], u[2], u[3]);
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
    const int tid = threadIdx.x;                                              \
    const int lane = tid & 63, wave = tid >> 6;                               \
    const int c = lane & 15, qd = lane >> 4;                                  \
    const int BH = a.B * a.nh;                                                \
    const int ntile = ((W_TILED) + WQ - 1) / WQ;                              \
    int bh, id_;                                                              \
    xcd_split(blockIdx.x, BH, ntile *(NROWS), bh, id_);                       \
    const int grp_ = id_ / (HG * ntile);                                      \
    const int grows_ = min(HG, (NROWS)-grp_ * HG);                            \
    id_ -= grp_ * HG * ntile;                                                 \
    const int wt = id_ / grows_;                                              \
    const int rowsel = grp_ * HG + id_ % grows_;                              \
    const int b = bh / a.nh, h = bh % a.nh;                                   \
    const int wg0 = wt * WQ;                          /* first longitude of the workgroup */ \
    const bool active = wg0 + HQ * wave < (W_TILED); /* a wavefront past the end of the row only helps staging */ \
    const int w0 = active ? wg0 + HQ * wave : 0;                              \
    const int nvalid = active ? min(HQ, (W_TILED)-w0) : 0;

// ---- forward ---------------------------------------------------------------------------------------------------
// Dynamic LDS of the three kernels: the rings of the two staged tensors (the dk/dv pass keeps two floats per band row in
// the padding of the first ring's rows: with 64 channels the two rings are exactly a quarter of a CU's LDS).
template <int D> constexpr int h16_lds_bytes() { return 2 * WgBand<D>::BYTES; }

// Uniform reads of the plan and the weights inside the walk.  A load through the constant address space is always a
// scalar load; through a plain pointer it becomes a vector load with a full wait as soon as the loop holds a workgroup
// barrier, whose fence the compiler has to assume orders a write to the same memory.  Neither array is written by a kernel.
template <typename V> __device__ inline V uniform_load(const V *p)
{
    typedef const V __attribute__((address_space(4))) * cptr;
    return *(cptr)(p);
}
__device__ inline Run uniform_load(const Run *p)
{
    typedef int i4v __attribute__((ext_vector_type(4)));
    const i4v r = uniform_load(reinterpret_cast<const i4v *>(p));
    return Run{r[0], r[1], r[2], r[3]};
}

// One step of the walk over the runs of a latitude, the same for every wavefront of the workgroup: where the walk
// stands after this step, and what has to be staged for it.
struct H16Walk {
    int ri, rend, pos;
    Run run;
    float w; // quadrature weight of the run's input latitude (gather side), read together with the run: a step before its use
    int nri, npos;
    Run nrun;
    float nw;
    bool more, fresh;
    int cnext; // longitude of the first band row, of the run staged last, that is not staged yet
    // first longitude to stage for the next step: c0 = longitude of band row 0 if that step starts a run (0 <= c0 < 2 W)
    __device__ inline int stage(bool fresh_, int c0, int W)
    {
        int cs = fresh_ ? c0 : cnext;
        while (cs >= W) cs -= W;
        cnext = cs + (fresh_ ? FRESH : HK);
        return cs;
    }
    __device__ inline void plan(const Run *runs, const float *weights = nullptr)
    {
        nri = ri;
        npos = pos + HK;
        nrun = run;
        nw = w;
        if (npos >= run.len + HQ - 1) {
            nri++;
            npos = 0;
            if (nri < rend) {
                nrun = uniform_load(runs + nri);
                if (weights) nw = uniform_load(weights + nrun.pad);
            }
        }
        more = nri < rend;
        fresh = npos == 0;
    }
    __device__ inline void advance()
    {
        ri = nri;
        pos = npos;
        run = nrun;
        w = nw;
    }
};

template <typename T, int D, bool PAD> __global__ __launch_bounds__(64 * NW) void fwd_h16_kernel(const Args a)
{
    typedef WgBand<D> Tile;
    typedef H16<T> M;
    constexpr int PITCH = Tile::PITCH, NS = D / 32, NCB = D / 16;
    extern __shared__ __attribute__((aligned(16))) char h16_lds[];
    char *Ks = h16_lds, *Vs = h16_lds + Tile::BYTES;

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

    H16Walk wk;
    wk.ri = a.goff[ho];
    wk.rend = a.goff[ho + 1];
    wk.pos = 0;
    wk.run = Run{0, 0, 0, 0};
    Tile bd;
    const unsigned ldbk = ldb * a.kps; // bytes between two columns of a virtual input latitude
    const bool piece_ok = 8 * (tid % Tile::CPR) < dr; // this thread's 16-byte piece of a staged row exists
    auto fetch = [&](const Run &rn, bool fresh) {
        const size_t lat_off = (size_t)key_row(a, rn.lat, rn.pad) * ldb;
        const int cs = wk.stage(fresh, rn.ws + wg0, a.Wi);
        if (fresh)
            bd.template fetch<FRESH, PAD>(kx + lat_off, vx + lat_off, tid, cs, a.Wi, ldbk, piece_ok);
        else
            bd.template fetch<HK, PAD>(kx + lat_off, vx + lat_off, tid, cs, a.Wi, ldbk, piece_ok);
    };
    wk.w = 1.f;
    if (wk.ri < wk.rend) {
        wk.run = a.gruns[wk.ri];
        wk.w = a.quad_w[wk.run.pad];
        fetch(wk.run, true);
        bd.template commit<FRESH>(Ks, Vs, tid, 0);
    }
    __syncthreads();
    settle(qop);

    while (wk.ri < wk.rend) {
        wk.plan(a.gruns, a.quad_w);
        if (wk.more) fetch(wk.nrun, wk.fresh);
        if (active) {
            const float lw = fast_log2(wk.w);
            const int len = wk.run.len, pos = wk.pos;
            const int xw = HQ * wave + pos; // band row of this wavefront's position `pos`
            const char *kblk[2] = {band_block<PITCH>(Ks, xw), band_block<PITCH>(Ks, xw + 16)};
            const char *vblk[2] = {band_block<PITCH>(Vs, xw), band_block<PITCH>(Vs, xw + 16)};
            f4v sc[2];
#pragma unroll
            for (int kb = 0; kb < 2; kb++) {
                sc[kb] = f4v{0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int s = 0; s < NS; s++) sc[kb] = M::mfma(h16_read_row<PITCH>(kblk[kb], s, c, qd), qop[s], sc[kb]);
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
            // The running maximum is only the reference point of the exponentials: it moves when a column's maximum has
            // grown by more than RESCALE_THR (probabilities stay below 2^RESCALE_THR), which after a row's first steps is
            // rare; until then the step needs no exchange between the four lanes of a column and no rescaling.
            if (__any(fmaf(mx, LOG2E, lw) > m + RESCALE_THR)) {
                const float cm = fmaf(h16_quarter_max(mx), LOG2E, lw);
                const float mn = (cm > m + RESCALE_THR) ? cm : m; // m starts finite, so mn is finite
                const float corr = fast_exp2(m - mn);
                S *= corr;
#pragma unroll
                for (int cb = 0; cb < NCB; cb++) acc[cb] *= corr;
                m = mn;
            }
            const float sh = lw - m;
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
            for (int cb = 0; cb < NCB; cb++) acc[cb] = M::mfma(h16_read_transposed<PITCH>(vblk[0], vblk[1], cb, c, qd), pop, acc[cb]);
        }
        if (wk.more) {
            if (wk.fresh) {
                __syncthreads(); // the next run's rows replace rows the slowest wavefront may still be reading
                bd.template commit<FRESH>(Ks, Vs, tid, 0);
            } else {
                bd.template commit<HK>(Ks, Vs, tid, FRESH - HK + wk.npos);
            }
        }
        __syncthreads();
        wk.advance();
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
template <typename T, int D, bool PAD> __global__ __launch_bounds__(64 * NW) void dq_h16_kernel(const Args a)
{
    typedef WgBand<D> Tile;
    typedef H16<T> M;
    constexpr int PITCH = Tile::PITCH, NS = D / 32, NCB = D / 16;
    extern __shared__ __attribute__((aligned(16))) char h16_lds[];
    char *Ks = h16_lds, *Vs = h16_lds + Tile::BYTES;

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
            qop[s] = h16_scale_log2e<M>(h16_load_piece(static_cast<const char *>(a.q) + off + 64 * s, ok));
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

    H16Walk wk;
    wk.ri = a.goff[ho];
    wk.rend = a.goff[ho + 1];
    wk.pos = 0;
    wk.run = Run{0, 0, 0, 0};
    Tile bd;
    const unsigned ldbk = ldb * a.kps; // bytes between two columns of a virtual input latitude
    const bool piece_ok = 8 * (tid % Tile::CPR) < dr; // this thread's 16-byte piece of a staged row exists
    auto fetch = [&](const Run &rn, bool fresh) {
        const size_t lat_off = (size_t)key_row(a, rn.lat, rn.pad) * ldb;
        const int cs = wk.stage(fresh, rn.ws + wg0, a.Wi);
        if (fresh)
            bd.template fetch<FRESH, PAD>(kx + lat_off, vx + lat_off, tid, cs, a.Wi, ldbk, piece_ok);
        else
            bd.template fetch<HK, PAD>(kx + lat_off, vx + lat_off, tid, cs, a.Wi, ldbk, piece_ok);
    };
    wk.w = 1.f;
    if (wk.ri < wk.rend) {
        wk.run = a.gruns[wk.ri];
        wk.w = a.quad_w[wk.run.pad];
        fetch(wk.run, true);
        bd.template commit<FRESH>(Ks, Vs, tid, 0);
    }
    __syncthreads();
    settle(qop);
    settle(gop);
    float lse_ = lse;
    settle(lse_);

    while (wk.ri < wk.rend) {
        wk.plan(a.gruns, a.quad_w);
        if (wk.more) fetch(wk.nrun, wk.fresh);
        if (active) {
            const float lwl = fast_log2(wk.w) - lse_;
            const int len = wk.run.len, pos = wk.pos;
            const int xw = HQ * wave + pos; // band row of this wavefront's position `pos`
            const char *kblk[2] = {band_block<PITCH>(Ks, xw), band_block<PITCH>(Ks, xw + 16)};
            const char *vblk[2] = {band_block<PITCH>(Vs, xw), band_block<PITCH>(Vs, xw + 16)};
            // The accumulators start at log2 w - lse and at -I, so the matrix cores hand back the exponent of p and g - I.
            f4v sc[2], gc[2];
#pragma unroll
            for (int kb = 0; kb < 2; kb++) {
                sc[kb] = f4v{lwl, lwl, lwl, lwl};
                gc[kb] = f4v{-I, -I, -I, -I};
#pragma unroll
                for (int s = 0; s < NS; s++) {
                    sc[kb] = M::mfma(h16_read_row<PITCH>(kblk[kb], s, c, qd), qop[s], sc[kb]);
                    gc[kb] = M::mfma(h16_read_row<PITCH>(vblk[kb], s, c, qd), gop[s], gc[kb]);
                }
            }
            const int tb = pos + 4 * qd - c;
            if (pos >= HQ - 1 && pos + HK <= len) { // every element of the step is a neighbor: no band mask
#pragma unroll
                for (int kb = 0; kb < 2; kb++) {
#pragma unroll
                    for (int v = 0; v < 4; v++) gc[kb][v] = fast_exp2(sc[kb][v]) * gc[kb][v];
                }
            } else {
#pragma unroll
                for (int kb = 0; kb < 2; kb++) {
#pragma unroll
                    for (int v = 0; v < 4; v++) {
                        const unsigned t = (unsigned)(tb + 16 * kb + v);
                        const float p = (t < (unsigned)len) ? fast_exp2(sc[kb][v]) : 0.f;
                        gc[kb][v] = p * gc[kb][v];
                    }
                }
            }
            const uint4 dop = make_uint4(M::pack2(gc[0][0], gc[0][1]), M::pack2(gc[0][2], gc[0][3]), M::pack2(gc[1][0], gc[1][1]), M::pack2(gc[1][2], gc[1][3]));
#pragma unroll
            for (int cb = 0; cb < NCB; cb++) acc[cb] = M::mfma(h16_read_transposed<PITCH>(kblk[0], kblk[1], cb, c, qd), dop, acc[cb]);
        }
        if (wk.more) {
            if (wk.fresh) {
                __syncthreads(); // the next run's rows replace rows the slowest wavefront may still be reading
                bd.template commit<FRESH>(Ks, Vs, tid, 0);
            } else {
                bd.template commit<HK>(Ks, Vs, tid, FRESH - HK + wk.npos);
            }
        }
        __syncthreads();
        wk.advance();
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
template <typename T, int D, bool PAD> __global__ __launch_bounds__(64 * NW) void dkdv_h16_kernel(const Args a)
{
    typedef WgBand<D> Tile;
    typedef H16<T> M;
    constexpr int PITCH = Tile::PITCH, NS = D / 32, NCB = D / 16;
    extern __shared__ __attribute__((aligned(16))) char h16_lds[];
    char *Qs = h16_lds, *Gs = h16_lds + Tile::BYTES;
    constexpr int STAT = 2 * D; // the 32 bytes of padding of ring row 4 j of Qs hold (lse, I = <dy, y>) of the queries staged in rows 4 j .. 4 j + 3

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
            kop[s] = h16_scale_log2e<M>(h16_load_piece(static_cast<const char *>(a.k) + off + 64 * s, ok));
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

    H16Walk wk;
    wk.ri = a.soff[hi];
    wk.rend = a.soff[hi + 1];
    wk.pos = 0;
    wk.run = Run{0, 0, 0, 0};
    wk.w = 1.f;
    Tile bd;
    float2 st = make_float2(0.f, 0.f);
    const unsigned ldbq = ldb * a.qps; // bytes between two columns of a virtual output latitude
    const bool piece_ok = 8 * (tid % Tile::CPR) < dr; // this thread's 16-byte piece of a staged row exists
    auto fetch = [&](const Run &rn, bool fresh) {
        int c0 = 0;
        if (fresh) { // longitude of band row 0, in [0, 2 W)
            c0 = wg0 - rn.ws - rn.len + 1 + a.Wo;
            while (c0 < 0) c0 += a.Wo;
        }
        const int cs = wk.stage(fresh, c0, a.Wo);
        const size_t lat_off = (size_t)query_row(a, rn.lat, rn.pad) * ldb;
        if (fresh)
            bd.template fetch<FRESH, PAD>(qy + lat_off, gy + lat_off, tid, cs, a.Wo, ldbq, piece_ok);
        else
            bd.template fetch<HK, PAD>(qy + lat_off, gy + lat_off, tid, cs, a.Wo, ldbq, piece_ok);
        if (tid < (fresh ? FRESH : HK)) { // the first threads fetch the statistics of the staged rows
            int col = cs + tid;
            while (col >= a.Wo) col -= a.Wo;
            st = stats[(size_t)rn.lat * a.Wo + col];
        }
    };
    auto commit = [&](int x0) {
        if (x0 == 0)
            bd.template commit<FRESH>(Qs, Gs, tid, 0);
        else
            bd.template commit<HK>(Qs, Gs, tid, x0);
        if (tid < (x0 == 0 ? FRESH : HK)) *reinterpret_cast<float2 *>(Qs + ((x0 + tid) & (BR - 4)) * PITCH + STAT + 8 * (tid & 3)) = make_float2(lw - st.x, -st.y);
    };
    if (wk.ri < wk.rend) {
        wk.run = a.sruns[wk.ri];
        fetch(wk.run, true);
        commit(0);
    }
    __syncthreads();
    settle(kop);
    settle(vop);

    while (wk.ri < wk.rend) {
        wk.plan(a.sruns);
        if (wk.more) fetch(wk.nrun, wk.fresh);
        if (active) {
            const int len = wk.run.len, pos = wk.pos;
            const int xw = HQ * wave + pos; // band row of this wavefront's position `pos`
            const char *qblk[2] = {band_block<PITCH>(Qs, xw), band_block<PITCH>(Qs, xw + 16)};
            const char *gblk[2] = {band_block<PITCH>(Gs, xw), band_block<PITCH>(Gs, xw + 16)};
            // The accumulators start at the staged statistics (log2 w - lse of the query, -I of the query: written in that form at
            // commit), so the matrix cores hand back the exponent of p and g - I.
            f4v sc[2], gc[2];
#pragma unroll
            for (int qb = 0; qb < 2; qb++) {
                const float4 *sp = reinterpret_cast<const float4 *>(qblk[qb] + 4 * qd * PITCH + STAT);
                const float4 s01 = sp[0], s23 = sp[1];
                sc[qb] = f4v{s01.x, s01.z, s23.x, s23.z};
                gc[qb] = f4v{s01.y, s01.w, s23.y, s23.w};
#pragma unroll
                for (int s = 0; s < NS; s++) {
                    sc[qb] = M::mfma(h16_read_row<PITCH>(qblk[qb], s, c, qd), kop[s], sc[qb]);
                    gc[qb] = M::mfma(h16_read_row<PITCH>(gblk[qb], s, c, qd), vop[s], gc[qb]);
                }
            }
            const int tb = pos + 4 * qd - c; // r - c of element (qb, v): tb + 16 qb + v
            const bool inner = pos >= HQ - 1 && pos + HK <= len; // every element of the step is a (query, key) pair of the run
#pragma unroll
            for (int qb = 0; qb < 2; qb++) {
#pragma unroll
                for (int v = 0; v < 4; v++) {
                    float p = fast_exp2(sc[qb][v]);
                    if (!inner) p = ((unsigned)(tb + 16 * qb + v) < (unsigned)len) ? p : 0.f; // band mask, first and last steps of a run only
                    sc[qb][v] = p;
                    gc[qb][v] = p * gc[qb][v];
                }
            }
            const uint4 pop = make_uint4(M::pack2(sc[0][0], sc[0][1]), M::pack2(sc[0][2], sc[0][3]), M::pack2(sc[1][0], sc[1][1]), M::pack2(sc[1][2], sc[1][3]));
            const uint4 dop = make_uint4(M::pack2(gc[0][0], gc[0][1]), M::pack2(gc[0][2], gc[0][3]), M::pack2(gc[1][0], gc[1][1]), M::pack2(gc[1][2], gc[1][3]));
#pragma unroll
            for (int cb = 0; cb < NCB; cb++) {
                dvt[cb] = M::mfma(h16_read_transposed<PITCH>(gblk[0], gblk[1], cb, c, qd), pop, dvt[cb]);
                dkt[cb] = M::mfma(h16_read_transposed<PITCH>(qblk[0], qblk[1], cb, c, qd), dop, dkt[cb]);
            }
        }
        if (wk.more) {
            if (wk.fresh) __syncthreads(); // the next run's rows replace rows the slowest wavefront may still be reading
            commit(wk.fresh ? 0 : FRESH - HK + wk.npos);
        }
        __syncthreads();
        wk.advance();
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
