// Matrix-core kernels for fp32 storage and head dims 64 / 128: forward, dq and dk/dv with v_mfma_f32_16x16x4_f32.
// Included by s2attn_kernels.hip inside namespace s2 after s2attn_h16.hpp, whose tiling they share: one wavefront owns
// HQ = 16 consecutive longitudes of one latitude for one (batch, head) and walks every run of that latitude in steps of
// HK = 32 band positions; lane l = (c = l % 16, qd = l / 16); scores are produced transposed, S^T[position][column].
//
// Shape domain: ck == cv = dr, a multiple of 4 with dr <= D (the tile is D channels wide; channels from dr on are staged
// as zeros and never stored), at least 32 columns per virtual latitude, 16-byte aligned rows.
//
// Facts about the instruction:  A operand: the lane supplies A[i = c][k = qd];  B operand: B[k = qd][j = c];
// D: register v of the lane holds D[i = 4 qd + v][j = c].  The k index of a product is only a summation index, so each
// product numbers it the way that makes its operands cheap:
//   scores (K Q^T, V dY^T, ...): k slot qd of instruction s <-> channel qd * D/4 + s.  A lane's B operands are then a
//     contiguous quarter of its column's vector, loaded once with 16-byte loads and kept in registers, and its A operands
//     a contiguous quarter of a staged row (16-byte LDS reads, four instructions each);
//   second products (V^T P^T, K^T dS^T, ...): k slot qd of instruction (kb, v) <-> position 16 kb + 4 qd + v.  B is
//     register v of score block kb as it stands, A one float of the staged tile (lanes c read consecutive channels).

// Heads wider than 128 channels: NS = 2 wavefronts per workgroup, each owning a contiguous group of D = 128 channels (its own
// tiles, operands and output channels); the partial scores of the groups are added through LDS once per step, after which
// both wavefronts hold the same probabilities.  One wavefront cannot hold a 256-channel step in registers.

#define S2_M32_IDS(W_TILED, NROWS)                                            \
    const int lane = NS > 1 ? (int)(threadIdx.x & 63) : (int)threadIdx.x;     \
    const int wv = NS > 1 ? (int)(threadIdx.x >> 6) : 0;                      \
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
    const int nvalid = min(HQ, (W_TILED)-w0);                                 \
    const int drt = a.dk_;                 /* real head width */              \
    const int cbase = wv * D;              /* first channel of this wavefront's group */ \
    const int dr = min(D, drt - cbase);    /* real channels in the group */

extern __shared__ float4 m32_smem[];

// LDS of a workgroup: a static array when it is one wavefront (addresses are then compile-time constants), the dynamic
// allocation of the launch when it is more (two 128-channel wavefronts need more than the 64 KB a static array may have).
template <int BYTES, int NS> __device__ inline char *m32_lds()
{
    if constexpr (NS == 1) {
        __shared__ __attribute__((aligned(16))) char buf[BYTES];
        return buf;
    } else {
        return reinterpret_cast<char *>(m32_smem);
    }
}

// LDS bytes of a kernel of this family: per wavefront two tiles (+ two rows of statistics in the dk/dv pass), then the
// exchange area of 16 floats per lane and wavefront when there is more than one.
template <int D, int NS> constexpr int m32_wave_bytes(bool stats) { return 2 * HK * (4 * D + 16) + (stats ? 2 * HK * 4 : 0); }
template <int D, int NS> constexpr int m32_lds_bytes(bool stats) { return NS * m32_wave_bytes<D, NS>(stats) + (NS > 1 ? NS * 64 * 16 * 4 : 0); }

// Replaces this wavefront's partial blocks by the sum over all wavefronts: x0 (and x1 when given) hold 8 floats per lane each.
template <int NS> __device__ inline void m32_exchange(float *xs, int wv, int lane, f4v (&x0)[2], f4v (*x1)[2])
{
    if constexpr (NS > 1) {
        float4 *mine = reinterpret_cast<float4 *>(xs + (wv * 64 + lane) * 16);
        mine[0] = make_float4(x0[0][0], x0[0][1], x0[0][2], x0[0][3]);
        mine[1] = make_float4(x0[1][0], x0[1][1], x0[1][2], x0[1][3]);
        if (x1) {
            mine[2] = make_float4((*x1)[0][0], (*x1)[0][1], (*x1)[0][2], (*x1)[0][3]);
            mine[3] = make_float4((*x1)[1][0], (*x1)[1][1], (*x1)[1][2], (*x1)[1][3]);
        }
        __syncthreads();
        // every wavefront adds the blocks in the same order (its own included), so all of them hold bit-identical sums
        x0[0] = x0[1] = f4v{0.f, 0.f, 0.f, 0.f};
        if (x1) (*x1)[0] = (*x1)[1] = f4v{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int o = 0; o < NS; o++) {
            const float4 *part = reinterpret_cast<const float4 *>(xs + (o * 64 + lane) * 16);
            const float4 a0 = part[0], a1 = part[1];
            x0[0] += f4v{a0.x, a0.y, a0.z, a0.w};
            x0[1] += f4v{a1.x, a1.y, a1.z, a1.w};
            if (x1) {
                const float4 b0 = part[2], b1 = part[3];
                (*x1)[0] += f4v{b0.x, b0.y, b0.z, b0.w};
                (*x1)[1] += f4v{b1.x, b1.y, b1.z, b1.w};
            }
        }
    }
}

// fp32 tile of D channels.  With a row pitch of 16 bytes modulo 128 the four-byte reads of the second products (two
// rows 4 apart per 32 lanes, 16 consecutive floats each) fall in distinct banks.
template <int D> struct FTile : BandTile<D / 4, 4 * D + 16> {};

__device__ inline f4v m32_mfma(float a, float b, f4v c) { return __builtin_amdgcn_mfma_f32_16x16x4f32(a, b, c, 0, 0, 0); }

// Both 16 x 16 blocks of transposed scores of a step: rows = staged rows 16 kb + c, summed over the D channels in four
// independent accumulation chains per block (smaller partial sums round less, and consecutive instructions do not depend
// on each other).  The LDS reads run LA pieces ahead of the instructions that consume them; the scheduling barriers keep
// the compiler from folding each read back next to its use, which would expose the LDS latency once per four instructions.
template <int D, int PITCH> __device__ inline void m32_scores(f4v (&sc)[2], const char *tile, int c, int qd, const float (&op)[D / 4])
{
    constexpr int NP = D / 16, NF = 2 * NP, LA = NF < 4 ? NF : 4;
    const char *row = tile + c * PITCH + qd * D; // this lane's quarter of staged row c: D/4 floats = D bytes
    float4 x[NF];
    f4v s[2][4];
#pragma unroll
    for (int kb = 0; kb < 2; kb++)
#pragma unroll
        for (int j = 0; j < 4; j++) s[kb][j] = f4v{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int i = 0; i < LA; i++) x[i] = *reinterpret_cast<const float4 *>(row + (i / NP) * 16 * PITCH + 16 * (i % NP));
#pragma unroll
    for (int i = 0; i < NF; i++) {
        if (i + LA < NF) x[i + LA] = *reinterpret_cast<const float4 *>(row + ((i + LA) / NP) * 16 * PITCH + 16 * ((i + LA) % NP));
        __builtin_amdgcn_sched_barrier(0);
        const int kb = i / NP, p = i % NP;
        s[kb][0] = m32_mfma(x[i].x, op[4 * p + 0], s[kb][0]);
        s[kb][1] = m32_mfma(x[i].y, op[4 * p + 1], s[kb][1]);
        s[kb][2] = m32_mfma(x[i].z, op[4 * p + 2], s[kb][2]);
        s[kb][3] = m32_mfma(x[i].w, op[4 * p + 3], s[kb][3]);
        __builtin_amdgcn_sched_barrier(0);
    }
#pragma unroll
    for (int kb = 0; kb < 2; kb++) sc[kb] = (s[kb][0] + s[kb][1]) + (s[kb][2] + s[kb][3]);
}

// acc[cb] (channels 16 cb + 4 qd + v of column c) += sum over the 32 staged rows of tile[row][channel] * coef[row][c].
// The eight rows of this lane (kb, v) are taken two at a time; the operands of the next two pairs are in flight while
// one pair is consumed.
template <int D, int PITCH> __device__ inline void m32_accumulate(f4v (&acc)[D / 16], const char *tile, int c, int qd, const f4v (&coef)[2])
{
    constexpr int NCB = D / 16;
    float av[4][2][NCB];
    const char *base = tile + (4 * qd) * PITCH + 4 * c;
    auto load = [&](int g) { // rows (kb = g / 2, v = 2 (g % 2) + r), r < 2
#pragma unroll
        for (int r = 0; r < 2; r++)
#pragma unroll
            for (int cb = 0; cb < NCB; cb++) av[g][r][cb] = *reinterpret_cast<const float *>(base + (16 * (g / 2) + 2 * (g % 2) + r) * PITCH + 64 * cb);
    };
    load(0);
    load(1);
#pragma unroll
    for (int g = 0; g < 4; g++) {
        if (g + 2 < 4) load(g + 2);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int r = 0; r < 2; r++)
#pragma unroll
            for (int cb = 0; cb < NCB; cb++) acc[cb] = m32_mfma(av[g][r][cb], coef[g / 2][2 * (g % 2) + r], acc[cb]);
        __builtin_amdgcn_sched_barrier(0);
    }
}

// this lane's quarter (channels qd * D/4 ..) of one grid point's vector of dr channels of storage type T; zeros from channel dr on
template <int D, typename T = float> __device__ inline void m32_load_quarter(float (&op)[D / 4], const char *vec, int qd, int dr)
{
#pragma unroll
    for (int i = 0; i < D / 16; i++) {
        float4 x = make_float4(0.f, 0.f, 0.f, 0.f);
        if (qd * (D / 4) + 4 * i < dr) x = load4(reinterpret_cast<const T *>(vec) + qd * (D / 4) + 4 * i);
        op[4 * i + 0] = x.x;
        op[4 * i + 1] = x.y;
        op[4 * i + 2] = x.z;
        op[4 * i + 3] = x.w;
    }
}

// four consecutive channels of storage type T, widened: one 16-byte piece of an fp32 tile row
template <typename T> __device__ inline u4v m32_piece(const char *p)
{
    const float4 x = load4(reinterpret_cast<const T *>(p));
    return u4v{__float_as_uint(x.x), __float_as_uint(x.y), __float_as_uint(x.z), __float_as_uint(x.w)};
}

// ---- forward ---------------------------------------------------------------------------------------------------
template <int D, int NS> __global__ __launch_bounds__(64 * NS) void fwd_m32_kernel(const Args a)
{
    typedef FTile<D> Tile;
    constexpr int PITCH = Tile::PITCH, NCB = D / 16;
    S2_M32_IDS(a.Wo, a.Ho)
    char *lds = m32_lds<m32_lds_bytes<D, NS>(false), NS>();
    char *Ks = lds + wv * m32_wave_bytes<D, NS>(false), *Vs = Ks + HK * PITCH;
    float *xs = reinterpret_cast<float *>(lds + NS * m32_wave_bytes<D, NS>(false));
    const int ho = a.gorder[a.row_first + rowsel];
    const unsigned ldb = a.nh * drt * 4; // bytes between two grid points
    const char *kx = static_cast<const char *>(a.k) + ((size_t)b * a.Hi * a.Wi * a.nh + h) * (drt * 4) + cbase * 4;
    const char *vx = static_cast<const char *>(a.v) + ((size_t)b * a.Hi * a.Wi * a.nh + h) * (drt * 4) + cbase * 4;
    const bool mine = c < nvalid;
    const size_t pt = (size_t)query_point(a, b, ho, ho / a.qps) + (size_t)(w0 + (mine ? c : 0)) * a.qps;

    float qop[D / 4];
    m32_load_quarter<D>(qop, static_cast<const char *>(a.q) + pt * ldb + (size_t)h * (drt * 4) + cbase * 4, qd, dr);
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
    const bool piece_ok = 4 * (lane % Tile::CPR) < dr; // this lane's 16-byte piece of a staged row exists
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
        m32_scores<D, PITCH>(sc, Ks, c, qd, qop);
        m32_exchange<NS>(xs, wv, lane, sc, nullptr);
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
        m32_accumulate<D, PITCH>(acc, Vs, c, qd, sc);

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
        if (a.lse && qd == 0 && wv == 0) a.lse[((size_t)bh * a.Ho + ho) * a.Wo + w0 + c] = m + fast_log2(S);
        const float inv = 1.0f / S;
        char *y = static_cast<char *>(a.y) + pt * ldb + (size_t)h * (drt * 4) + cbase * 4 + 16 * qd;
#pragma unroll
        for (int cb = 0; cb < NCB; cb++)
            if (16 * cb + 4 * qd < dr)
                *reinterpret_cast<float4 *>(y + 64 * cb) = make_float4(acc[cb][0] * inv, acc[cb][1] * inv, acc[cb][2] * inv, acc[cb][3] * inv);
    }
}

// ---- backward, dq pass (needs the forward's y and lse) -------------------------------------------------------------
// Three products per step:  S^T = K Q^T,  G^T = V dY^T,  dQ^T += K^T dS^T  with dS = P o (G - I),  I = <dy, y>.
template <int D, int NS> __global__ __launch_bounds__(64 * NS) void dq_m32_kernel(const Args a)
{
    typedef FTile<D> Tile;
    constexpr int PITCH = Tile::PITCH, NCB = D / 16;
    S2_M32_IDS(a.Wo, a.Ho)
    char *lds = m32_lds<m32_lds_bytes<D, NS>(false), NS>();
    char *Ks = lds + wv * m32_wave_bytes<D, NS>(false), *Vs = Ks + HK * PITCH;
    float *xs = reinterpret_cast<float *>(lds + NS * m32_wave_bytes<D, NS>(false));
    const int ho = a.gorder[a.row_first + rowsel];
    const unsigned ldb = a.nh * drt * 4;
    const char *kx = static_cast<const char *>(a.k) + ((size_t)b * a.Hi * a.Wi * a.nh + h) * (drt * 4) + cbase * 4;
    const char *vx = static_cast<const char *>(a.v) + ((size_t)b * a.Hi * a.Wi * a.nh + h) * (drt * 4) + cbase * 4;
    const bool mine = c < nvalid;
    const size_t pt = (size_t)query_point(a, b, ho, ho / a.qps) + (size_t)(w0 + (mine ? c : 0)) * a.qps;
    const size_t sidx = ((size_t)bh * a.Ho + ho) * a.Wo + w0 + (mine ? c : 0);

    float qop[D / 4], gop[D / 4];
    float I = 0.f;
    {
        const size_t off = pt * ldb + (size_t)h * (drt * 4) + cbase * 4;
        m32_load_quarter<D>(qop, static_cast<const char *>(a.q) + off, qd, dr);
        m32_load_quarter<D>(gop, static_cast<const char *>(a.dy) + off, qd, dr);
        float yq[D / 4];
        m32_load_quarter<D>(yq, static_cast<const char *>(a.ysaved) + off, qd, dr);
#pragma unroll
        for (int i = 0; i < D / 4; i++) I = fmaf(gop[i], yq[i], I);
    }
    I = h16_quarter_sum(I);
    if constexpr (NS > 1) { // <dy, y> over all channel groups
        xs[wv * 64 + lane] = I;
        __syncthreads();
        float t = 0.f;
#pragma unroll
        for (int o = 0; o < NS; o++) t += xs[o * 64 + lane];
        I = t;
        __syncthreads();
    }
    const float lse = a.lse[sidx];

    f4v acc[NCB];
#pragma unroll
    for (int cb = 0; cb < NCB; cb++) acc[cb] = f4v{0.f, 0.f, 0.f, 0.f};

    int ri = a.goff[ho];
    const int rend = a.goff[ho + 1];
    int pos = 0;
    Run run = {0, 0, 0, 0};
    Tile kt, vt;
    const unsigned ldbk = ldb * a.kps;
    const unsigned lane_off = (unsigned)(lane / Tile::CPR) * ldbk + 16u * (lane % Tile::CPR);
    const bool piece_ok = 4 * (lane % Tile::CPR) < dr; // this lane's 16-byte piece of a staged row exists
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
        m32_scores<D, PITCH>(sc, Ks, c, qd, qop);
        m32_scores<D, PITCH>(gc, Vs, c, qd, gop);
        m32_exchange<NS>(xs, wv, lane, sc, &gc);
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
        m32_accumulate<D, PITCH>(acc, Ks, c, qd, gc);

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
    if (mine && qd == 0 && wv == 0) a.stats[sidx] = make_float2(lse, I);
    if (mine) {
        char *dq = static_cast<char *>(a.dq) + pt * ldb + (size_t)h * (drt * 4) + cbase * 4 + 16 * qd;
#pragma unroll
        for (int cb = 0; cb < NCB; cb++)
            if (16 * cb + 4 * qd < dr) *reinterpret_cast<float4 *>(dq + 64 * cb) = make_float4(acc[cb][0], acc[cb][1], acc[cb][2], acc[cb][3]);
    }
}

// ---- backward, dk/dv pass: transposed gather ---------------------------------------------------------------------
// The wavefront owns 16 INPUT longitudes (column c = key) and walks the runs grouped by input latitude; staged rows
// are queries.  Staged row r of a run (first row = longitude w0 - ws - len + 1) sees key c iff 0 <= r - c < len.
// Four products per step:  S = Q K^T,  G = dY V^T  (rows = queries, columns = keys),  dV^T += dY^T P,  dK^T += Q^T dS.
template <int D, int NS> __global__ __launch_bounds__(64 * NS) void dkdv_m32_kernel(const Args a)
{
    typedef FTile<D> Tile;
    constexpr int PITCH = Tile::PITCH, NCB = D / 16;
    S2_M32_IDS(a.Wi, a.Hi)
    char *lds = m32_lds<m32_lds_bytes<D, NS>(true), NS>();
    char *Qs = lds + wv * m32_wave_bytes<D, NS>(true), *Gs = Qs + HK * PITCH;
    float *Ls = reinterpret_cast<float *>(Gs + HK * PITCH), *Is = Ls + HK;
    float *xs = reinterpret_cast<float *>(lds + NS * m32_wave_bytes<D, NS>(true));
    const int hi = a.sorder[a.row_first + rowsel];
    const unsigned ldb = a.nh * drt * 4;
    const char *qy = static_cast<const char *>(a.q) + ((size_t)b * a.Ho * a.Wo * a.nh + h) * (drt * 4) + cbase * 4;
    const char *gy = static_cast<const char *>(a.dy) + ((size_t)b * a.Ho * a.Wo * a.nh + h) * (drt * 4) + cbase * 4;
    const float2 *stats = a.stats + (size_t)bh * a.Ho * a.Wo;
    const bool mine = c < nvalid;
    const size_t pt = (size_t)key_point(a, b, hi, hi / a.kps) + (size_t)(w0 + (mine ? c : 0)) * a.kps;

    float kop[D / 4], vop[D / 4]; // this lane's quarter of key c
    {
        const size_t off = pt * ldb + (size_t)h * (drt * 4) + cbase * 4;
        m32_load_quarter<D>(kop, static_cast<const char *>(a.k) + off, qd, dr);
        m32_load_quarter<D>(vop, static_cast<const char *>(a.v) + off, qd, dr);
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
    const bool piece_ok = 4 * (lane % Tile::CPR) < dr; // this lane's 16-byte piece of a staged row exists
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
        m32_scores<D, PITCH>(sc, Qs, c, qd, kop);
        m32_scores<D, PITCH>(gc, Gs, c, qd, vop);
        m32_exchange<NS>(xs, wv, lane, sc, &gc);
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
        m32_accumulate<D, PITCH>(dvt, Gs, c, qd, sc);
        m32_accumulate<D, PITCH>(dkt, Qs, c, qd, gc);

        __syncthreads();
        if (more) commit();
        __syncthreads();
        ri = nri;
        pos = npos;
        run = nrun;
    }

    if (mine) {
        const size_t off = pt * ldb + (size_t)h * (drt * 4) + cbase * 4 + 16 * qd;
        char *dk = static_cast<char *>(a.dk) + off, *dv = static_cast<char *>(a.dv) + off;
#pragma unroll
        for (int cb = 0; cb < NCB; cb++) {
            if (16 * cb + 4 * qd < dr) {
                *reinterpret_cast<float4 *>(dk + 64 * cb) = make_float4(dkt[cb][0], dkt[cb][1], dkt[cb][2], dkt[cb][3]);
                *reinterpret_cast<float4 *>(dv + 64 * cb) = make_float4(dvt[cb][0], dvt[cb][1], dvt[cb][2], dvt[cb][3]);
            }
        }
    }
}

// ---- forward, one ring step --------------------------------------------------------------------------------------
// The forward above for ONE longitude chunk of K/V (input latitudes r_lat0 .. + r_nlat, real input longitudes
// r_lon_lo .. + r_nkx; k, v = [batch, r_nlat, r_nkx, channels]) that continues a running softmax kept by the caller in the
// reference's form: y_acc = sum_j alpha_j v_j, alpha_sum = sum_j alpha_j, qdotk_max = max_j q.k_j (natural units) with
// alpha_j = exp(q.k_j - qdotk_max) w_j over the neighbors seen so far.  A row of the staged band is one input longitude, so
// the chunk clips ROWS of the band, not queries: the band positions u of a run whose longitude (ws + w0 + u) mod W lies in
// the chunk are up to three intervals, and the walk visits only the 32-position steps inside them (a chunk of a quarter of
// the circle costs a polar tile a quarter of its steps, an equatorial tile one step per run in the one or two chunks its
// neighborhood touches).  Tiles without any such step leave the state untouched.
// k, v, q, dy have storage type T (fp32, bf16 or fp16: 16-bit rows are widened when they are fetched, so the staged tiles,
// the matrix instructions and the caller's state are fp32 whatever the storage); dk, dv of pass 2 are fp32.
constexpr float NEG_BIG_NAT = -1.0e38f; // "no neighbor yet" for a maximum in natural units (times log2 e stays finite)

struct RingWalk {
    const Run *runs;
    const float *weights;
    int ri, rend;
    int W, kps, w0, lon_lo, nkx, lat0, nlat, wlat0; // wlat0: quadrature weight of the run's latitude Run::pad is weights[pad + wlat0]
    // the run the walk stands in
    Run run;
    float w;
    int rl, par, vlo, nv, u0, L, m;
    // the step: band positions pos .. pos + HK of the interval [ua, ub); vca = virtual column of position ua
    int pos, ua, ub, vca;
    bool valid;
    __device__ inline void start(const Run *runs_, const float *weights_, int first, int rend_)
    {
        runs = runs_, weights = weights_, ri = first - 1, rend = rend_, m = 1, valid = false;
    }
    __device__ inline bool advance()
    {
        if (valid && pos + HK < ub) {
            pos += HK;
            return true;
        }
        for (;;) {
            m++;
            if (m > 1) { // next run
                ri++;
                if (ri >= rend) return valid = false;
                run = uniform_load(runs + ri);
                rl = run.pad - lat0; // row of the chunk
                m = 1;               // (skip the run unless the chunk holds part of it)
                if (rl < 0 || rl >= nlat) continue;
                par = 0, vlo = lon_lo, nv = nkx;
                if (kps > 1) {
                    par = run.lat - run.pad * kps; // column class: virtual column vc is real longitude vc * kps + par
                    vlo = (lon_lo - par + kps - 1) / kps;
                    nv = (lon_lo + nkx - par + kps - 1) / kps - vlo; // virtual columns vlo .. vlo + nv are in the chunk
                    if (nv <= 0) continue;
                }
                w = uniform_load(weights + (run.pad + wlat0));
                L = run.len + HQ - 1;
                u0 = vlo - run.ws - w0; // in (-2 W, W)
                u0 += (u0 < 0) ? W : 0;
                u0 += (u0 < 0) ? W : 0; // first band position at virtual column vlo
                m = -2;
                continue;
            }
            const int a0 = u0 + m * W;
            const int a_ = a0 < 0 ? 0 : a0, b_ = a0 + nv > L ? L : a0 + nv;
            if (a_ >= b_) continue;
            ua = pos = a_, ub = b_, vca = vlo + (a_ - a0);
            return valid = true;
        }
    }
};

// MODE 0: the forward step (state y_acc, alpha_sum, qdotk_max).  MODE 1: pass 1 of the backward in the gather direction,
// which walks the same steps and re-accumulates alpha_sum and qdotk_max (the same operations in the same order as the
// forward step: the two sums are bit-identical) together with integral = sum_j alpha_j <dy, v_j>, alpha_k = sum_j alpha_j k_j
// and alpha_kvw = sum_j alpha_j <dy, v_j> k_j: a second score product G^T = V dY^T and two accumulations against K^T.
// MODE 2: pass 1 of the up-sampling direction, which is handed the forward's FINAL qdotk_max and adds the same three sums
// relative to it (no running maximum, no alpha_sum).
// Both directions: in the up-sampling direction (r_qps = nlon_out / nlon_in > 1) the plan's output latitudes are virtual
// (real latitude * r_qps + column class), a tile's queries are the local output columns (w0 + c) * r_qps + class, input
// latitudes are rows of the chunk as they stand and r_wlat0 turns them into quadrature-weight indices.
template <int D, int MODE, typename T> __global__ __launch_bounds__(64, (D <= 32 && MODE == 0) ? 4 : (D <= 32 ? 3 : (D <= 64 && MODE == 0 ? 2 : 1))) void ring_m32_kernel(const Args a)
{
    constexpr int NS = 1;
    constexpr bool PASS1 = MODE != 0, FIXED = MODE == 2;
    typedef FTile<D> Tile;
    constexpr int PITCH = Tile::PITCH, NCB = D / 16;
    S2_M32_IDS(a.Wo, a.Ho)
    (void)h; // heads are folded into the batch
    (void)nvalid;
    char *lds = m32_lds<m32_lds_bytes<D, 1>(false), 1>();
    char *Ks = lds, *Vs = Ks + HK * PITCH;
    const int ho = a.gorder[a.row_first + rowsel]; // (virtual) output latitude
    const int hor = ho / a.r_qps, parq = ho - hor * a.r_qps;
    const int nval = min(HQ, (a.r_wo - parq + a.r_qps - 1) / a.r_qps - w0); // queries of the tile inside the local window
    if (nval <= 0) return;
    const unsigned ldb = drt * sizeof(T); // bytes between two grid points
    const char *kx = static_cast<const char *>(a.k) + (size_t)b * a.r_nlat * a.r_nkx * ldb;
    const char *vx = static_cast<const char *>(a.v) + (size_t)b * a.r_nlat * a.r_nkx * ldb;
    const bool mine = c < nval;
    const size_t pt = ((size_t)b * (a.Ho / a.r_qps) + hor) * a.r_wo + (size_t)(w0 + (mine ? c : 0)) * a.r_qps + parq;

    { // the arc of columns this tile's queries can see, against the virtual columns that can lie in the chunk: most tiles of
      // an equatorial latitude leave here, without reading a run
        typedef int i2v __attribute__((ext_vector_type(2)));
        const i2v span = uniform_load(reinterpret_cast<const i2v *>(a.gspan) + ho);
        const int la = span[1] + HQ - 1, b0 = a.r_lon_lo / a.kps, lb = (a.r_lon_lo + a.r_nkx - 1) / a.kps + 1 - b0;
        if (span[1] <= 0) return;
        if (la < a.Wi && lb < a.Wi) {
            int dab = (b0 - (w0 + span[0])) % a.Wi; // chunk start relative to the arc's start
            dab += dab < 0 ? a.Wi : 0;
            if (dab >= la && a.Wi - dab >= lb) return;
        }
    }
    RingWalk wk;
    wk.W = a.Wi, wk.kps = a.kps, wk.w0 = w0, wk.lon_lo = a.r_lon_lo, wk.nkx = a.r_nkx, wk.lat0 = a.r_lat0, wk.nlat = a.r_nlat, wk.wlat0 = a.r_wlat0;
    wk.start(a.gruns, a.quad_w, a.goff[ho], a.goff[ho + 1]);
    if (!wk.advance()) return; // nothing of this tile's neighborhood is in the chunk

    float qop[D / 4], gop[PASS1 ? D / 4 : 1];
    m32_load_quarter<D, T>(qop, static_cast<const char *>(a.q) + pt * ldb, qd, dr);
    if constexpr (PASS1) m32_load_quarter<D, T>(gop, static_cast<const char *>(a.dy) + pt * ldb, qd, dr);
    // forward: Y^T; pass 1: alpha_k^T (acc) and alpha_kvw^T (acc2): register v of block cb is channel 16 cb + 4 qd + v of column c
    float *const acc_state = PASS1 ? a.r_ak : a.r_yacc;
    f4v acc[NCB], acc2[PASS1 ? NCB : 1];
#pragma unroll
    for (int cb = 0; cb < NCB; cb++) {
        float4 x = make_float4(0.f, 0.f, 0.f, 0.f), x2 = x;
        if (16 * cb + 4 * qd < dr) {
            x = *reinterpret_cast<const float4 *>(acc_state + pt * drt + 16 * cb + 4 * qd);
            if constexpr (PASS1) x2 = *reinterpret_cast<const float4 *>(a.r_akvw + pt * drt + 16 * cb + 4 * qd);
        }
        acc[cb] = f4v{x.x, x.y, x.z, x.w};
        if constexpr (PASS1) acc2[cb] = f4v{x2.x, x2.y, x2.z, x2.w};
    }
    // The exponentials are taken relative to a reference point m that is moved lazily (when a column's maximum has grown by
    // more than RESCALE_THR binary orders: after a tile's first steps that is rare, and a step then needs neither an exchange
    // between the four lanes of a column nor a rescaling); the exact maximum the state asks for is kept per lane (mtrue)
    // and the sums are brought to it once, at the end.
    float m = fmaxf(a.r_qmax[pt], NEG_BIG_NAT), mtrue = -INFINITY;
    float S = 0.f, I = 0.f; // the four lanes of a column each keep a share of the sums
    if constexpr (!FIXED) S = qd == 0 ? a.r_asum[pt] : 0.f;
    if constexpr (PASS1) I = qd == 0 ? a.r_integral[pt] : 0.f;

    Tile kt, vt;
    const int r0 = lane / Tile::CPR;
    const unsigned pc = 4u * sizeof(T) * (lane % Tile::CPR);
    const bool piece_ok = 4 * (lane % Tile::CPR) < dr; // this lane's four channels of a staged row exist
    const unsigned colb = ldb * a.kps;                 // bytes between two virtual columns
    auto fetch = [&]() { // the rows of the step the walk stands at; rows beyond the interval are staged as zeros
        const size_t base = ((size_t)wk.rl * a.r_nkx + (size_t)((wk.vca + wk.pos - wk.ua) * a.kps + wk.par - a.r_lon_lo)) * ldb + pc;
        const int nrows = wk.ub - wk.pos;
#pragma unroll
        for (int it = 0; it < Tile::NIT; it++) {
            const int row = r0 + it * Tile::RPI;
            kt.raw[it] = u4v{0u, 0u, 0u, 0u};
            vt.raw[it] = u4v{0u, 0u, 0u, 0u};
            if (row < nrows && piece_ok) {
                kt.raw[it] = m32_piece<T>(kx + base + (size_t)row * colb);
                vt.raw[it] = m32_piece<T>(vx + base + (size_t)row * colb);
            }
        }
    };
    fetch();
    kt.commit(Ks, lane);
    vt.commit(Vs, lane);
    __syncthreads();
    settle(qop);
    if constexpr (PASS1) settle(gop);

    for (;;) {
        const float lw = fast_log2(wk.w);
        const int len = wk.run.len, pos = wk.pos, ub = wk.ub;
        const bool more = wk.advance();
        if (more) fetch();

        f4v sc[2], gc[2];
        m32_scores<D, PITCH>(sc, Ks, c, qd, qop);
        if constexpr (PASS1) m32_scores<D, PITCH>(gc, Vs, c, qd, gop);
        // element (kb, v) is band position u = pos + 16 kb + 4 qd + v and neighbor t = u - c of column c: it counts iff
        // 0 <= t < len and u < ub, i.e. t < min(len, ub - c) as unsigned numbers
        const int tb = pos + 4 * qd - c;
        const unsigned lim = (unsigned)max(0, min(len, ub - c));
        float mx = -INFINITY;
        if (pos >= HQ - 1 && pos + HK <= min(len, ub)) { // every element of the step counts
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
                    sc[kb][v] = (t < lim) ? sc[kb][v] : -INFINITY;
                    mx = fmaxf(mx, sc[kb][v]);
                }
            }
        }
        if constexpr (!FIXED) mtrue = fmaxf(mtrue, mx);
        constexpr float THR = RESCALE_THR * 0.69314718f; // natural units
        if (!FIXED && __any(mx > m + THR)) {
            const float cm = h16_quarter_max(mx);
            const float mn = cm > m + THR ? cm : m; // m is finite, so mn is
            const float corr = fast_exp2((m - mn) * LOG2E);
            S *= corr;
#pragma unroll
            for (int cb = 0; cb < NCB; cb++) acc[cb] *= corr;
            if constexpr (PASS1) {
                I *= corr;
#pragma unroll
                for (int cb = 0; cb < NCB; cb++) acc2[cb] *= corr;
            }
            m = mn;
        }
        const float sh = fmaf(-m, LOG2E, lw);
#pragma unroll
        for (int kb = 0; kb < 2; kb++) {
#pragma unroll
            for (int v = 0; v < 4; v++) {
                const float p = fast_exp2(fmaf(sc[kb][v], LOG2E, sh)); // = exp(q.k - m) w; not counted: exp2(-inf) = 0
                sc[kb][v] = p;
                S += p;
                if constexpr (PASS1) {
                    gc[kb][v] *= p; // rows outside the chunk are staged as zeros, so <dy, v> is finite wherever p = 0
                    I += gc[kb][v];
                }
            }
        }
        if constexpr (PASS1) {
            m32_accumulate<D, PITCH>(acc, Ks, c, qd, sc);
            m32_accumulate<D, PITCH>(acc2, Ks, c, qd, gc);
        } else {
            m32_accumulate<D, PITCH>(acc, Vs, c, qd, sc);
        }

        __syncthreads();
        if (!more) break;
        kt.commit(Ks, lane);
        vt.commit(Vs, lane);
        __syncthreads();
    }

    S = h16_quarter_sum(S);
    if constexpr (PASS1) I = h16_quarter_sum(I);
    float f = 1.f;
    if constexpr (!FIXED) {
        mtrue = fmaxf(h16_quarter_max(mtrue), a.r_qmax[pt]); // the maximum over everything this column has seen, earlier chunks included (read again: a register less in the loop)
        f = mtrue > -INFINITY ? fast_exp2((m - mtrue) * LOG2E) : 1.f; // m <= mtrue <= m + THR; a column without neighbors keeps its zeros
    }
    if (mine) {
        if (qd == 0) {
            if constexpr (!FIXED) {
                a.r_asum[pt] = S * f;
                a.r_qmax[pt] = mtrue;
            }
            if constexpr (PASS1) a.r_integral[pt] = I * f;
        }
#pragma unroll
        for (int cb = 0; cb < NCB; cb++) {
            if (16 * cb + 4 * qd < dr) {
                *reinterpret_cast<float4 *>(acc_state + pt * drt + 16 * cb + 4 * qd) = make_float4(acc[cb][0] * f, acc[cb][1] * f, acc[cb][2] * f, acc[cb][3] * f);
                if constexpr (PASS1)
                    *reinterpret_cast<float4 *>(a.r_akvw + pt * drt + 16 * cb + 4 * qd) = make_float4(acc2[cb][0] * f, acc2[cb][1] * f, acc2[cb][2] * f, acc2[cb][3] * f);
            }
        }
    }
}

// The walk of pass 2 over the scatter runs of one (virtual) input latitude: staged rows are queries, and only the band
// positions whose query column lies in the local window are visited (the window is the whole circle on one device, a sector
// of it in a longitude-sharded layer, where most positions of a polar run fall outside).  Band position u of run (ws, len)
// of a tile at key column w0 is (virtual) query column (w0 - ws - len + 1 + u) mod W; the window holds the virtual
// columns 0 .. nv of the run's column class.
struct RingWalk2 {
    const Run *runs;
    int ri, rend, W, w0, qps, wo;
    Run run;
    int parq, nv, c0, u0, L, m;
    int pos, ua, ub, col; // the step: positions pos .. pos + HK of [ua, ub); col = query column of position pos (no wrap inside an interval)
    bool valid;
    __device__ inline void start(const Run *runs_, int first, int rend_) { runs = runs_, ri = first - 1, rend = rend_, m = 1, valid = false; }
    __device__ inline bool advance()
    {
        if (valid && pos + HK < ub) {
            pos += HK;
            col += HK;
            col -= (col >= W) ? W : 0; // (the whole-circle interval; W >= HK)
            return true;
        }
        for (;;) {
            m++;
            if (m > 1) { // next run
                ri++;
                if (ri >= rend) return valid = false;
                run = uniform_load(runs + ri);
                m = 1;
                parq = run.lat - run.pad * qps;
                nv = (wo - parq + qps - 1) / qps; // virtual columns of this class inside the window
                if (nv <= 0) continue;
                L = run.len + HQ - 1;
                c0 = w0 - run.ws - run.len + 1; // in (-2 W, W): query column of position 0
                c0 += (c0 < 0) ? W : 0;
                c0 += (c0 < 0) ? W : 0;
                if (nv >= W) { // the whole circle is local: one interval
                    ua = pos = 0, ub = L, col = c0;
                    m = 2;
                    return valid = true;
                }
                u0 = c0 == 0 ? 0 : W - c0; // first position at column 0
                m = -2;
                continue;
            }
            const int a0 = u0 + m * W;
            const int a_ = a0 < 0 ? 0 : a0, b_ = a0 + nv > L ? L : a0 + nv;
            if (a_ >= b_) continue;
            ua = pos = a_, ub = b_, col = a_ - a0;
            return valid = true;
        }
    }
};

// ---- backward, pass 2 of a ring step ---------------------------------------------------------------------------------
// The dk/dv pass above for the keys of ONE chunk: a wavefront owns 16 consecutive virtual columns of one column class of a
// chunk latitude (real longitudes (w0 + c) * kps + par) and walks the scatter runs of that virtual latitude; staged rows are
// local queries with their statistics (alpha_sum, qdotk_max, integral_norm of the caller, natural units) - a row whose query
// column lies outside the local window of Wo longitudes is staged as zeros and weighs nothing.  dk, dv (fp32, shaped like
// the chunk) are ADDED to; every key belongs to one wavefront, so plainly.
// WRITE = false (gather direction): dk, dv are added to.  WRITE = true (up-sampling direction: r_qps > 1, the plan's output
// latitudes are virtual, a staged row of virtual column j is the local query column j * r_qps + class): every element of
// the chunk's dk, dv is written, zeros where no query sees the key.
template <int D, bool WRITE, typename T> __global__ __launch_bounds__(64) void ring_pass2_m32_kernel(const Args a)
{
    typedef FTile<D> Tile;
    constexpr int PITCH = Tile::PITCH, NCB = D / 16;
    const int lane = threadIdx.x, c = lane & 15, qd = lane >> 4;
    const int drt = a.dk_, dr = min(D, drt);
    // workgroup -> (batch, virtual input latitude in the plan's order, tile of 16 virtual columns of the chunk)
    const int ntile = (a.r_nkx / a.kps + 1 + HQ - 1) / HQ + 1; // enough for every column class and any alignment of the chunk
    int id = blockIdx.x;
    const int b = id % a.B;
    id /= a.B;
    const int hv = a.sorder[id / ntile], tile = id % ntile;
    const int hreal = hv / a.kps, par = hv - hreal * a.kps, rl = hreal - a.r_lat0;
    if (rl < 0 || rl >= a.r_nlat) return;
    const int vlo = (a.r_lon_lo - par + a.kps - 1) / a.kps, nv = (a.r_lon_lo + a.r_nkx - par + a.kps - 1) / a.kps - vlo;
    const int w0 = vlo + HQ * tile; // first virtual column of the tile
    const int nvalid = min(HQ, vlo + nv - w0);
    if (nvalid <= 0) return;
    const bool mine = c < nvalid;
    const size_t pt = ((size_t)b * a.r_nlat + rl) * a.r_nkx + (size_t)((w0 + (mine ? c : 0)) * a.kps + par - a.r_lon_lo); // the key in the chunk
    int ri = a.soff[hv];
    const int rend = a.soff[hv + 1];
    if (ri >= rend) { // no query sees this latitude
        if (WRITE && mine) {
            float *dk = static_cast<float *>(a.dk) + pt * drt + 4 * qd, *dv = static_cast<float *>(a.dv) + pt * drt + 4 * qd;
#pragma unroll
            for (int cb = 0; cb < NCB; cb++) {
                if (16 * cb + 4 * qd < dr) {
                    *reinterpret_cast<float4 *>(dk + 16 * cb) = make_float4(0.f, 0.f, 0.f, 0.f);
                    *reinterpret_cast<float4 *>(dv + 16 * cb) = make_float4(0.f, 0.f, 0.f, 0.f);
                }
            }
        }
        return;
    }

    char *lds = m32_lds<m32_lds_bytes<D, 1>(true), 1>();
    char *Qs = lds, *Gs = Qs + HK * PITCH;
    float *Ls = reinterpret_cast<float *>(Gs + HK * PITCH), *Is = Ls + HK;
    const unsigned ldb = drt * sizeof(T); // bytes between two grid points
    const int Hor = a.Ho / a.r_qps; // real local output latitudes
    const size_t sbase = (size_t)b * Hor * a.r_wo;
    const char *qy = static_cast<const char *>(a.q) + sbase * ldb;
    const char *gy = static_cast<const char *>(a.dy) + sbase * ldb;

    float kop[D / 4], vop[D / 4]; // this lane's quarter of key c
    m32_load_quarter<D, T>(kop, static_cast<const char *>(a.k) + pt * ldb, qd, dr);
    m32_load_quarter<D, T>(vop, static_cast<const char *>(a.v) + pt * ldb, qd, dr);
    f4v dkt[NCB], dvt[NCB];
#pragma unroll
    for (int cb = 0; cb < NCB; cb++) {
        dkt[cb] = f4v{0.f, 0.f, 0.f, 0.f};
        dvt[cb] = f4v{0.f, 0.f, 0.f, 0.f};
    }
    const float lw = fast_log2(a.quad_w[hreal + a.r_wlat0]);

    Tile qt, gt;
    float2 st = make_float2(0.f, 0.f);
    const int r0 = lane / Tile::CPR;
    const unsigned pc = 4u * sizeof(T) * (lane % Tile::CPR);
    const bool piece_ok = 4 * (lane % Tile::CPR) < dr; // this lane's four channels of a staged row exist
    RingWalk2 wk;
    wk.W = a.Wi, wk.w0 = w0, wk.qps = a.r_qps, wk.wo = a.r_wo;
    wk.start(a.sruns, ri, rend);
    const bool any = wk.advance(); // false: none of the queries that see these keys is local
    auto fetch = [&]() { // the rows of the step the walk stands at; rows beyond the interval are staged as zeros and weigh nothing
        // the run's output latitude is virtual (real latitude Run::pad, column class parq): virtual column j is the local
        // query column j * r_qps + parq
        const size_t lat = (size_t)wk.run.pad * a.r_wo + wk.parq;
        const int nrows = wk.ub - wk.pos;
#pragma unroll
        for (int it = 0; it < Tile::NIT; it++) {
            const int row = r0 + it * Tile::RPI;
            qt.raw[it] = u4v{0u, 0u, 0u, 0u};
            gt.raw[it] = u4v{0u, 0u, 0u, 0u};
            if (row < nrows && piece_ok) {
                int cr = wk.col + row; // wraps only when the window is the whole circle
                cr -= (cr >= a.Wi) ? a.Wi : 0;
                const size_t o = (lat + (size_t)cr * a.r_qps) * ldb + pc;
                qt.raw[it] = m32_piece<T>(qy + o);
                gt.raw[it] = m32_piece<T>(gy + o);
            }
        }
        if (lane < HK) { // lanes 0..31 fetch the statistics of the staged rows: (log2-sum-exp, integral_norm)
            st = make_float2(INFINITY, 0.f); // exp2(-inf) = 0
            if (lane < nrows) {
                int cr = wk.col + lane;
                cr -= (cr >= a.Wi) ? a.Wi : 0;
                const size_t s = sbase + lat + (size_t)cr * a.r_qps;
                const float as = a.r_asum[s];
                if (as > 0.f) st = make_float2(fmaf(a.r_qmax[s], LOG2E, fast_log2(as)), a.r_integral[s]); // (a query that saw nothing weighs nothing)
            }
        }
    };
    auto commit = [&]() {
        qt.commit(Qs, lane);
        gt.commit(Gs, lane);
        if (lane < HK) {
            Ls[lane] = st.x;
            Is[lane] = st.y;
        }
    };
    if (any) {
        fetch();
        commit();
    }
    __syncthreads();
    settle(kop);
    settle(vop);

    while (any) {
        const int len = wk.run.len, pos = wk.pos, ub = wk.ub;
        const bool more = wk.advance();
        if (more) fetch();

        f4v sc[2], gc[2];
        m32_scores<D, PITCH>(sc, Qs, c, qd, kop);
        m32_scores<D, PITCH>(gc, Gs, c, qd, vop);
        // element (qb, v) is staged row u = pos + 16 qb + 4 qd + v, which sees key c as its neighbor t = u - c: it counts iff
        // 0 <= t < len and u < ub, i.e. t < min(len, ub - c) as unsigned numbers
        const int tb = pos + 4 * qd - c;
        const unsigned lim = (unsigned)max(0, min(len, ub - c));
        const bool inner = pos >= HQ - 1 && pos + HK <= min(len, ub); // every element of the step counts
#pragma unroll
        for (int qb = 0; qb < 2; qb++) {
            const float4 l4 = *reinterpret_cast<const float4 *>(Ls + 16 * qb + 4 * qd);
            const float4 i4 = *reinterpret_cast<const float4 *>(Is + 16 * qb + 4 * qd);
            const float lv[4] = {l4.x, l4.y, l4.z, l4.w};
            const float iv[4] = {i4.x, i4.y, i4.z, i4.w};
#pragma unroll
            for (int v = 0; v < 4; v++) {
                float p = fast_exp2(fmaf(sc[qb][v], LOG2E, lw - lv[v])); // = alpha / alpha_sum
                if (!inner) p = ((unsigned)(tb + 16 * qb + v) < lim) ? p : 0.f;
                sc[qb][v] = p;
                gc[qb][v] = p * (gc[qb][v] - iv[v]);
            }
        }
        m32_accumulate<D, PITCH>(dvt, Gs, c, qd, sc);
        m32_accumulate<D, PITCH>(dkt, Qs, c, qd, gc);

        __syncthreads();
        if (!more) break;
        commit();
        __syncthreads();
    }

    if (mine) {
        float *dk = static_cast<float *>(a.dk) + pt * drt + 4 * qd, *dv = static_cast<float *>(a.dv) + pt * drt + 4 * qd;
#pragma unroll
        for (int cb = 0; cb < NCB; cb++) {
            if (16 * cb + 4 * qd < dr) {
                float4 x = make_float4(0.f, 0.f, 0.f, 0.f), y = x;
                if (!WRITE) x = *reinterpret_cast<const float4 *>(dk + 16 * cb), y = *reinterpret_cast<const float4 *>(dv + 16 * cb);
                x.x += dkt[cb][0], x.y += dkt[cb][1], x.z += dkt[cb][2], x.w += dkt[cb][3];
                y.x += dvt[cb][0], y.y += dvt[cb][1], y.z += dvt[cb][2], y.w += dvt[cb][3];
                *reinterpret_cast<float4 *>(dk + 16 * cb) = x;
                *reinterpret_cast<float4 *>(dv + 16 * cb) = y;
            }
        }
    }
}
