// Pair path of the hybrid fp32 kernels (head dim 32), forward and dk/dv pass: one wavefront works TWO adjacent latitudes of
// the short-run kind on the same 32 longitudes.  Included by s2attn_kernels.hip inside namespace s2, after Tile40.
//
// Why: on the short-run latitudes (the equatorial nine tenths of an equiangular grid: a handful of runs of 1-9 longitudes
// per latitude) the vector path is bound by LDS reads and by the fixed cost of a step (fetch, commit, two barriers, run
// bookkeeping), not by its FMAs.  Adjacent latitudes see nearly the same bands of the other grid (7 + 1 latitudes for two
// rows instead of 7 + 7), so staging the UNION band once and reading each of its rows once for two queries (or two keys)
// per lane halves both.  The plan lists the pairs and their merged runs (PRun); a lane keeps the state of both latitudes,
// in the same (j, half) layout as the single-latitude path: lane (j, half) owns channels 8g + 4 half + e of longitude j.
//
// Band position i of a merged run belongs to latitude A iff dA <= i < dA + lenA (B likewise); all predicates are
// wave-uniform.  A merged band longer than one chunk (VC positions) is walked in chunks like a run of the single path.  Results are the same sums in the same order as the single-latitude vector path.

struct PRun {
    int lat, ws, len, aux, dA, lenA, dB, lenB;
};

// The merged runs of a pair (at most S2_PAIR_MAX_RUNS of 8 ints) are copied to LDS once; every step then reads its run from
// there (LDS latency instead of a dependent global load in front of every tile fetch).  A run is the same for the whole
// wavefront: reading it through readfirstlane tells the compiler so, and everything derived from it (band start, row base
// address, the position predicates) lives in scalar registers.
__device__ inline void stage_pruns(int *Rs, const PRun *src, int n, int lane)
{
    const int *g = reinterpret_cast<const int *>(src);
    for (int i = lane; i < 8 * n; i += 64) Rs[i] = g[i];
}
__device__ inline PRun load_prun(const int *Rs, int k)
{
    const int4 lo = *reinterpret_cast<const int4 *>(Rs + 8 * k), hi = *reinterpret_cast<const int4 *>(Rs + 8 * k + 4);
    PRun r;
    r.lat = __builtin_amdgcn_readfirstlane(lo.x), r.ws = __builtin_amdgcn_readfirstlane(lo.y);
    r.len = __builtin_amdgcn_readfirstlane(lo.z), r.aux = __builtin_amdgcn_readfirstlane(lo.w);
    r.dA = __builtin_amdgcn_readfirstlane(hi.x), r.lenA = __builtin_amdgcn_readfirstlane(hi.y);
    r.dB = __builtin_amdgcn_readfirstlane(hi.z), r.lenB = __builtin_amdgcn_readfirstlane(hi.w);
    return r;
}

// Four independent chains of four FMAs, then a tree add: a single chain of 16 dependent FMAs leaves a wavefront waiting on
// its own previous instruction most of the time (few wavefronts are resident to fill the gaps).
__device__ inline float dot16(const float (&q)[16], const float4 (&x)[4])
{
    float p[4];
#pragma unroll
    for (int g = 0; g < 4; g++) {
        p[g] = q[4 * g] * x[g].x;
        p[g] = fmaf(q[4 * g + 1], x[g].y, p[g]);
        p[g] = fmaf(q[4 * g + 2], x[g].z, p[g]);
        p[g] = fmaf(q[4 * g + 3], x[g].w, p[g]);
    }
    return (p[0] + p[1]) + (p[2] + p[3]);
}

__device__ inline void axpy16(float (&acc)[16], float c, const float4 (&x)[4])
{
#pragma unroll
    for (int g = 0; g < 4; g++) {
        acc[4 * g] = fmaf(c, x[g].x, acc[4 * g]);
        acc[4 * g + 1] = fmaf(c, x[g].y, acc[4 * g + 1]);
        acc[4 * g + 2] = fmaf(c, x[g].z, acc[4 * g + 2]);
        acc[4 * g + 3] = fmaf(c, x[g].w, acc[4 * g + 3]);
    }
}

__device__ inline void read_row(float4 (&x)[4], const float *row)
{
#pragma unroll
    for (int g = 0; g < 4; g++) x[g] = *reinterpret_cast<const float4 *>(row + 8 * g);
}

template <typename T> __device__ inline void load_half_row(float (&dst)[16], const T *row, float scale)
{
#pragma unroll
    for (int g = 0; g < 4; g++) {
        const float4 x = load4(row + 8 * g);
        dst[4 * g] = x.x * scale, dst[4 * g + 1] = x.y * scale, dst[4 * g + 2] = x.z * scale, dst[4 * g + 3] = x.w * scale;
    }
}

template <typename T> __device__ inline void store_half_row(T *row, const float (&v)[16], float scale)
{
#pragma unroll
    for (int g = 0; g < 4; g++) store4(row + 8 * g, make_float4(v[4 * g] * scale, v[4 * g + 1] * scale, v[4 * g + 2] * scale, v[4 * g + 3] * scale));
}

// ---- forward ---------------------------------------------------------------------------------------------------------
template <typename T>
__device__ inline void fwd_pair(const Args &a, float *Ks, float *Vs, int *Rs, int lane, int b, int h, int w0, int nvalid, int hoA, int pidx)
{
    const int j = lane & 31, half = lane >> 5, bh = b * a.nh + h, hoB = hoA + 1;
    const unsigned ldk = a.ldk, ldv = a.ldv;
    const T *kx = static_cast<const T *>(a.k) + (size_t)b * a.Hi * a.Wi * ldk + (size_t)h * 32;
    const T *vx = static_cast<const T *>(a.v) + (size_t)b * a.Hi * a.Wi * ldv + (size_t)h * 32;
    const bool mine = j < nvalid;
    const size_t col = (size_t)(w0 + (mine ? j : 0)) * a.qps;
    const size_t ptA = (size_t)query_point(a, b, hoA, hoA / a.qps) + col, ptB = (size_t)query_point(a, b, hoB, hoB / a.qps) + col;

    float qA[16], qB[16], accA[16], accB[16];
    load_half_row(qA, static_cast<const T *>(a.q) + ptA * a.ldq + (size_t)h * 32 + 4 * half, LOG2E);
    load_half_row(qB, static_cast<const T *>(a.q) + ptB * a.ldq + (size_t)h * 32 + 4 * half, LOG2E);
#pragma unroll
    for (int v = 0; v < 16; v++) accA[v] = 0.f, accB[v] = 0.f;
    float mA = NEG_BIG, SA = 0.f, mB = NEG_BIG, SB = 0.f;

    int ri = 0;
    const int rend = a.gpoff[pidx + 1] - a.gpoff[pidx];
    stage_pruns(Rs, a.gpruns + a.gpoff[pidx], rend, lane);
    __syncthreads();
    PRun run = load_prun(Rs, 0);
    Tile40<T> kt, vt;
    auto fetch = [&](const PRun &rn, int p) {
        const int c0 = (rn.ws + w0 + p) % a.Wi;
        kt.fetch(kx + (size_t)key_row(a, rn.lat, rn.aux) * ldk, ldk * a.kps, c0, a.Wi, lane, true);
        vt.fetch(vx + (size_t)key_row(a, rn.lat, rn.aux) * ldv, ldv * a.kps, c0, a.Wi, lane, true);
    };
    fetch(run, 0);
    int pos = 0;
    kt.commit(Ks, lane, true);
    vt.commit(Vs, lane, true);
    __syncthreads();
    settle(qA);
    settle(qB);

    const float *kq = Ks + j * MLK + 4 * half, *vq = Vs + j * MLK + 4 * half;
    while (ri < rend) {
        const float w = a.quad_w[run.aux];
        const int L = min(VC, run.len - pos); // band positions pos .. pos + L - 1 in this step
        int nri = ri, npos = pos + VC;
        PRun nrun = run;
        if (npos >= run.len) {
            nri++;
            npos = 0;
            if (nri < rend) nrun = load_prun(Rs, nri);
        }
        const bool more = nri < rend;
        if (more) fetch(nrun, npos);
        // One pass per band position, software-pipelined over the LDS reads: the K row of a position is read while the
        // previous position's exponentials and accumulations run, its V row while its two dot products do, so a step does
        // not begin by waiting a full LDS round trip (the same registers as reading both rows up front: a K row is dead once
        // both scores exist).  The running maximum is only a reference point of the exponentials, so it is moved lazily
        // (see RESCALE_THR).
        float4 x[4], z[4];
        read_row(x, kq);
#pragma unroll
        for (int u = 0; u < VC; u++) {
            if (u < L) {
                const bool inA = (unsigned)(pos + u - run.dA) < (unsigned)run.lenA, inB = (unsigned)(pos + u - run.dB) < (unsigned)run.lenB;
                read_row(z, vq + u * MLK);
                float scA = 0.f, scB = 0.f;
                if (inA) scA = xor32_sum(dot16(qA, x));
                if (inB) scB = xor32_sum(dot16(qB, x));
                __builtin_amdgcn_sched_barrier(0);
                read_row(x, kq + (u + 1) * MLK); // (past the last position: a row nobody uses, still inside the buffer)
                __builtin_amdgcn_sched_barrier(0);
                if (inA) {
                    const float sc = scA;
                    if (__any(sc > mA + RESCALE_THR)) {
                        const float mn = sc > mA + RESCALE_THR ? sc : mA, corr = fast_exp2(mA - mn);
                        SA *= corr;
#pragma unroll
                        for (int v = 0; v < 16; v++) accA[v] *= corr;
                        mA = mn;
                    }
                    const float p = fast_exp2(sc - mA) * w;
                    SA += p;
                    axpy16(accA, p, z);
                }
                if (inB) {
                    const float sc = scB;
                    if (__any(sc > mB + RESCALE_THR)) {
                        const float mn = sc > mB + RESCALE_THR ? sc : mB, corr = fast_exp2(mB - mn);
                        SB *= corr;
#pragma unroll
                        for (int v = 0; v < 16; v++) accB[v] *= corr;
                        mB = mn;
                    }
                    const float p = fast_exp2(sc - mB) * w;
                    SB += p;
                    axpy16(accB, p, z);
                }
            }
        }
        __syncthreads();
        if (more) {
            kt.commit(Ks, lane, true);
            vt.commit(Vs, lane, true);
        }
        __syncthreads();
        ri = nri;
        pos = npos;
        run = nrun;
    }

    if (mine) {
        if (a.lse && half == 0) {
            a.lse[((size_t)bh * a.Ho + hoA) * a.Wo + w0 + j] = mA + fast_log2(SA);
            a.lse[((size_t)bh * a.Ho + hoB) * a.Wo + w0 + j] = mB + fast_log2(SB);
        }
        store_half_row(static_cast<T *>(a.y) + ptA * a.ldy + (size_t)h * 32 + 4 * half, accA, 1.0f / SA);
        store_half_row(static_cast<T *>(a.y) + ptB * a.ldy + (size_t)h * 32 + 4 * half, accB, 1.0f / SB);
    }
}

// ---- backward, dk and dv: the pair is two adjacent INPUT latitudes, staged rows are queries --------------------------------
template <typename T>
__device__ inline void dkdv_pair(const Args &a, float *Qs, float *Gs, float *Ls, float *Is, int *Rs, int lane, int b, int h, int w0, int nvalid, int hiA, int pidx)
{
    const int j = lane & 31, half = lane >> 5, bh = b * a.nh + h, hiB = hiA + 1;
    const unsigned ldq = a.ldq, ldg = a.ldg;
    const T *qy = static_cast<const T *>(a.q) + (size_t)b * a.Ho * a.Wo * ldq + (size_t)h * 32;
    const T *gy = static_cast<const T *>(a.dy) + (size_t)b * a.Ho * a.Wo * ldg + (size_t)h * 32;
    const float2 *stats = a.stats + (size_t)bh * a.Ho * a.Wo;
    const bool mine = j < nvalid;
    const size_t col = (size_t)(w0 + (mine ? j : 0)) * a.kps;
    const size_t ptA = (size_t)key_point(a, b, hiA, hiA / a.kps) + col, ptB = (size_t)key_point(a, b, hiB, hiB / a.kps) + col;

    float kA[16], kB[16], vA[16], vB[16], dkA[16], dkB[16], dvA[16], dvB[16];
    {
        const size_t ofs = (size_t)h * 32 + 4 * half;
        load_half_row(kA, static_cast<const T *>(a.k) + ptA * a.ldk + ofs, LOG2E);
        load_half_row(kB, static_cast<const T *>(a.k) + ptB * a.ldk + ofs, LOG2E);
        load_half_row(vA, static_cast<const T *>(a.v) + ptA * a.ldv + ofs, 1.0f);
        load_half_row(vB, static_cast<const T *>(a.v) + ptB * a.ldv + ofs, 1.0f);
    }
#pragma unroll
    for (int v = 0; v < 16; v++) dkA[v] = 0.f, dkB[v] = 0.f, dvA[v] = 0.f, dvB[v] = 0.f;
    const float wA = a.quad_w[hiA / a.kps], wB = a.quad_w[hiB / a.kps];

    int ri = 0;
    const int rend = a.spoff[pidx + 1] - a.spoff[pidx];
    stage_pruns(Rs, a.spruns + a.spoff[pidx], rend, lane);
    __syncthreads();
    PRun run = load_prun(Rs, 0);
    Tile40<T> qt, gt;
    float2 st = make_float2(0.f, 0.f);
    auto fetch = [&](const PRun &rn, int p) {
        int c0 = (w0 - rn.ws - rn.len + 1 + p) % a.Wo; // longitude of staged row 0
        c0 += (c0 < 0) ? a.Wo : 0;
        qt.fetch(qy + (size_t)query_row(a, rn.lat, rn.aux) * ldq, ldq * a.qps, c0, a.Wo, lane, true);
        gt.fetch(gy + (size_t)query_row(a, rn.lat, rn.aux) * ldg, ldg * a.qps, c0, a.Wo, lane, true);
        int cs = c0 + lane; // lanes 0..39 fetch the statistics of the staged rows
        cs -= (cs >= a.Wo) ? a.Wo : 0;
        if (lane < MR) st = stats[(size_t)rn.lat * a.Wo + cs];
    };
    auto commit = [&]() {
        qt.commit(Qs, lane, true);
        gt.commit(Gs, lane, true);
        if (lane < MR) {
            Ls[lane] = st.x;
            Is[lane] = st.y;
        }
    };
    fetch(run, 0);
    int pos = 0;
    commit();
    __syncthreads();
    settle(kA);
    settle(kB);
    settle(vA);
    settle(vB);

    const float *qq = Qs + j * MLK + 4 * half, *gq = Gs + j * MLK + 4 * half;
    while (ri < rend) {
        const int L = min(VC, run.len - pos); // band positions pos .. pos + L - 1 in this step
        int nri = ri, npos = pos + VC;
        PRun nrun = run;
        if (npos >= run.len) {
            nri++;
            npos = 0;
            if (nri < rend) nrun = load_prun(Rs, nri);
        }
        const bool more = nri < rend;
        if (more) fetch(nrun, npos);
#pragma unroll
        for (int i = 0; i < VC; i++) {
            if (i < L) {
                const bool inA = (unsigned)(pos + i - run.dA) < (unsigned)run.lenA, inB = (unsigned)(pos + i - run.dB) < (unsigned)run.lenB;
                float4 xq[4], xg[4];
                read_row(xq, qq + i * MLK);
                read_row(xg, gq + i * MLK);
                const float L = Ls[j + i], I = Is[j + i];
                if (inA) {
                    const float s = xor32_sum(dot16(kA, xq)), gd = xor32_sum(dot16(vA, xg));
                    const float p = fast_exp2(s - L) * wA;
                    axpy16(dkA, p * (gd - I), xq);
                    axpy16(dvA, p, xg);
                }
                if (inB) {
                    const float s = xor32_sum(dot16(kB, xq)), gd = xor32_sum(dot16(vB, xg));
                    const float p = fast_exp2(s - L) * wB;
                    axpy16(dkB, p * (gd - I), xq);
                    axpy16(dvB, p, xg);
                }
            }
        }
        __syncthreads();
        if (more) commit();
        __syncthreads();
        ri = nri;
        pos = npos;
        run = nrun;
    }

    if (mine) {
        const size_t ofs = (size_t)h * 32 + 4 * half;
        store_half_row(static_cast<T *>(a.dk) + ptA * a.lddk + ofs, dkA, 1.0f);
        store_half_row(static_cast<T *>(a.dk) + ptB * a.lddk + ofs, dkB, 1.0f);
        store_half_row(static_cast<T *>(a.dv) + ptA * a.lddv + ofs, dvA, 1.0f);
        store_half_row(static_cast<T *>(a.dv) + ptB * a.lddv + ofs, dvB, 1.0f);
    }
}
