// Host-side conversion of the CSR neighborhood into longitude runs (see include/s2attn.h).
//
// The reference keeps the neighborhood as one int64 column index per neighbor and
// only reorders rows by length (attention_cuda_utils.cu:74-113).  On the sphere
// every row is a stack of longitude intervals, one per input latitude, so a row of
// thousands of neighbors collapses to a handful of (lat, start, len) runs.  Runs
// are what lets a wavefront stage one contiguous band of K/V per latitude in LDS
// and slide all of its queries over it.

#include "s2attn_internal.h"

#include <algorithm>
#include <cstdio>
#include <numeric>
#include <vector>

namespace {

struct HostRun {
    int32_t ho, hi, ws, len; // virtual output latitude, virtual input latitude, first column, length (see include/s2attn.h)
};

// One CSR row -> maximal runs of consecutive columns inside one latitude of the OTHER grid (nlon columns per latitude);
// a run that ends at nlon - 1 is joined with a run of the same latitude that starts at 0 into one circular run.
struct RawRun {
    int32_t lat, ws, len;
};
int row_runs(const int64_t *col_idx, int64_t z0, int64_t z1, int nlat, int nlon, std::vector<RawRun> &row)
{
    const int64_t ncol = (int64_t)nlat * nlon;
    row.clear();
    for (int64_t z = z0; z < z1; z++) {
        const int64_t col = col_idx[z];
        if (col < 0 || col >= ncol)
            return s2attn_fail(S2ATTN_E_INVALID, "col_idx[%lld] = %lld outside [0, %lld)", (long long)z, (long long)col, (long long)ncol);
        const int32_t lat = (int32_t)(col / nlon), w = (int32_t)(col % nlon);
        if (!row.empty() && row.back().lat == lat && row.back().ws + row.back().len == w && row.back().len < nlon) {
            row.back().len++;
        } else {
            row.push_back({lat, w, 1});
        }
    }
    size_t i = 0;
    while (i < row.size()) {
        size_t j = i;
        while (j + 1 < row.size() && row[j + 1].lat == row[i].lat) j++;
        if (j > i && row[i].ws == 0 && row[j].ws + row[j].len == nlon && row[i].len + row[j].len <= nlon) {
            row[j].len += row[i].len;
            row[i].len = 0; // dropped
        }
        i = j + 1;
    }
    return S2ATTN_OK;
}

// Converts the CSR into runs on virtual latitudes.  Two directions, told apart by the longitude counts:
//
// gather (nlon_in = ps * nlon_out): rows are output latitudes ho, columns hi * nlon_in + wi; query column wo sees input
//   columns ws + t + ps * wo.  Every run is split by column class par = column mod ps: on the sub-lattice
//   {par, par + ps, ...} of latitude hi (virtual input latitude hi * ps + par, nlon_out columns) the same neighbors are
//   a run (ws', len') with unit stride in wo.
// scatter (nlon_out = ps * nlon_in, ps > 1): rows are INPUT latitudes hi, columns ho * nlon_out + wo; input column wi is
//   seen by output columns ws + t + ps * wi.  Split by output column class: on virtual output latitude ho * ps + par
//   (nlon_in columns j) input column wi is seen by j = us + u + wi, u in [0, len'), i.e. query column j sees the input
//   columns (j - us - len' + 1) + t', t' in [0, len'): the run (ws'' = -us - len' + 1 mod nlon_in, len').
// Either way the result reads: query column j of virtual output latitude `ho` sees columns (ws + t + j) mod W of virtual
// input latitude `hi`, t in [0, len), W = min(nlon_in, nlon_out).
int decompose(const int64_t *col_idx, const int64_t *row_off, int64_t nnz, int nlat_in, int nlon_in, int nlat_out,
              int nlon_out, std::vector<HostRun> *out, int64_t *count)
{
    if (!col_idx && nnz > 0) return s2attn_fail(S2ATTN_E_INVALID, "col_idx is null");
    if (!row_off) return s2attn_fail(S2ATTN_E_INVALID, "row_off is null");
    if (nlat_in < 1 || nlon_in < 1 || nlat_out < 1 || nlon_out < 1)
        return s2attn_fail(S2ATTN_E_INVALID, "grid extents must be positive");
    const bool up = nlon_out % nlon_in == 0 && nlon_out != nlon_in;
    if (!up && nlon_in % nlon_out != 0)
        return s2attn_fail(S2ATTN_E_INVALID, "nlon_in (%d) must be an integer multiple of nlon_out (%d), or the other way round", nlon_in, nlon_out);
    const int nrow = up ? nlat_in : nlat_out;
    if (row_off[0] != 0 || row_off[nrow] != nnz)
        return s2attn_fail(S2ATTN_E_INVALID, "row_off must start at 0 and end at nnz (%lld), got %lld..%lld", (long long)nnz,
                           (long long)row_off[0], (long long)row_off[nrow]);

    const int ps = up ? nlon_out / nlon_in : nlon_in / nlon_out;
    const int W = up ? nlon_in : nlon_out;             // columns of a virtual latitude
    const int nlat_other = up ? nlat_out : nlat_in;    // grid the CSR columns live on
    const int nlon_other = up ? nlon_out : nlon_in;
    int64_t total = 0;
    std::vector<RawRun> row;
    for (int r = 0; r < nrow; r++) {
        const int64_t z0 = row_off[r], z1 = row_off[r + 1];
        if (z1 < z0) return s2attn_fail(S2ATTN_E_INVALID, "row_off decreases at row %d", r);
        const int rc = row_runs(col_idx, z0, z1, nlat_other, nlon_other, row);
        if (rc != S2ATTN_OK) return rc;
        for (const RawRun &rr : row) {
            if (rr.len == 0) continue;
            for (int par = 0; par < ps; par++) {
                const int t0 = ((par - rr.ws) % ps + ps) % ps; // first entry of the run in this column class
                if (t0 >= rr.len) continue;
                const int first = (rr.ws + t0) % nlon_other;
                const int us = (first - par) / ps, len = (rr.len - t0 + ps - 1) / ps;
                total++;
                if (!out) continue;
                if (up) {
                    out->push_back({rr.lat * ps + par, r, ((-us - len + 1) % W + W) % W, len});
                } else {
                    out->push_back({r, rr.lat * ps + par, us, len});
                }
            }
        }
    }
    if (total > 0x7fffffffLL) return s2attn_fail(S2ATTN_E_UNSUPPORTED, "the neighborhood has %lld runs, more than the plan's 32-bit offsets index", (long long)total);
    *count = total;
    return S2ATTN_OK;
}

} // namespace

namespace {

// Cost model (SIMD cycles per 32 grid points) deciding which kernel family a latitude goes to.  The matrix-core
// kernels pay per 32 x 32 tile whether or not the band fills it; the vector kernels pay per neighbor plus a fixed
// amount per chunk of 8.  Constants fitted to measured kernel times on MI355X.
struct RowCost {
    int64_t dense = 0, vector = 0;
    void add(int len)
    {
        dense += (int64_t)((len + 31 + 31) / 32) * 5200;
        vector += (int64_t)len * 770;
    }
};

// order: latitudes with long runs first, then the others; inside each class most work first -- but by cost CLASS
// (steps of 1/8 in log2), keeping the natural order inside a class.  A plain sort by cost interleaves the two
// hemispheres (mirror latitudes cost the same); with classes, consecutive entries are neighboring latitudes, whose
// tiles share most of their K/V rows in L2.  Returns the number of long-run latitudes.
// mixed: the same two lists merged so that at every point of the launch about the same share of each list's work has
// been handed out (see merge_by_share).
int cost_class(int64_t c)
{
    int cls = 0;
    while ((c >> cls) > 15) cls++; // c = m * 2^cls, 8 <= m < 16
    return c <= 0 ? -1 : cls * 8 + (int)((c >> cls) - 8);
}

// Two work lists (matrix-core-heavy and vector-heavy units, each most work first) merged in proportion to their work.
// The kernels that treat long runs on the matrix cores and short runs on the vector ALU take this order: both kinds of
// workgroups then sit side by side on a SIMD for the whole launch instead of one kind after the other (measured 6-7 %
// on 721x1440 grids).  `hold` bounds the long-run list's share of work handed out relative to the other list's.  Gather
// grouping (forward, dq pass): 0.7, the long-run list held back a little (measured best between 0.5 and 0.8, 1.5-2 % of
// the step over equal shares).  Scatter grouping (dk/dv pass): 1.2 - its long-run steps run on the bf16 matrix
// instructions and cost less than the model's common weight says, so they are handed out a little ahead (dk/dv pass at
// 721x1440 self-attention 4.47 -> 4.38 ms, 4.60 -> 4.45 on unstructured inputs; 2.0 gives the same there but costs the
// 721x1440 -> 360x720 down-sampling 5 %; the dq pass loses 3 % with values above 1).
constexpr double HOLD_GATHER = 0.7, HOLD_SCATTER = 1.2;
template <typename Emit> void merge_by_share(const std::vector<int64_t> &cd_, const std::vector<int64_t> &cv_, double hold, Emit emit)
{
    double wd = 0, wv = 0;
    for (int64_t c : cd_) wd += (double)c;
    for (int64_t c : cv_) wv += (double)c;
    size_t i = 0, j = 0;
    double cd = 0, cv = 0;
    while (i < cd_.size() || j < cv_.size()) {
        const bool take_dense = j >= cv_.size() || (i < cd_.size() && cd * wv <= hold * cv * wd);
        if (take_dense) {
            cd += (double)cd_[i];
            emit(true, i++);
        } else {
            cv += (double)cv_[j];
            emit(false, j++);
        }
    }
}

int32_t order_rows(const std::vector<RowCost> &cost, int32_t *order, int32_t *mixed, double hold)
{
    const int n = (int)cost.size();
    std::vector<int32_t> dense, vec;
    for (int i = 0; i < n; i++) (cost[i].dense < cost[i].vector ? dense : vec).push_back(i);
    std::stable_sort(dense.begin(), dense.end(), [&](int32_t a, int32_t b) { return cost_class(cost[a].dense) > cost_class(cost[b].dense); });
    std::stable_sort(vec.begin(), vec.end(), [&](int32_t a, int32_t b) { return cost_class(cost[a].vector) > cost_class(cost[b].vector); });
    std::copy(dense.begin(), dense.end(), order);
    std::copy(vec.begin(), vec.end(), order + dense.size());
    std::vector<int64_t> cd, cv;
    for (int32_t r : dense) cd.push_back(cost[r].dense);
    for (int32_t r : vec) cv.push_back(cost[r].vector);
    int32_t *out = mixed;
    merge_by_share(cd, cv, hold, [&](bool d, size_t k) { *out++ = d ? dense[k] : vec[k]; });
    return (int32_t)dense.size();
}

// ---- latitude pairs ------------------------------------------------------------------------------------------------
// The hybrid kernels (fp32 heads of 32 channels) work two ADJACENT latitudes of the short-run kind in one wavefront: both
// latitudes' neighborhoods lie in nearly the same bands of the other grid, so one staged band and one LDS read of each
// of its rows serve two queries (or two keys) per lane.  A pair is formed when, latitude by latitude of the other grid,
// the two runs fit into one band shorter than S2_LMIN positions; its runs are stored merged:
//   (lat, ws, len, aux, dA, lenA, dB, lenB)
// (lat, ws, len, aux) is the union band in the form of a single run of the same grouping; position i of the band
// (0 <= i < len) belongs to the first latitude iff dA <= i < dA + lenA and to the second iff dB <= i < dB + lenB.
struct Group {
    const int32_t *runs; // 4 ints each
    int n;
};

// centred representative of a circular start column
int centred(int ws, int W) { return ws < (W + 1) / 2 ? ws : ws - W; }

bool short_sorted(const Group &g)
{
    for (int i = 0; i < g.n; i++) {
        if (g.runs[4 * i + 2] >= S2_LMIN) return false;
        if (i > 0 && g.runs[4 * i] <= g.runs[4 * (i - 1)]) return false; // one run per latitude, ascending
    }
    return g.n > 0;
}

// merges the runs of two groups; scatter = the d offsets are measured from the END of the union band (the dk/dv kernels
// index a band backwards: staged row 0 is the query column that sees the tile's first key through the LAST neighbor).
bool merge_pair(const Group &A, const Group &B, int W, bool scatter, std::vector<int32_t> *out)
{
    if (!short_sorted(A) || !short_sorted(B) || W < 4 * S2_LMIN) return false;
    std::vector<int32_t> tmp;
    int i = 0, j = 0;
    while (i < A.n || j < B.n) {
        const int32_t *ra = i < A.n ? A.runs + 4 * i : nullptr, *rb = j < B.n ? B.runs + 4 * j : nullptr;
        const bool useA = ra && (!rb || ra[0] <= rb[0]), useB = rb && (!ra || rb[0] <= ra[0]);
        const int32_t *any = useA ? ra : rb;
        int s0 = 0, e1 = 0, sA = 0, lenA = 0, sB = 0, lenB = 0;
        if (useA) sA = centred(ra[1], W), lenA = ra[2];
        if (useB) sB = centred(rb[1], W), lenB = rb[2];
        if (useA && useB) {
            s0 = std::min(sA, sB), e1 = std::max(sA + lenA, sB + lenB);
        } else if (useA) {
            s0 = sA, e1 = sA + lenA, sB = sA;
        } else {
            s0 = sB, e1 = sB + lenB, sA = sB;
        }
        if (e1 - s0 >= S2_LMIN) return false;
        const int dA = scatter ? e1 - (sA + lenA) : sA - s0, dB = scatter ? e1 - (sB + lenB) : sB - s0;
        const int32_t rec[8] = {any[0], ((s0 % W) + W) % W, e1 - s0, any[3], dA, lenA, dB, lenB};
        tmp.insert(tmp.end(), rec, rec + 8);
        i += useA, j += useB;
    }
    if (tmp.size() > 8 * (size_t)S2_PAIR_MAX_RUNS) return false;
    out->insert(out->end(), tmp.begin(), tmp.end());
    return true;
}

// Work list of one grouping for the hybrid kernels: items (latitude, pair index or -1), long-run latitudes and short-run
// units (single latitudes or pairs) merged by share of work as in order_rows.
void build_items(const int32_t *off, const int32_t *runs, int ngroups, int W, bool scatter, const std::vector<RowCost> &cost,
                 std::vector<int32_t> *items, std::vector<int32_t> *pair_off, std::vector<int32_t> *pair_runs)
{
    struct Unit {
        int32_t lat, pair;
        int64_t c;
    };
    std::vector<Unit> dense, vec;
    pair_off->assign(1, 0);
    for (int r = 0; r < ngroups; r++) {
        if (cost[r].dense < cost[r].vector) {
            dense.push_back({r, -1, cost[r].dense});
            continue;
        }
        if (r + 1 < ngroups && cost[r + 1].dense >= cost[r + 1].vector) {
            const Group A = {runs + 4 * (size_t)off[r], off[r + 1] - off[r]}, B = {runs + 4 * (size_t)off[r + 1], off[r + 2] - off[r + 1]};
            if (merge_pair(A, B, W, scatter, pair_runs)) {
                vec.push_back({r, (int32_t)pair_off->size() - 1, cost[r].vector + cost[r + 1].vector});
                pair_off->push_back((int32_t)(pair_runs->size() / 8));
                r++;
                continue;
            }
        }
        vec.push_back({r, -1, cost[r].vector});
    }
    std::stable_sort(dense.begin(), dense.end(), [&](const Unit &a, const Unit &b) { return cost_class(a.c) > cost_class(b.c); });
    std::stable_sort(vec.begin(), vec.end(), [&](const Unit &a, const Unit &b) { return cost_class(a.c) > cost_class(b.c); });
    std::vector<int64_t> cd, cv;
    for (const Unit &u : dense) cd.push_back(u.c);
    for (const Unit &u : vec) cv.push_back(u.c);
    merge_by_share(cd, cv, scatter ? HOLD_SCATTER : HOLD_GATHER, [&](bool d, size_t k) {
        const Unit &u = d ? dense[k] : vec[k];
        items->push_back(u.lat);
        items->push_back(u.pair);
    });
}

// appends an array to the blob at a 16-byte boundary, returns its offset in ints
int32_t append(std::vector<int32_t> &blob, const int32_t *data, size_t n)
{
    while (blob.size() % 4) blob.push_back(0);
    const size_t at = blob.size();
    blob.insert(blob.end(), data, data + n);
    return (int32_t)at;
}

int build_blob(const int64_t *col_idx, const int64_t *row_off, int64_t nnz, int nlat_in, int nlon_in, int nlat_out, int nlon_out,
               std::vector<int32_t> &blob)
{
    std::vector<HostRun> runs;
    int64_t n = 0;
    const int rc = decompose(col_idx, row_off, nnz, nlat_in, nlon_in, nlat_out, nlon_out, &runs, &n);
    if (rc != S2ATTN_OK) return rc;

    const bool up = nlon_out % nlon_in == 0 && nlon_out != nlon_in;
    const int psk = up ? 1 : nlon_in / nlon_out, psq = up ? nlon_out / nlon_in : 1;
    const int nvin = nlat_in * psk, nvout = nlat_out * psq; // virtual latitudes
    const int W = up ? nlon_in : nlon_out;

    // both groupings by stable counting sort (entries keep the CSR's order inside a group)
    std::vector<RowCost> gcost(nvout), scost(nvin);
    std::vector<int32_t> goff(nvout + 1, 0), soff(nvin + 1, 0), gruns(4 * (size_t)n), sruns(4 * (size_t)n);
    for (int64_t i = 0; i < n; i++) {
        goff[runs[i].ho + 1]++;
        soff[runs[i].hi + 1]++;
    }
    for (int r = 0; r < nvout; r++) goff[r + 1] += goff[r];
    for (int r = 0; r < nvin; r++) soff[r + 1] += soff[r];
    std::vector<int32_t> gcur(goff.begin(), goff.end() - 1), scur(soff.begin(), soff.end() - 1);
    for (int64_t i = 0; i < n; i++) {
        const HostRun &r = runs[i];
        const int32_t g = gcur[r.ho]++, sidx = scur[r.hi]++;
        gruns[4 * g + 0] = r.hi;
        gruns[4 * g + 1] = r.ws;
        gruns[4 * g + 2] = r.len;
        gruns[4 * g + 3] = r.hi / psk; // real input latitude: quadrature weight index, row address
        sruns[4 * sidx + 0] = r.ho;
        sruns[4 * sidx + 1] = r.ws;
        sruns[4 * sidx + 2] = r.len;
        sruns[4 * sidx + 3] = r.ho / psq; // real output latitude: row address
        gcost[r.ho].add(r.len);
        scost[r.hi].add(r.len);
    }
    // per virtual output latitude: an arc (first column, columns) of the circle that holds every neighbor column of query
    // column 0 (of query column j: shifted by j); the ring step uses it to leave a tile whose arc misses the chunk at once
    std::vector<int32_t> gspan(2 * (size_t)nvout, 0);
    for (int r = 0; r < nvout; r++) {
        int lo = 0, hi = 0;
        for (int32_t g = goff[r]; g < goff[r + 1]; g++) {
            const int c0 = centred(gruns[4 * g + 1], W), c1 = c0 + gruns[4 * g + 2];
            if (g == goff[r] || c0 < lo) lo = c0;
            if (g == goff[r] || c1 > hi) hi = c1;
        }
        const int n_ = hi - lo >= W ? W : hi - lo;
        gspan[2 * r + 0] = n_ >= W ? 0 : ((lo % W) + W) % W;
        gspan[2 * r + 1] = n_;
    }
    std::vector<int32_t> gorder(nvout), gmixed(nvout), sorder(nvin), smixed(nvin);
    const int32_t gnd = order_rows(gcost, gorder.data(), gmixed.data(), HOLD_GATHER);
    const int32_t snd = order_rows(scost, sorder.data(), smixed.data(), HOLD_SCATTER);
    std::vector<int32_t> gitems, gpoff, gpruns, sitems, spoff, spruns;
    build_items(goff.data(), gruns.data(), nvout, W, false, gcost, &gitems, &gpoff, &gpruns);
    build_items(soff.data(), sruns.data(), nvin, W, true, scost, &sitems, &spoff, &spruns);

    blob.assign(S2ATTN_PLAN_HEADER_INTS, 0);
    int32_t h[S2ATTN_PLAN_HEADER_INTS] = {};
    h[S2ATTN_PH_MAGIC] = S2ATTN_PLAN_MAGIC;
    h[S2ATTN_PH_NVOUT] = nvout, h[S2ATTN_PH_NVIN] = nvin, h[S2ATTN_PH_NRUNS] = (int32_t)n;
    h[S2ATTN_PH_GATHER_NDENSE] = gnd, h[S2ATTN_PH_SCATTER_NDENSE] = snd;
    h[S2ATTN_PH_NLAT_IN] = nlat_in, h[S2ATTN_PH_NLON_IN] = nlon_in, h[S2ATTN_PH_NLAT_OUT] = nlat_out, h[S2ATTN_PH_NLON_OUT] = nlon_out;
    h[S2ATTN_PH_GATHER_OFF] = append(blob, goff.data(), goff.size());
    h[S2ATTN_PH_GATHER_RUNS] = append(blob, gruns.data(), gruns.size());
    h[S2ATTN_PH_GATHER_ORDER] = append(blob, gorder.data(), gorder.size());
    h[S2ATTN_PH_GATHER_ORDER_MIXED] = append(blob, gmixed.data(), gmixed.size());
    h[S2ATTN_PH_SCATTER_OFF] = append(blob, soff.data(), soff.size());
    h[S2ATTN_PH_SCATTER_RUNS] = append(blob, sruns.data(), sruns.size());
    h[S2ATTN_PH_SCATTER_ORDER] = append(blob, sorder.data(), sorder.size());
    h[S2ATTN_PH_SCATTER_ORDER_MIXED] = append(blob, smixed.data(), smixed.size());
    h[S2ATTN_PH_GATHER_NITEMS] = (int32_t)(gitems.size() / 2);
    h[S2ATTN_PH_GATHER_ITEMS] = append(blob, gitems.data(), gitems.size());
    h[S2ATTN_PH_GATHER_PAIR_OFF] = append(blob, gpoff.data(), gpoff.size());
    h[S2ATTN_PH_GATHER_PAIR_RUNS] = append(blob, gpruns.data(), gpruns.size());
    h[S2ATTN_PH_GATHER_NPAIRS] = (int32_t)gpoff.size() - 1;
    h[S2ATTN_PH_SCATTER_NITEMS] = (int32_t)(sitems.size() / 2);
    h[S2ATTN_PH_SCATTER_ITEMS] = append(blob, sitems.data(), sitems.size());
    h[S2ATTN_PH_SCATTER_PAIR_OFF] = append(blob, spoff.data(), spoff.size());
    h[S2ATTN_PH_SCATTER_PAIR_RUNS] = append(blob, spruns.data(), spruns.size());
    h[S2ATTN_PH_SCATTER_NPAIRS] = (int32_t)spoff.size() - 1;
    h[S2ATTN_PH_GATHER_SPAN] = append(blob, gspan.data(), gspan.size());
    while (blob.size() % 4) blob.push_back(0);
    if (blob.size() > 0x7fffffffULL) return s2attn_fail(S2ATTN_E_UNSUPPORTED, "the plan needs %zu ints, more than its 32-bit offsets index", blob.size());
    h[S2ATTN_PH_TOTAL] = (int32_t)blob.size();
    std::copy(h, h + S2ATTN_PLAN_HEADER_INTS, blob.begin());
    return S2ATTN_OK;
}

} // namespace

extern "C" int64_t s2attn_plan_count(const int64_t *col_idx, const int64_t *row_off, int64_t nnz, int nlat_in, int nlon_in,
                                     int nlat_out, int nlon_out)
{
    int64_t n = 0;
    const int rc = decompose(col_idx, row_off, nnz, nlat_in, nlon_in, nlat_out, nlon_out, nullptr, &n);
    return rc == S2ATTN_OK ? n : (int64_t)rc;
}

extern "C" int64_t s2attn_plan_size(const int64_t *col_idx, const int64_t *row_off, int64_t nnz, int nlat_in, int nlon_in,
                                    int nlat_out, int nlon_out)
{
    std::vector<int32_t> blob;
    const int rc = build_blob(col_idx, row_off, nnz, nlat_in, nlon_in, nlat_out, nlon_out, blob);
    return rc == S2ATTN_OK ? (int64_t)blob.size() : (int64_t)rc;
}

extern "C" int s2attn_plan_build(const int64_t *col_idx, const int64_t *row_off, int64_t nnz, int nlat_in, int nlon_in,
                                 int nlat_out, int nlon_out, int32_t *blob_out, int64_t blob_ints)
{
    if (!blob_out) return s2attn_fail(S2ATTN_E_INVALID, "plan output buffer is null");
    std::vector<int32_t> blob;
    const int rc = build_blob(col_idx, row_off, nnz, nlat_in, nlon_in, nlat_out, nlon_out, blob);
    if (rc != S2ATTN_OK) return rc;
    if ((int64_t)blob.size() != blob_ints)
        return s2attn_fail(S2ATTN_E_INVALID, "the plan of this CSR has %zu ints, the buffer %lld (size it with s2attn_plan_size)", blob.size(), (long long)blob_ints);
    std::copy(blob.begin(), blob.end(), blob_out);
    return S2ATTN_OK;
}

// Regrouped psi for the ring-step kernels (see include/s2attn.h): a stable counting sort of the CSR entries by the
// latitude named in col, on host arrays like the plan builder.  Entries whose key is outside [key_lo, key_lo + nkeys)
// are left out; t_lat / t_lon need room for nnz entries.  Returns the number of entries written, or a negative error.
extern "C" int64_t s2attn_ring_regroup_psi(const int64_t *col_idx, const int64_t *row_off, int nrows, int modulus, int key_lo, int nkeys,
                                           int32_t *t_lat, int32_t *t_lon, int64_t *t_off, int32_t *t_order)
{
    if (!col_idx || !row_off || !t_lat || !t_lon || !t_off) return s2attn_fail(S2ATTN_E_INVALID, "null array pointer");
    if (nrows < 0 || modulus < 1 || nkeys < 0) return s2attn_fail(S2ATTN_E_INVALID, "nrows and nkeys must not be negative, modulus must be positive");
    const int64_t nnz = row_off[nrows];
    for (int r = 0; r < nrows; r++)
        if (row_off[r] > row_off[r + 1] || row_off[r] < 0) return s2attn_fail(S2ATTN_E_INVALID, "row_off must start at or above 0 and not decrease (row %d)", r);
    auto key_of = [&](int64_t col) -> int64_t { // floor division: a negative col never maps into the window by accident
        const int64_t q = col / modulus;
        return (col % modulus != 0 && col < 0 ? q - 1 : q) - key_lo;
    };
    std::vector<int64_t> count((size_t)nkeys + 1, 0);
    for (int64_t z = 0; z < nnz; z++) {
        const int64_t k = key_of(col_idx[z]);
        if (k >= 0 && k < nkeys) count[(size_t)k + 1]++;
    }
    for (int i = 0; i < nkeys; i++) count[(size_t)i + 1] += count[(size_t)i];
    for (int i = 0; i <= nkeys; i++) t_off[i] = count[(size_t)i];
    std::vector<int64_t> cursor(count.begin(), count.end() - (nkeys >= 0 ? 1 : 0));
    for (int r = 0; r < nrows; r++) {
        for (int64_t z = row_off[r]; z < row_off[r + 1]; z++) {
            const int64_t col = col_idx[z], k = key_of(col);
            if (k < 0 || k >= nkeys) continue;
            const int64_t at = cursor[(size_t)k]++;
            t_lat[at] = r;
            t_lon[at] = (int32_t)(col - (k + key_lo) * modulus);
        }
    }
    if (t_order) { // keys by decreasing number of entries, ties in key order
        std::iota(t_order, t_order + nkeys, 0);
        std::stable_sort(t_order, t_order + nkeys, [&](int32_t a, int32_t b) { return t_off[a + 1] - t_off[a] > t_off[b + 1] - t_off[b]; });
    }
    return t_off[nkeys];
}
