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

extern "C" int64_t s2attn_plan_count(const int64_t *col_idx, const int64_t *row_off, int64_t nnz, int nlat_in, int nlon_in,
                                     int nlat_out, int nlon_out)
{
    int64_t n = 0;
    const int rc = decompose(col_idx, row_off, nnz, nlat_in, nlon_in, nlat_out, nlon_out, nullptr, &n);
    return rc == S2ATTN_OK ? n : (int64_t)rc;
}

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
// mixed (may be null): the same two lists merged so that at every point of the launch about the same share of each list's
// work has been handed out.  The kernels that treat long runs on the matrix cores and short runs on the vector ALU take this
// order: their matrix-core-heavy and vector-heavy workgroups then sit side by side on a SIMD for the whole launch instead
// of one kind after the other (measured 6-7 % on 721x1440 grids); the kernels that put every run on the matrix cores
// lose 8-35 % with it (their long rows must start first) and keep `order`.
int cost_class(int64_t c)
{
    int cls = 0;
    while ((c >> cls) > 15) cls++; // c = m * 2^cls, 8 <= m < 16
    return c <= 0 ? -1 : cls * 8 + (int)((c >> cls) - 8);
}
int32_t order_rows(const std::vector<RowCost> &cost, int32_t *order, int32_t *mixed)
{
    const int n = (int)cost.size();
    std::vector<int32_t> dense, vec;
    for (int i = 0; i < n; i++) (cost[i].dense < cost[i].vector ? dense : vec).push_back(i);
    std::stable_sort(dense.begin(), dense.end(), [&](int32_t a, int32_t b) { return cost_class(cost[a].dense) > cost_class(cost[b].dense); });
    std::stable_sort(vec.begin(), vec.end(), [&](int32_t a, int32_t b) { return cost_class(cost[a].vector) > cost_class(cost[b].vector); });
    std::copy(dense.begin(), dense.end(), order);
    std::copy(vec.begin(), vec.end(), order + dense.size());
    if (!mixed) return (int32_t)dense.size();
    double wd = 0, wv = 0;
    for (int32_t r : dense) wd += (double)cost[r].dense;
    for (int32_t r : vec) wv += (double)cost[r].vector;
    size_t i = 0, j = 0;
    double cd = 0, cv = 0;
    int32_t *out = mixed;
    while (i < dense.size() || j < vec.size()) {
        // the long-run list is held back a little (its share of work handed out <= 0.7 of the other's): measured best
        // between 0.5 and 0.8, 1.5-2 % of the step over equal shares
        const bool take_dense = j >= vec.size() || (i < dense.size() && cd * wv <= 0.7 * cv * wd);
        if (take_dense) {
            cd += (double)cost[dense[i]].dense;
            *out++ = dense[i++];
        } else {
            cv += (double)cost[vec[j]].vector;
            *out++ = vec[j++];
        }
    }
    return (int32_t)dense.size();
}

} // namespace

extern "C" int s2attn_plan_build(const int64_t *col_idx, const int64_t *row_off, int64_t nnz, int nlat_in, int nlon_in,
                                 int nlat_out, int nlon_out, int64_t nruns, int32_t *gather_off, int32_t *gather_runs,
                                 int32_t *gather_order, int32_t *scatter_off, int32_t *scatter_runs, int32_t *scatter_order,
                                 int32_t *ndense, int32_t *gather_order_mixed, int32_t *scatter_order_mixed)
{
    if (!gather_off || !gather_order || !scatter_off || !scatter_order || !ndense || (nruns > 0 && (!gather_runs || !scatter_runs)))
        return s2attn_fail(S2ATTN_E_INVALID, "plan output array is null");

    std::vector<HostRun> runs;
    int64_t n = 0;
    const int rc = decompose(col_idx, row_off, nnz, nlat_in, nlon_in, nlat_out, nlon_out, &runs, &n);
    if (rc != S2ATTN_OK) return rc;
    if (n != nruns) return s2attn_fail(S2ATTN_E_INVALID, "nruns = %lld does not match the CSR (%lld runs)", (long long)nruns, (long long)n);

    const bool up = nlon_out % nlon_in == 0 && nlon_out != nlon_in;
    const int psk = up ? 1 : nlon_in / nlon_out, psq = up ? nlon_out / nlon_in : 1;
    const int nvin = nlat_in * psk, nvout = nlat_out * psq; // virtual latitudes

    // both groupings by stable counting sort (entries keep the CSR's order inside a group)
    std::vector<RowCost> gcost(nvout), scost(nvin);
    std::fill(gather_off, gather_off + nvout + 1, 0);
    std::fill(scatter_off, scatter_off + nvin + 1, 0);
    for (int64_t i = 0; i < n; i++) {
        gather_off[runs[i].ho + 1]++;
        scatter_off[runs[i].hi + 1]++;
    }
    for (int r = 0; r < nvout; r++) gather_off[r + 1] += gather_off[r];
    for (int r = 0; r < nvin; r++) scatter_off[r + 1] += scatter_off[r];
    std::vector<int32_t> gcur(gather_off, gather_off + nvout), scur(scatter_off, scatter_off + nvin);
    for (int64_t i = 0; i < n; i++) {
        const HostRun &r = runs[i];
        const int32_t g = gcur[r.ho]++, sidx = scur[r.hi]++;
        gather_runs[4 * g + 0] = r.hi;
        gather_runs[4 * g + 1] = r.ws;
        gather_runs[4 * g + 2] = r.len;
        gather_runs[4 * g + 3] = r.hi / psk; // real input latitude: quadrature weight index, row address
        scatter_runs[4 * sidx + 0] = r.ho;
        scatter_runs[4 * sidx + 1] = r.ws;
        scatter_runs[4 * sidx + 2] = r.len;
        scatter_runs[4 * sidx + 3] = r.ho / psq; // real output latitude: row address
        gcost[r.ho].add(r.len);
        scost[r.hi].add(r.len);
    }

    ndense[0] = order_rows(gcost, gather_order, gather_order_mixed);
    ndense[1] = order_rows(scost, scatter_order, scatter_order_mixed);
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
