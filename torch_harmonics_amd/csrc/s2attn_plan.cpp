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
    int32_t ho, hi, ws, len; // after decompose(): hi is the virtual latitude (real latitude * ps + parity class)
};

// Splits the CSR into maximal runs of consecutive longitudes inside one input
// latitude, then joins a run that ends at nlon_in-1 with a run of the same
// latitude that starts at 0 into a single circular run.
int decompose(const int64_t *col_idx, const int64_t *row_off, int64_t nnz, int nlat_in, int nlon_in, int nlat_out,
              int nlon_out, std::vector<HostRun> *out, int64_t *count)
{
    if (!col_idx && nnz > 0) return s2attn_fail(S2ATTN_E_INVALID, "col_idx is null");
    if (!row_off) return s2attn_fail(S2ATTN_E_INVALID, "row_off is null");
    if (nlat_in < 1 || nlon_in < 1 || nlat_out < 1 || nlon_out < 1)
        return s2attn_fail(S2ATTN_E_INVALID, "grid extents must be positive");
    if (nlon_in % nlon_out != 0)
        return s2attn_fail(S2ATTN_E_INVALID, "nlon_in (%d) must be an integer multiple of nlon_out (%d)", nlon_in, nlon_out);
    if (row_off[0] != 0 || row_off[nlat_out] != nnz)
        return s2attn_fail(S2ATTN_E_INVALID, "row_off must start at 0 and end at nnz (%lld), got %lld..%lld", (long long)nnz,
                           (long long)row_off[0], (long long)row_off[nlat_out]);

    const int64_t ncol = (int64_t)nlat_in * nlon_in;
    const int ps = nlon_in / nlon_out;
    int64_t total = 0;
    std::vector<HostRun> row;
    for (int ho = 0; ho < nlat_out; ho++) {
        const int64_t z0 = row_off[ho], z1 = row_off[ho + 1];
        if (z1 < z0) return s2attn_fail(S2ATTN_E_INVALID, "row_off decreases at row %d", ho);
        row.clear();
        for (int64_t z = z0; z < z1; z++) {
            const int64_t col = col_idx[z];
            if (col < 0 || col >= ncol)
                return s2attn_fail(S2ATTN_E_INVALID, "col_idx[%lld] = %lld outside [0, %lld)", (long long)z, (long long)col,
                                   (long long)ncol);
            const int32_t hi = (int32_t)(col / nlon_in), wi = (int32_t)(col % nlon_in);
            if (!row.empty() && row.back().hi == hi && row.back().ws + row.back().len == wi && row.back().len < nlon_in) {
                row.back().len++;
            } else {
                row.push_back({ho, hi, wi, 1});
            }
        }
        // circular join inside each group of runs that share a latitude
        size_t i = 0;
        while (i < row.size()) {
            size_t j = i;
            while (j + 1 < row.size() && row[j + 1].hi == row[i].hi) j++;
            if (j > i && row[i].ws == 0 && row[j].ws + row[j].len == nlon_in && row[i].len + row[j].len <= nlon_in) {
                row[j].len += row[i].len;
                row[i].len = 0; // dropped
            }
            i = j + 1;
        }
        // Longitude ratio ps = nlon_in / nlon_out > 1: query wo sees columns ws + t + ps * wo.  Split every run by
        // column parity class: on the sub-lattice {par, par + ps, par + 2 ps, ...} of latitude hi (a "virtual latitude"
        // hi * ps + par with nlon_out columns) the same neighbors are the run (ws', len') with unit stride in wo.
        for (const HostRun &r : row) {
            if (r.len == 0) continue;
            for (int par = 0; par < ps; par++) {
                const int t0 = ((par - r.ws) % ps + ps) % ps; // first neighbor of the run in this class
                if (t0 >= r.len) continue;
                const int first = (r.ws + t0) % nlon_in;
                total++;
                if (out) out->push_back({ho, r.hi * ps + par, (first - par) / ps, (r.len - t0 + ps - 1) / ps});
            }
        }
    }
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

// order: dense latitudes first (most work first), then the others (most work first); returns the dense count
int32_t order_rows(const std::vector<RowCost> &cost, int32_t *order)
{
    const int n = (int)cost.size();
    std::vector<int32_t> dense, vec;
    for (int i = 0; i < n; i++) (cost[i].dense < cost[i].vector ? dense : vec).push_back(i);
    std::stable_sort(dense.begin(), dense.end(), [&](int32_t a, int32_t b) { return cost[a].dense > cost[b].dense; });
    std::stable_sort(vec.begin(), vec.end(), [&](int32_t a, int32_t b) { return cost[a].vector > cost[b].vector; });
    std::copy(dense.begin(), dense.end(), order);
    std::copy(vec.begin(), vec.end(), order + dense.size());
    return (int32_t)dense.size();
}

} // namespace

extern "C" int s2attn_plan_build(const int64_t *col_idx, const int64_t *row_off, int64_t nnz, int nlat_in, int nlon_in,
                                 int nlat_out, int nlon_out, int64_t nruns, int32_t *gather_off, int32_t *gather_runs,
                                 int32_t *gather_order, int32_t *scatter_off, int32_t *scatter_runs, int32_t *scatter_order,
                                 int32_t *ndense)
{
    if (!gather_off || !gather_order || !scatter_off || !scatter_order || !ndense || (nruns > 0 && (!gather_runs || !scatter_runs)))
        return s2attn_fail(S2ATTN_E_INVALID, "plan output array is null");

    std::vector<HostRun> runs;
    int64_t n = 0;
    const int rc = decompose(col_idx, row_off, nnz, nlat_in, nlon_in, nlat_out, nlon_out, &runs, &n);
    if (rc != S2ATTN_OK) return rc;
    if (n != nruns) return s2attn_fail(S2ATTN_E_INVALID, "nruns = %lld does not match the CSR (%lld runs)", (long long)nruns, (long long)n);

    const int ps = nlon_in / nlon_out;
    const int nvlat = nlat_in * ps; // virtual input latitudes

    // gather side: runs are already grouped by ho, in CSR order
    std::vector<RowCost> gcost(nlat_out), scost(nvlat);
    std::fill(gather_off, gather_off + nlat_out + 1, 0);
    for (int64_t i = 0; i < n; i++) {
        const HostRun &r = runs[i];
        gather_runs[4 * i + 0] = r.hi;
        gather_runs[4 * i + 1] = r.ws;
        gather_runs[4 * i + 2] = r.len;
        gather_runs[4 * i + 3] = r.hi / ps; // real latitude: quadrature weight index, row address
        gather_off[r.ho + 1]++;
        gcost[r.ho].add(r.len);
    }
    for (int ho = 0; ho < nlat_out; ho++) gather_off[ho + 1] += gather_off[ho];

    // scatter side: stable counting sort by hi keeps ho ascending inside a group
    std::fill(scatter_off, scatter_off + nvlat + 1, 0);
    for (int64_t i = 0; i < n; i++) scatter_off[runs[i].hi + 1]++;
    for (int hi = 0; hi < nvlat; hi++) scatter_off[hi + 1] += scatter_off[hi];
    std::vector<int32_t> cursor(scatter_off, scatter_off + nvlat);
    for (int64_t i = 0; i < n; i++) {
        const HostRun &r = runs[i];
        const int32_t s = cursor[r.hi]++;
        scatter_runs[4 * s + 0] = r.ho;
        scatter_runs[4 * s + 1] = r.ws;
        scatter_runs[4 * s + 2] = r.len;
        scatter_runs[4 * s + 3] = 0;
        scost[r.hi].add(r.len);
    }

    ndense[0] = order_rows(gcost, gather_order);
    ndense[1] = order_rows(scost, scatter_order);
    return S2ATTN_OK;
}
