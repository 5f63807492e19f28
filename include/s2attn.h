/*
 * s2attn: spherical neighborhood attention (self-attention, down-sampling and up-sampling) for AMD gfx950.
 *
 * Plain C ABI of libs2attn.so.  No torch types cross this boundary: device
 * buffers are raw pointers, sizes are ints, the stream is a hipStream_t passed
 * as void*.  Every entry point returns S2ATTN_OK (0) or a negative S2ATTN_E_*
 * code; s2attn_last_error() returns the message of the last failure on the
 * calling thread.  Nothing here allocates or frees device memory and nothing
 * synchronises the stream.
 *
 * Tensor contract (same as the reference ops, attention_interface.cpp:85-119):
 *   k  [B, nlat_in,  nlon_in,  num_heads*ck]   v  [B, nlat_in,  nlon_in,  num_heads*cv]
 *   q  [B, nlat_out, nlon_out, num_heads*ck]   y, dy [B, nlat_out, nlon_out, num_heads*cv]
 * physical NHWC, contiguous, heads packed along the channel axis, one storage
 * dtype for all activations; quad_weights [nlat_in] fp32; q arrives already
 * multiplied by the softmax scale.  Either nlon_in is a multiple of nlon_out
 * (self-attention and down-sampling, "gather" direction) or nlon_out is a
 * proper multiple of nlon_in (up-sampling, "scatter" direction); the two
 * directions are told apart by the longitude counts, as in the reference
 * (attention.py:337).
 *
 * Accuracy, fp32 storage, against a float64 evaluation of the reference's torch loop (attention_torch.py:97-104): y, dk, dv,
 * dq within rtol = atol = 1e-5 for heads of up to 128 channels and a query that carries the softmax scale.  Measured
 * exceptions: dq on smooth fields (neighboring v almost equal, so the backward's g_j - <dy, y> cancels) lies within
 * atol 2e-5 + rtol 1e-5 (1.6e-5 on values of magnitude 1 at 721 x 1440; the reference's CPU operators are 1.4e-4 from float64
 * on the same tensors); heads wider than 128 channels and unscaled N(0,1) queries are as exact as a plain fp32 CPU evaluation
 * of the same inputs (4.2e-5 absolute on values of magnitude 3 at 512 channels), with dv of the head-dim-32 kernels up to
 * 1.2e-6 beyond 1e-5 on such a query; heads of 64 and more channels with neighborhoods of a few points, one of them dominant:
 * dq up to 5e-6 beyond 1e-5 on values of magnitude 30-70, as far as a plain fp32 CPU evaluation is off there.  16-bit storage (arithmetic in fp32, P and dS enter the
 * matrix instructions in the storage type): fp16 within 2e-2 |x| + 2e-2 RMS per element; bf16 the same on typical problems, single
 * elements of dq (wide heads) and dk (sums over many queries of both signs) up to 0.2 RMS off in a sweep of random problems.
 */
#ifndef S2ATTN_H
#define S2ATTN_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define S2ATTN_OK 0
#define S2ATTN_E_INVALID (-1)     /* bad shape, dtype, null pointer, psi entry out of range */
#define S2ATTN_E_UNSUPPORTED (-2) /* a shape the kernels are not instantiated for */
#define S2ATTN_E_LAUNCH (-3)      /* HIP reported an error at launch */

/* storage dtype of k, v, q, y, dy, dk, dv, dq */
#define S2ATTN_F32 0
#define S2ATTN_BF16 1
#define S2ATTN_F16 2

const char *s2attn_last_error(void);

/* Library version, bumped when the ABI below changes. */
int s2attn_abi_version(void);

/*
 * Neighborhood plan.  The reference kernels walk the CSR neighborhood entry by entry and re-sort its rows by length
 * on every call (attention_cuda_utils.cu:74-113, called from attention_cuda_fwd.cu:476 and attention_cuda_bwd.cu:792).
 *   gather direction:  row_off[nlat_out+1], col = hi*nlon_in + wi: the input points output point (ho, 0) attends to;
 *                      output column wo sees them shifted by (nlon_in/nlon_out)*wo      (attention_torch.py:97-104)
 *   scatter direction: row_off[nlat_in+1],  col = ho*nlon_out + wo: the output points that attend to input point
 *                      (hi, 0); input column wi is seen by them shifted by (nlon_out/nlon_in)*wi (attention_torch.py:613-621)
 * This library converts either CSR once, on the host, into runs of consecutive longitudes:
 *
 *   run = (lat, ws, len, aux)   four int32
 *
 * The longitude ratio ps > 1 is removed in the plan, not in the kernels: every latitude of the FINER grid is split into
 * ps "virtual latitudes" (real latitude * ps + column class par: its columns par, par + ps, ...), each with
 * W = min(nlon_in, nlon_out) columns, and every CSR run into one run per column class it touches.  On virtual latitudes
 * all neighborhoods have unit stride: query column j of virtual output latitude vo sees columns (ws + t + j) mod W of
 * virtual input latitude vi, t in [0, len); that is the only form the kernels implement.  (The coarser grid's virtual
 * latitudes are its real ones; with nlon_in == nlon_out nothing is split.)
 *   nvin = nlat_in * (nlon_in / W),  nvout = nlat_out * (nlon_out / W)
 *
 * gather runs   grouped by virtual output latitude:  lat = virtual input latitude, aux = real input latitude
 * scatter runs  the same runs grouped by virtual input latitude: lat = virtual output latitude, aux = real output latitude;
 *               key column j is seen by query columns (j - ws - t) mod W
 *
 * plus, for each grouping, the group offsets and a launch order of the groups.  The order lists first the
 * latitudes whose runs are long (ndense of them, most work first) and then the others (most work first); starting
 * the longest latitudes first is the load balancing for the ~200:1 spread of row lengths between the poles and
 * the equator.  Any CSR is representable (worst case every entry is its own run).
 *
 * The plan is ONE position-independent array of int32 (the "blob"): a header of S2ATTN_PLAN_HEADER_INTS ints (counts, and
 * the offset in ints of every array inside the blob) followed by the arrays, each starting on a 16-byte boundary:
 *     gather_off  [nvout+1]   gather_runs  [4*nruns]   gather_order  [nvout]   gather_order_mixed  [nvout]
 *     scatter_off [nvin+1]    scatter_runs [4*nruns]   scatter_order [nvin]    scatter_order_mixed [nvin]
 *     *_order_mixed: the same latitudes with the long-run and the short-run ones interleaved in proportion to their work
 *     gather_items  [2*n]  scatter_items [2*n]   work lists of the kernels that put long runs on the matrix cores and short
 *                 runs on the vector ALU (fp32 heads of 32 channels on at least 64 longitudes): (latitude, pair) with
 *                 pair = -1 for a single latitude, else the index of a PAIR of adjacent short-run latitudes (latitude,
 *                 latitude + 1) that one wavefront works together; long-run and short-run units interleaved by work
 *     *_pair_off [npairs+1], *_pair_runs [8 * ...]   merged runs of each pair: (lat, ws, len, aux, dA, lenA, dB, lenB) =
 *                 the union band in the form of a run of that grouping; band position i belongs to the first latitude of
 *                 the pair iff dA <= i < dA + lenA, to the second iff dB <= i < dB + lenB (len < 32)
 *     gather_span [2*nvout]   per virtual output latitude (first column, columns): an arc of the circle that holds every
 *                 neighbor column of query column 0 (of query column j: the arc shifted by j); columns = the whole
 *                 circle when the runs do not fit a shorter arc
 * The builder runs on the host; the caller copies the blob to the device unchanged (it can also be stored and reused:
 * it depends only on the CSR and the four grid extents) and passes the device address with a host copy of the header.
 *
 * s2attn_plan_count   number of runs the CSR decomposes into, or a negative error.
 * s2attn_plan_size    number of int32 in the blob of this CSR, or a negative error.
 * s2attn_plan_build   fills blob_out[blob_ints] (host memory; blob_ints as returned by s2attn_plan_size).
 */
#define S2ATTN_PLAN_HEADER_INTS 32
#define S2ATTN_PLAN_MAGIC 0x53324133 /* "S2A3" */
enum {
    S2ATTN_PH_MAGIC = 0,
    S2ATTN_PH_TOTAL = 1, /* ints in the blob */
    S2ATTN_PH_NVOUT = 2,
    S2ATTN_PH_NVIN = 3,
    S2ATTN_PH_NRUNS = 4,
    S2ATTN_PH_GATHER_NDENSE = 5,  /* leading entries of gather_order that are long-run latitudes */
    S2ATTN_PH_SCATTER_NDENSE = 6, /* the same for scatter_order */
    S2ATTN_PH_GATHER_OFF = 8,
    S2ATTN_PH_GATHER_RUNS = 9,
    S2ATTN_PH_GATHER_ORDER = 10,
    S2ATTN_PH_GATHER_ORDER_MIXED = 11,
    S2ATTN_PH_SCATTER_OFF = 12,
    S2ATTN_PH_SCATTER_RUNS = 13,
    S2ATTN_PH_SCATTER_ORDER = 14,
    S2ATTN_PH_SCATTER_ORDER_MIXED = 15,
    S2ATTN_PH_GATHER_NITEMS = 16,
    S2ATTN_PH_GATHER_ITEMS = 17,
    S2ATTN_PH_GATHER_PAIR_OFF = 18,
    S2ATTN_PH_GATHER_PAIR_RUNS = 19,
    S2ATTN_PH_GATHER_NPAIRS = 20,
    S2ATTN_PH_SCATTER_NITEMS = 21,
    S2ATTN_PH_SCATTER_ITEMS = 22,
    S2ATTN_PH_SCATTER_PAIR_OFF = 23,
    S2ATTN_PH_SCATTER_PAIR_RUNS = 24,
    S2ATTN_PH_SCATTER_NPAIRS = 25,
    S2ATTN_PH_GATHER_SPAN = 26, /* nvout x (first column, columns): an arc holding every neighbor column of query column 0 */
    S2ATTN_PH_NLAT_IN = 28, /* the grid extents the plan was built for: checked against the shape of every call */
    S2ATTN_PH_NLON_IN = 29,
    S2ATTN_PH_NLAT_OUT = 30,
    S2ATTN_PH_NLON_OUT = 31
};

int64_t s2attn_plan_count(const int64_t *col_idx, const int64_t *row_off, int64_t nnz, int nlat_in, int nlon_in, int nlat_out,
                          int nlon_out);

int64_t s2attn_plan_size(const int64_t *col_idx, const int64_t *row_off, int64_t nnz, int nlat_in, int nlon_in, int nlat_out,
                         int nlon_out);

int s2attn_plan_build(const int64_t *col_idx, const int64_t *row_off, int64_t nnz, int nlat_in, int nlon_in, int nlat_out,
                      int nlon_out, int32_t *blob_out, int64_t blob_ints);

typedef struct s2attn_plan {
    const int32_t *data;                     /* device copy of the blob */
    int32_t header[S2ATTN_PLAN_HEADER_INTS]; /* host copy of the blob's first S2ATTN_PLAN_HEADER_INTS ints */
} s2attn_plan;

typedef struct s2attn_shape {
    int batch, num_heads;
    int nlat_in, nlon_in, nlat_out, nlon_out;
    int ck; /* per-head channels of q and k */
    int cv; /* per-head channels of v and y */
    int dtype;
    /* Point strides: elements between two consecutive grid points of a tensor.  0 means packed (num_heads*ck or
     * num_heads*cv, the reference's contract).  A larger value lets a tensor be a column block of a wider row-major buffer:
     * q | k | v written by ONE fused projection GEMM and read in place, dq | dk | dv written into one buffer so that the
     * input gradient is one GEMM (the reference runs three projections, attention.py:530-532).  Latitude and batch strides
     * follow from it (nlon * ld, nlat * nlon * ld).  Strides must be multiples of 4 elements.  Only the kernels for fp32
     * heads of 32 channels on at least 64 longitudes take unpacked tensors; other shapes return S2ATTN_E_UNSUPPORTED.
     * ld_y applies to y (forward output, and the saved output handed to the backward), ld_dy to the upstream gradient. */
    int ld_k, ld_v, ld_q, ld_y, ld_dy, ld_dk, ld_dv, ld_dq;
} s2attn_shape;

/*
 * Forward.  Replaces attention_kernels::forward (attention_interface.cpp:114-116;
 * CUDA implementations s2_attention_fwd_cuda, attention_cuda_fwd.cu:539-633, and the up-sampling
 * kernels of attention_cuda_fwd_upsample.cu:70-289).
 *   y = sum_j a_j v_j / sum_j a_j,  a_j = exp(q.k_j - max) * quad_weights[hi_j]
 * y must not alias an input.
 */
int s2attn_forward(const void *k, const void *v, const void *q, const float *quad_weights, void *y,
                   const s2attn_plan *plan, const s2attn_shape *shape, void *stream);

/*
 * Forward that also returns the softmax statistic lse[B, num_heads, nlat_out, nlon_out] (fp32, log2 of
 * sum_j exp(q.k_j) quad_weights[hi_j], i.e. in the log2 domain the kernels work in) for s2attn_backward_saved.
 * Same reference entry point as s2attn_forward; the reference saves only its inputs for backward
 * (_attention_utils.py:94-100) and recomputes the statistics.
 */
int s2attn_forward_lse(const void *k, const void *v, const void *q, const float *quad_weights, void *y, float *lse,
                       const s2attn_plan *plan, const s2attn_shape *shape, void *stream);

/*
 * Backward.  Replaces attention_kernels::backward (attention_interface.cpp:117-119;
 * CUDA implementation s2_attention_bwd_dkvq_cuda, attention_cuda_bwd.cu:856-956).
 * Writes dk, dv, dq (every element; no pre-zeroing needed, no atomics).
 * workspace: device scratch of s2attn_backward_workspace_bytes(shape) bytes, 8-byte aligned (16 for the matrix-core
 * shapes below): two fp32 softmax statistics per (batch, head, output point), plus, for the shapes whose dq pass works
 * from the forward's output and normaliser (16-bit storage with a head dim that is a multiple of 8 from 16 to 256, fp32 with
 * one that is a multiple of 4 from 16 to 512, ck == cv, at least 32 columns per virtual latitude), room for that output
 * and normaliser, which this entry point first recomputes with the forward kernel.  s2attn_backward_saved and its two
 * halves, which are handed both, need only the statistics: s2attn_backward_saved_workspace_bytes(shape).
 */
int64_t s2attn_backward_saved_workspace_bytes(const s2attn_shape *shape);
int64_t s2attn_backward_workspace_bytes(const s2attn_shape *shape);

int s2attn_backward(const void *k, const void *v, const void *q, const void *dy, const float *quad_weights, void *dk,
                    void *dv, void *dq, void *workspace, const s2attn_plan *plan, const s2attn_shape *shape,
                    void *stream);

/*
 * The two phases of s2attn_backward as separate launches (same arguments, same workspace), for callers that time
 * them individually or need only one side.  Together they replace the same reference entry point as
 * s2attn_backward (attention_cuda_bwd.cu:856-956).
 *   s2attn_backward_dq    writes dq and fills the workspace with the per-query softmax statistics
 *   s2attn_backward_dkdv  reads that workspace (so it must follow s2attn_backward_dq on the stream) and writes dk, dv
 */
int s2attn_backward_dq(const void *k, const void *v, const void *q, const void *dy, const float *quad_weights, void *dq,
                       void *workspace, const s2attn_plan *plan, const s2attn_shape *shape, void *stream);

int s2attn_backward_dkdv(const void *k, const void *v, const void *q, const void *dy, const float *quad_weights,
                         void *dk, void *dv, const void *workspace, const s2attn_plan *plan, const s2attn_shape *shape,
                         void *stream);

/*
 * Backward from saved forward results: y (the forward output) and lse (from s2attn_forward_lse) make the softmax
 * final from the first neighbor on, which saves one of the four matrix products of the dq pass and all running-maximum
 * bookkeeping.  Same outputs as s2attn_backward to rounding; workspace of s2attn_backward_saved_workspace_bytes().  Shapes that run on the vector kernels
 * (other head dims, ck != cv, narrow grids, unaligned tensors) ignore y and lse and take the
 * s2attn_backward path.
 */
int s2attn_backward_saved(const void *k, const void *v, const void *q, const void *dy, const void *y, const float *lse,
                          const float *quad_weights, void *dk, void *dv, void *dq, void *workspace, const s2attn_plan *plan,
                          const s2attn_shape *shape, void *stream);

int s2attn_backward_dq_saved(const void *k, const void *v, const void *q, const void *dy, const void *y, const float *lse,
                             const float *quad_weights, void *dq, void *workspace, const s2attn_plan *plan,
                             const s2attn_shape *shape, void *stream);

/*
 * s2attn_backward_saved for callers that cannot allocate device memory (code under HIP graph capture, tight loops,
 * harnesses that forbid hipMalloc).  It has no counterpart in the reference.  Same arguments and same results as
 * s2attn_backward_saved minus the workspace: the two statistics per (batch, head, output point) live in a device array
 * built into the library, S2ATTN_NOALLOC_SCRATCH_BYTES large (every GPU the library runs on holds its copy until the
 * process ends).  Shapes whose s2attn_backward_saved_workspace_bytes() exceed that return S2ATTN_E_UNSUPPORTED (64 MiB holds
 * 8.3 M output points x heads x batch entries with fp32 heads of 32 channels on wide grids, e.g. 721 x 1440 x 8 heads).
 * Calls no hipMalloc / hipFree.  The first call on a device looks the array's address up (hipGetSymbolAddress): make
 * that call outside a graph capture.  All calls on one GPU share the array: calls that overlap there (two streams, two
 * threads) race; calls on one stream are ordered by the stream.
 */
#define S2ATTN_NOALLOC_SCRATCH_BYTES (64 * 1024 * 1024)

int s2attn_backward_saved_noalloc(const void *k, const void *v, const void *q, const void *dy, const void *y, const float *lse,
                                  const float *quad_weights, void *dk, void *dv, void *dq, const s2attn_plan *plan,
                                  const s2attn_shape *shape, void *stream);

/*
 * Layout conversion.  Replace attention_kernels::permute_to_nhwc / permute_to_nchw
 * (attention_interface.cpp:85-86; CUDA kernels attention_cuda_utils.cuh:417-576).
 * Pure element moves; elem_size is 2, 4 or 8 bytes.  dst must not alias src.
 *   to_nhwc: src [B, C, H, W] -> dst [B, H, W, C]
 *   to_nchw: src [B, H, W, C] -> dst [B, C, H, W]
 */
int s2attn_permute_to_nhwc(const void *src, void *dst, int64_t B, int64_t C, int64_t H, int64_t W, int elem_size,
                           void *stream);
int s2attn_permute_to_nchw(const void *src, void *dst, int64_t B, int64_t H, int64_t W, int64_t C, int elem_size,
                           void *stream);

/*
 * Ring-step variants of the gather direction (nlon_in a multiple of nlon_out): the pieces a longitude-sharded layer is
 * built from.  K/V arrive one longitude chunk at a time (in such a layer the chunks travel around a ring of devices);
 * q, dy and the per-point softmax state stay with the caller.  Each call handles ONE chunk on ONE device and talks to
 * nobody.  Replace attention_kernels::forward_ring_step, backward_ring_step_pass1, backward_ring_step_pass2
 * (attention_interface.cpp:138-156; CUDA: attention_cuda_fwd_ring.cu:66-175, attention_cuda_bwd_ring.cu:78-205 and
 * 1312-1440; caller: torch_harmonics/distributed/distributed_attention.py:141-176, 303-431).
 *
 * Tensors (heads folded into the batch, NHWC, contiguous):
 *   k, v         [batch, nlat_halo, nlon_kx, ck / cv]   the chunk: input latitudes lat_halo_start .. + nlat_halo,
 *                                                      input longitudes lon_lo_kx .. + nlon_kx
 *   q, dy        [batch, nlat_out, nlon_out, ck / cv]   local output points
 *   y_acc        [batch, nlat_out, nlon_out, cv] fp32;  alpha_sum, qdotk_max, integral(_norm) [batch, nlat_out, nlon_out] fp32
 *   alpha_k, alpha_kvw [batch, nlat_out, nlon_out, ck] fp32;   dk, dv: fp32, shaped like k, v (ADDED to; with fp32 atomics
 *                                                      in s2attn_ring_backward_pass2, plainly in ..._pass2_transposed)
 *   quad_weights [global nlat_in] fp32, indexed by global input latitude
 *   col_idx, row_off: the local CSR in device memory, int64: row_off has nlat_out + 1 entries, col_idx = hi_global *
 *     nlon_in + wi with wi already shifted by pscale * (first local output longitude); row_idx (int32, nlat_out entries,
 *     may be null) is the order in which output latitudes are launched.
 * State starts as y_acc = alpha_sum = integral = alpha_k = alpha_kvw = 0, qdotk_max = -inf; after all chunks
 *   y = y_acc / alpha_sum,   dq = (alpha_sum * alpha_kvw - integral * alpha_k) / alpha_sum^2,   integral_norm = integral / alpha_sum.
 * The statistics are in the natural-exponential domain, as the reference's.
 */
typedef struct s2attn_ring_shape {
    int32_t batch;          /* batch * heads */
    int32_t nlat_halo;      /* input latitudes held in the chunk */
    int32_t nlon_kx;        /* input longitudes held in the chunk */
    int32_t nlat_out;       /* local output latitudes */
    int32_t nlon_out;       /* local output longitudes */
    int32_t ck, cv;         /* channels of k/q and of v/y (<= 512) */
    int32_t nlon_in;        /* global input longitudes */
    int32_t pscale;         /* global nlon_in / global nlon_out */
    int32_t lon_lo_kx;      /* first global input longitude of the chunk */
    int32_t lat_halo_start; /* first global input latitude of the chunk */
    int32_t dtype;          /* S2ATTN_F32 / BF16 / F16: storage of k, v, q, dy */
} s2attn_ring_shape;

int s2attn_ring_forward_step(const void *k, const void *v, const void *q, float *y_acc, float *alpha_sum, float *qdotk_max,
                             const float *quad_weights, const int64_t *col_idx, const int64_t *row_off, const int32_t *row_idx,
                             const s2attn_ring_shape *shape, void *stream);

int s2attn_ring_backward_pass1(const void *k, const void *v, const void *q, const void *dy, float *alpha_sum, float *qdotk_max,
                               float *integral, float *alpha_k, float *alpha_kvw, const float *quad_weights,
                               const int64_t *col_idx, const int64_t *row_off, const int32_t *row_idx,
                               const s2attn_ring_shape *shape, void *stream);

int s2attn_ring_backward_pass2(const void *k, const void *v, const void *q, const void *dy, const float *alpha_sum,
                               const float *qdotk_max, const float *integral_norm, float *dk, float *dv,
                               const float *quad_weights, const int64_t *col_idx, const int64_t *row_off,
                               const int32_t *row_idx, const s2attn_ring_shape *shape, void *stream);

/*
 * s2attn_ring_forward_step and s2attn_ring_backward_pass1 / pass2 on the band-staged matrix-core kernels (same reference operators,
 * attention_interface.cpp:138-156, attention_cuda_fwd_ring.cu:66-175, attention_cuda_bwd_ring.cu:78-205; same tensors and
 * state, same results up to the order of the fp32 sums): instead of the CSR they take the run-length plan of the LOCAL psi,
 * built once per psi by s2attn_plan_build(col_idx, row_off, nnz, nlat_in = global input latitudes, nlon_in, nlat_out =
 * local output latitudes, nlon_out = nlon_in / pscale) on host copies of the same col_idx / row_off.  A row of a staged
 * band is one input longitude, so the chunk clips rows of the band and the kernels walk only the steps of each run that
 * hold a longitude of the chunk.  Shapes: ck == cv a multiple of 4 from 16 to 128, nlon_in / pscale >= 32, k, v, q, dy
 * of any storage dtype aligned to four channels (16 bytes fp32, 8 bytes bf16 / fp16: 16-bit rows are widened as they are
 * staged, so tiles, matrix instructions and state are fp32 whatever the storage), state and dk, dv fp32 and 16-byte
 * aligned; anything else returns S2ATTN_E_UNSUPPORTED and the caller uses the entry points above.
 * Pass 1 re-accumulates alpha_sum and qdotk_max with the forward step's operations in the forward step's order: fed the
 * same chunks in the same order the two alpha_sum are bit-identical, which the dq formula above (the forward's alpha_sum
 * with pass 1's other sums, as the reference combines them) relies on for wide heads - use the two together.
 */
int s2attn_ring_forward_step_plan(const void *k, const void *v, const void *q, float *y_acc, float *alpha_sum, float *qdotk_max,
                                  const float *quad_weights, const s2attn_plan *plan, const s2attn_ring_shape *shape, void *stream);

int s2attn_ring_backward_pass1_plan(const void *k, const void *v, const void *q, const void *dy, float *alpha_sum, float *qdotk_max,
                                    float *integral, float *alpha_k, float *alpha_kvw, const float *quad_weights,
                                    const s2attn_plan *plan, const s2attn_ring_shape *shape, void *stream);

/* s2attn_ring_backward_pass2 likewise (attention_interface.cpp:151-156, attention_cuda_bwd_ring.cu:1312-1440): a wavefront owns 16
 * keys of the chunk and gathers over the plan's runs grouped by input latitude; dk, dv are added to plainly (no atomics). */
int s2attn_ring_backward_pass2_plan(const void *k, const void *v, const void *q, const void *dy, const float *alpha_sum,
                                    const float *qdotk_max, const float *integral_norm, float *dk, float *dv,
                                    const float *quad_weights, const s2attn_plan *plan, const s2attn_ring_shape *shape, void *stream);

/*
 * Regrouped psi.  Every ring kernel of this library is a gather: the cell that owns a sum walks the entries of its own
 * latitude.  Where psi is keyed by the other grid, the caller supplies, once per psi, the CSR entries regrouped by
 * the owner's latitude -- a STABLE sort of the entries (row r, col) by key = col / modulus:
 *   t_off[i]  (int64, nkeys + 1 entries)  entries of key key_lo + i are t_off[i] .. t_off[i + 1] - 1, in CSR order
 *   t_lat[z]  (int32)                     the entry's CSR row r (the partner's local latitude)
 *   t_lon[z]  (int32)                     col mod modulus
 * Keys outside [key_lo, key_lo + nkeys) are left out.  The Python operators build these arrays with device operations
 * and cache them per psi; s2attn_ring_regroup_psi does the same on HOST arrays (like s2attn_plan_build: the caller copies
 * the results to the device): t_lat, t_lon with room for row_off[nrows] entries, t_off [nkeys + 1], t_order [nkeys] (may
 * be null) = the keys by decreasing number of entries, the row_order argument of the pass 2 entry points.  Returns the
 * number of entries written or a negative error.
 *
 * Backward pass 2 of the gather direction on the regrouped psi (modulus nlon_in, key_lo = lat_halo_start, nkeys =
 * nlat_halo; t_lat = local output latitude): the same dk, dv as s2attn_ring_backward_pass2
 * (attention_cuda_bwd_ring.cu:1312-1440), summed per chunk point in a fixed order and added to dk, dv without atomics.
 * row_order (here and in s2attn_ring_backward_pass2_upsample; may be null) lists the nlat_halo chunk latitudes in the
 * order to launch them, the ones with the most entries first, which keeps the end of the launch busy.
 */
int64_t s2attn_ring_regroup_psi(const int64_t *col_idx, const int64_t *row_off, int nrows, int modulus, int key_lo, int nkeys,
                                int32_t *t_lat, int32_t *t_lon, int64_t *t_off, int32_t *t_order);

int s2attn_ring_backward_pass2_transposed(const void *k, const void *v, const void *q, const void *dy, const float *alpha_sum,
                                          const float *qdotk_max, const float *integral_norm, float *dk, float *dv,
                                          const float *quad_weights, const int32_t *t_lat, const int32_t *t_lon,
                                          const int64_t *t_off, const int32_t *row_order, const s2attn_ring_shape *shape,
                                          void *stream);

/*
 * The same three steps for the up-sampling (scatter) direction, nlon_out a multiple of nlon_in.  Replace
 * attention_kernels::forward_ring_step_upsample, backward_ring_step_upsample_pass1 / _pass2
 * (attention_interface.cpp:158-189; CUDA: attention_cuda_fwd_ring_upsample.cu:108-300,
 * attention_cuda_bwd_ring_upsample.cu:88-240).  psi is keyed by the chunk's LOCAL input latitude: row_off has
 * nlat_halo + 1 entries (empty rows for pole padding), col_idx = ho_local * nlon_out_global + wo_shifted with
 * wo_shifted = (wo - first local output longitude) mod nlon_out_global.  The reference's forward scatters in three
 * phases (maxima, rescale, sums) with atomics; here the forward step and pass 1 gather per OUTPUT cell over psi regrouped
 * by output latitude (modulus nlon_out_global, key_lo = 0, nkeys = nlat_out; t_lat = local input latitude), with the
 * running maximum kept per cell: same state after every step, no scratch, no atomics.  Pass 1 needs the forward's FINAL
 * qdotk_max and adds into integral, alpha_k, alpha_kvw; pass 2 takes psi as given and WRITES the chunk's dk and dv
 * (every element).
 */
typedef struct s2attn_ring_up_shape {
    int32_t batch, nlat_halo, nlon_kx, nlat_out, nlon_out; /* as s2attn_ring_shape; nlon_out is the LOCAL output width */
    int32_t ck, cv;
    int32_t nlon_out_global; /* global output longitudes */
    int32_t pscale_out;      /* global nlon_out / global nlon_in */
    int32_t lon_lo_kx;       /* first global input longitude of the chunk */
    int32_t lat_halo_start;  /* global input latitude of the chunk's row 0 (quadrature weight index; may be negative when
                                the halo is padded past the pole: such rows must be empty in psi) */
    int32_t dtype;
} s2attn_ring_up_shape;

int s2attn_ring_forward_step_upsample(const void *k, const void *v, const void *q, float *y_acc, float *alpha_sum, float *qdotk_max,
                                      const float *quad_weights, const int32_t *t_lat, const int32_t *t_lon, const int64_t *t_off,
                                      const s2attn_ring_up_shape *shape, void *stream);

int s2attn_ring_backward_pass1_upsample(const void *k, const void *v, const void *q, const void *dy, const float *qdotk_max,
                                        float *integral, float *alpha_k, float *alpha_kvw, const float *quad_weights,
                                        const int32_t *t_lat, const int32_t *t_lon, const int64_t *t_off,
                                        const s2attn_ring_up_shape *shape, void *stream);

int s2attn_ring_backward_pass2_upsample(const void *k, const void *v, const void *q, const void *dy, const float *alpha_sum,
                                        const float *qdotk_max, const float *integral_norm, float *dk, float *dv,
                                        const float *quad_weights, const int64_t *col_idx, const int64_t *row_off,
                                        const int32_t *row_order, const s2attn_ring_up_shape *shape, void *stream);

/*
 * The three up-sampling steps on the band-staged matrix-core kernels (same operators, same tensors and state): they take the
 * run-length plan of the local psi, built once per psi by s2attn_plan_build(col_idx, row_off, nnz, nlat_in = nlat_halo (the
 * chunk's rows, pole padding included), nlon_in, nlat_out = local output latitudes, nlon_out = nlon_out_global) on host
 * copies of the same col_idx / row_off.  Shapes as for the gather direction: any storage dtype, ck == cv a multiple of 4 from 16
 * to 128, nlon_in >= 32, tensors aligned to four channels; anything else returns S2ATTN_E_UNSUPPORTED.  (Pass 1 of this direction
 * works from the forward's final maximum, so its sums and the forward's alpha_sum are rounded differently whatever the
 * kernels; the dq formula amplifies that by |alpha_kvw| / alpha_sum, which grows with the head width: 3.5e-5 on values of
 * magnitude 1 at 128 channels.  The Python operators therefore take these entry points up to 64 channels.)
 */
int s2attn_ring_forward_step_upsample_plan(const void *k, const void *v, const void *q, float *y_acc, float *alpha_sum, float *qdotk_max,
                                           const float *quad_weights, const s2attn_plan *plan, const s2attn_ring_up_shape *shape, void *stream);

int s2attn_ring_backward_pass1_upsample_plan(const void *k, const void *v, const void *q, const void *dy, const float *qdotk_max,
                                             float *integral, float *alpha_k, float *alpha_kvw, const float *quad_weights,
                                             const s2attn_plan *plan, const s2attn_ring_up_shape *shape, void *stream);

int s2attn_ring_backward_pass2_upsample_plan(const void *k, const void *v, const void *q, const void *dy, const float *alpha_sum,
                                             const float *qdotk_max, const float *integral_norm, float *dk, float *dv,
                                             const float *quad_weights, const s2attn_plan *plan, const s2attn_ring_up_shape *shape, void *stream);

#ifdef __cplusplus
}
#endif

#endif /* S2ATTN_H */
