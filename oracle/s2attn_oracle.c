/*
 * CPU oracle for spherical neighborhood attention (gather direction).
 *
 * TEST INFRASTRUCTURE ONLY.  Nothing in the shipped package may link, load or
 * call this file; it exists so the HIP path can be checked against an
 * independent CPU restatement of the reference algorithm, and so that the
 * reference's CPU algorithm can be timed as a baseline.
 *
 * Two families of functions:
 *
 *  s2o_fwd_f32 / s2o_bwd_f32
 *      fp32 restatements of the reference's OpenMP CPU kernels
 *        torch_harmonics/attention/optimized/kernels_cpu/attention_cpu_fwd.h:63-204
 *        torch_harmonics/attention/optimized/kernels_cpu/attention_cpu_bwd.h:75-347
 *      (same loop nests, same online-softmax update, same three backward
 *      phases with their per-cell scratch and filtered psi rescans).  The
 *      reference folds heads into the batch with a copy
 *      (attention_cpu_fwd.cpp:48-62); here a head is addressed in place inside
 *      the packed NHWC tensor, which changes no arithmetic.
 *
 *  s2o_fwd_f64 / s2o_bwd_f64
 *      double-precision statement of the semantic spec
 *        torch_harmonics/attention/kernels_torch/attention_torch.py:74-125  (forward)
 *        torch_harmonics/attention/kernels_torch/attention_torch.py:130-206 (dv)
 *        torch_harmonics/attention/kernels_torch/attention_torch.py:211-301 (dk)
 *        torch_harmonics/attention/kernels_torch/attention_torch.py:306-390 (dq)
 *      evaluated per query with a two-pass softmax.  It takes fp32 tensors,
 *      accumulates in double and can be restricted to a range of output
 *      latitudes so that large grids can be sampled.
 *
 * Parity pins (tests/test_oracle.py): both families are checked against a dense
 * masked softmax evaluated by torch in float64 with autograd, against
 * F.scaled_dot_product_attention for a cutoff covering the sphere, against the
 * closed forms (constant v, single-neighbor rows, longitude-roll equivariance)
 * and against the committed vectors in tests/golden/.  On top of those, both
 * families are held against the reference's OWN CPU operators: its CPU sources
 * compiled by `make -C oracle ref` and run on the same seeded inputs
 * (tests/test_oracle_reference.py, where that build exists), and their outputs
 * committed as vectors (tests/golden/reference_cpu/, tests/test_golden_reference.py).
 *
 * Tensor layout everywhere: physical NHWC with heads packed along channels,
 *   k : [B, Hi, Wi, nh*Ck]   v : [B, Hi, Wi, nh*Cv]
 *   q : [B, Ho, Wo, nh*Ck]   y, dy : [B, Ho, Wo, nh*Cv]
 * psi: row_off[Ho+1], col_idx[nnz] with col = hi*Wi + wi for output longitude 0;
 * for output longitude wo the input longitude is (wi + pscale*wo) mod Wi,
 * pscale = Wi / Wo.
 */

#include <float.h>
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#define S2O_WO_BLOCK 64

static inline int64_t imin64(int64_t a, int64_t b) { return a < b ? a : b; }

/* ------------------------------------------------------------------------- */
/* fp32 forward: attention_cpu_fwd.h:63-204                                    */
/* ------------------------------------------------------------------------- */
void s2o_fwd_f32(const float *kx, const float *vx, const float *qy, const float *quad_w, const int64_t *col_idx,
                 const int64_t *row_off, float *y, int64_t B, int64_t nh, int64_t Hi, int64_t Wi, int64_t Ho,
                 int64_t Wo, int64_t Ck, int64_t Cv)
{
    const int64_t pscale = Wi / Wo;
    const int64_t nblk = (Wo + S2O_WO_BLOCK - 1) / S2O_WO_BLOCK;
    const int64_t ldk = nh * Ck, ldv = nh * Cv;
    const int64_t BH = B * nh;

#pragma omp parallel
    {
        float *acc = (float *)malloc(sizeof(float) * S2O_WO_BLOCK * Cv);

#pragma omp for collapse(3) schedule(static)
        for (int64_t bh = 0; bh < BH; bh++) {
            for (int64_t ho = 0; ho < Ho; ho++) {
                for (int64_t blk = 0; blk < nblk; blk++) {
                    const int64_t b = bh / nh, h = bh % nh;
                    const int64_t w0 = blk * S2O_WO_BLOCK;
                    const int64_t w1 = imin64(Wo, w0 + S2O_WO_BLOCK);
                    const int64_t nw = w1 - w0;

                    float asum[S2O_WO_BLOCK];
                    float smax[S2O_WO_BLOCK];
                    for (int64_t i = 0; i < nw; i++) {
                        asum[i] = 0.0f;
                        smax[i] = -FLT_MAX;
                    }
                    memset(acc, 0, sizeof(float) * nw * Cv);

                    const float *q_row = qy + ((b * Ho + ho) * Wo) * ldk + h * Ck;
                    const float *k_b = kx + (b * Hi * Wi) * ldk + h * Ck;
                    const float *v_b = vx + (b * Hi * Wi) * ldv + h * Cv;

                    for (int64_t z = row_off[ho]; z < row_off[ho + 1]; z++) {
                        const int64_t col = col_idx[z];
                        const int64_t hi = col / Wi;
                        const int64_t wi = col % Wi;
                        const float wq = quad_w[hi];
                        int64_t wip = (wi + pscale * w0) % Wi;

                        for (int64_t wo = w0; wo < w1; wo++) {
                            const int64_t i = wo - w0;
                            const float *qp = q_row + wo * ldk;
                            const float *kp = k_b + (hi * Wi + wip) * ldk;
                            const float *vp = v_b + (hi * Wi + wip) * ldv;

                            float s = 0.0f;
                            for (int64_t c = 0; c < Ck; c++) s += qp[c] * kp[c];

                            const float mnew = smax[i] > s ? smax[i] : s;
                            const float disc = expf(smax[i] - mnew);
                            const float a = expf(s - mnew) * wq;
                            asum[i] = a + asum[i] * disc;

                            float *ap = acc + i * Cv;
                            for (int64_t c = 0; c < Cv; c++) ap[c] = ap[c] * disc + a * vp[c];

                            smax[i] = mnew;
                            wip += pscale;
                            if (wip >= Wi) wip -= Wi;
                        }
                    }

                    for (int64_t wo = w0; wo < w1; wo++) {
                        const int64_t i = wo - w0;
                        const float inv = 1.0f / asum[i];
                        float *yp = y + ((b * Ho + ho) * Wo + wo) * ldv + h * Cv;
                        const float *ap = acc + i * Cv;
                        for (int64_t c = 0; c < Cv; c++) yp[c] = ap[c] * inv;
                    }
                }
            }
        }
        free(acc);
    }
}

/* ------------------------------------------------------------------------- */
/* fp32 backward: attention_cpu_bwd.h:75-347                                   */
/*   phase A  per (bh, ho, wo): two-pass softmax, cache alpha and <dy,v> per   */
/*            neighbor plus their sums                       (bwd.h:119-216)  */
/*   phase B  per (bh, ci): for every input latitude rescan psi, accumulate a  */
/*            dk row and a persistent dq plane               (bwd.h:218-295)  */
/*   phase C  per (bh, co): same scan for dv                 (bwd.h:297-346)  */
/* Scratch is 2*BH*Ho*Wo*max_row_len floats; returns 1 when that cannot be     */
/* allocated (the reference would throw std::bad_alloc), 0 on success.         */
/* dk, dv, dq must be zero-filled by the caller (the reference allocates       */
/* zeros, attention_cpu_bwd.cpp:104-106).                                      */
/* ------------------------------------------------------------------------- */
int s2o_bwd_f32(const float *kx, const float *vx, const float *qy, const float *dy, const float *quad_w,
                const int64_t *col_idx, const int64_t *row_off, float *dk, float *dv, float *dq, int64_t B,
                int64_t nh, int64_t Hi, int64_t Wi, int64_t Ho, int64_t Wo, int64_t Ck, int64_t Cv)
{
    const int64_t pscale = Wi / Wo;
    const int64_t ldk = nh * Ck, ldv = nh * Cv;
    const int64_t BH = B * nh;

    int64_t max_len = 0;
    for (int64_t ho = 0; ho < Ho; ho++) {
        const int64_t len = row_off[ho + 1] - row_off[ho];
        if (len > max_len) max_len = len;
    }

    const int64_t ncell = BH * Ho * Wo;
    float *alpha_nz = (float *)malloc(sizeof(float) * (size_t)(ncell * max_len + 1));
    float *gdotv_nz = (float *)malloc(sizeof(float) * (size_t)(ncell * max_len + 1));
    float *alpha_sum = (float *)malloc(sizeof(float) * (size_t)(ncell + 1));
    float *alpha_gv = (float *)malloc(sizeof(float) * (size_t)(ncell + 1));
    if (!alpha_nz || !gdotv_nz || !alpha_sum || !alpha_gv) {
        free(alpha_nz);
        free(gdotv_nz);
        free(alpha_sum);
        free(alpha_gv);
        return 1;
    }

    /* ---- phase A ---- */
#pragma omp parallel
    {
        float *sc = (float *)malloc(sizeof(float) * (size_t)(max_len + 1));

#pragma omp for collapse(3) schedule(static)
        for (int64_t bh = 0; bh < BH; bh++) {
            for (int64_t ho = 0; ho < Ho; ho++) {
                for (int64_t wo = 0; wo < Wo; wo++) {
                    const int64_t b = bh / nh, h = bh % nh;
                    const int64_t cell = (bh * Ho + ho) * Wo + wo;
                    const int64_t z0 = row_off[ho], z1 = row_off[ho + 1];
                    float *a_nz = alpha_nz + cell * max_len;
                    float *g_nz = gdotv_nz + cell * max_len;
                    const float *qp = qy + ((b * Ho + ho) * Wo + wo) * ldk + h * Ck;
                    const float *gp = dy + ((b * Ho + ho) * Wo + wo) * ldv + h * Cv;

                    float smax = -FLT_MAX;
                    for (int64_t z = z0; z < z1; z++) {
                        const int64_t col = col_idx[z];
                        const int64_t hi = col / Wi;
                        int64_t wip = col % Wi + pscale * wo;
                        if (wip >= Wi) wip -= Wi;
                        const float *kp = kx + ((b * Hi + hi) * Wi + wip) * ldk + h * Ck;
                        float s = 0.0f;
                        for (int64_t c = 0; c < Ck; c++) s += qp[c] * kp[c];
                        sc[z - z0] = s;
                        if (s > smax) smax = s;
                    }

                    float asum = 0.0f, agv = 0.0f;
                    for (int64_t z = z0; z < z1; z++) {
                        const int64_t col = col_idx[z];
                        const int64_t hi = col / Wi;
                        int64_t wip = col % Wi + pscale * wo;
                        if (wip >= Wi) wip -= Wi;
                        const float *vp = vx + ((b * Hi + hi) * Wi + wip) * ldv + h * Cv;
                        const float a = expf(sc[z - z0] - smax) * quad_w[hi];
                        float g = 0.0f;
                        for (int64_t c = 0; c < Cv; c++) g += gp[c] * vp[c];
                        a_nz[z - z0] = a;
                        g_nz[z - z0] = g;
                        asum += a;
                        agv += a * g;
                    }
                    alpha_sum[cell] = asum;
                    alpha_gv[cell] = agv;
                }
            }
        }
        free(sc);
    }

    /* ---- phase B: dq and dk ---- */
#pragma omp parallel
    {
        float *dq_plane = (float *)malloc(sizeof(float) * (size_t)(Ho * Wo));
        float *dk_row = (float *)malloc(sizeof(float) * (size_t)Wi);

#pragma omp for collapse(2) schedule(static)
        for (int64_t bh = 0; bh < BH; bh++) {
            for (int64_t ci = 0; ci < Ck; ci++) {
                const int64_t b = bh / nh, h = bh % nh;
                memset(dq_plane, 0, sizeof(float) * (size_t)(Ho * Wo));

                for (int64_t hi = 0; hi < Hi; hi++) {
                    memset(dk_row, 0, sizeof(float) * (size_t)Wi);

                    for (int64_t ho = 0; ho < Ho; ho++) {
                        const int64_t z0 = row_off[ho], z1 = row_off[ho + 1];
                        for (int64_t z = z0; z < z1; z++) {
                            const int64_t col = col_idx[z];
                            if (col / Wi != hi) continue;
                            const int64_t wi = col % Wi;
                            for (int64_t wo = 0; wo < Wo; wo++) {
                                int64_t wip = wi + pscale * wo;
                                if (wip >= Wi) wip -= Wi;
                                const int64_t cell = (bh * Ho + ho) * Wo + wo;
                                const float a = alpha_nz[cell * max_len + (z - z0)];
                                const float g = gdotv_nz[cell * max_len + (z - z0)];
                                const float inv = 1.0f / alpha_sum[cell];
                                const float mean_g = alpha_gv[cell] * inv;
                                const float wgt = a * inv * (g - mean_g);
                                const float kval = kx[((b * Hi + hi) * Wi + wip) * ldk + h * Ck + ci];
                                const float qval = qy[((b * Ho + ho) * Wo + wo) * ldk + h * Ck + ci];
                                dk_row[wip] += qval * wgt;
                                dq_plane[ho * Wo + wo] += kval * wgt;
                            }
                        }
                    }
                    for (int64_t w = 0; w < Wi; w++) dk[((b * Hi + hi) * Wi + w) * ldk + h * Ck + ci] += dk_row[w];
                }
                for (int64_t ho = 0; ho < Ho; ho++)
                    for (int64_t wo = 0; wo < Wo; wo++)
                        dq[((b * Ho + ho) * Wo + wo) * ldk + h * Ck + ci] += dq_plane[ho * Wo + wo];
            }
        }
        free(dq_plane);
        free(dk_row);
    }

    /* ---- phase C: dv ---- */
#pragma omp parallel
    {
        float *dv_row = (float *)malloc(sizeof(float) * (size_t)Wi);

#pragma omp for collapse(2) schedule(static)
        for (int64_t bh = 0; bh < BH; bh++) {
            for (int64_t co = 0; co < Cv; co++) {
                const int64_t b = bh / nh, h = bh % nh;
                for (int64_t hi = 0; hi < Hi; hi++) {
                    memset(dv_row, 0, sizeof(float) * (size_t)Wi);
                    for (int64_t ho = 0; ho < Ho; ho++) {
                        const int64_t z0 = row_off[ho], z1 = row_off[ho + 1];
                        for (int64_t z = z0; z < z1; z++) {
                            const int64_t col = col_idx[z];
                            if (col / Wi != hi) continue;
                            const int64_t wi = col % Wi;
                            for (int64_t wo = 0; wo < Wo; wo++) {
                                int64_t wip = wi + pscale * wo;
                                if (wip >= Wi) wip -= Wi;
                                const int64_t cell = (bh * Ho + ho) * Wo + wo;
                                const float p = alpha_nz[cell * max_len + (z - z0)] * (1.0f / alpha_sum[cell]);
                                dv_row[wip] += p * dy[((b * Ho + ho) * Wo + wo) * ldv + h * Cv + co];
                            }
                        }
                    }
                    for (int64_t w = 0; w < Wi; w++) dv[((b * Hi + hi) * Wi + w) * ldv + h * Cv + co] += dv_row[w];
                }
            }
        }
        free(dv_row);
    }

    free(alpha_nz);
    free(gdotv_nz);
    free(alpha_sum);
    free(alpha_gv);
    return 0;
}

/* ------------------------------------------------------------------------- */
/* float64 spec, forward: attention_torch.py:74-125.                           */
/* Output rows ho in [ho_lo, ho_hi) only; other rows of y are left untouched.  */
/* ------------------------------------------------------------------------- */
void s2o_fwd_f64(const float *kx, const float *vx, const float *qy, const float *quad_w, const int64_t *col_idx,
                 const int64_t *row_off, double *y, int64_t B, int64_t nh, int64_t Hi, int64_t Wi, int64_t Ho,
                 int64_t Wo, int64_t Ck, int64_t Cv, int64_t ho_lo, int64_t ho_hi)
{
    const int64_t pscale = Wi / Wo;
    const int64_t ldk = nh * Ck, ldv = nh * Cv;
    const int64_t BH = B * nh;

    int64_t max_len = 0;
    for (int64_t ho = ho_lo; ho < ho_hi; ho++) {
        const int64_t len = row_off[ho + 1] - row_off[ho];
        if (len > max_len) max_len = len;
    }

#pragma omp parallel
    {
        double *sc = (double *)malloc(sizeof(double) * (size_t)(max_len + 1));
        double *acc = (double *)malloc(sizeof(double) * (size_t)(Cv + 1));

#pragma omp for collapse(3) schedule(dynamic, 16)
        for (int64_t bh = 0; bh < BH; bh++) {
            for (int64_t ho = ho_lo; ho < ho_hi; ho++) {
                for (int64_t wo = 0; wo < Wo; wo++) {
                    const int64_t b = bh / nh, h = bh % nh;
                    const int64_t z0 = row_off[ho], z1 = row_off[ho + 1];
                    const float *qp = qy + ((b * Ho + ho) * Wo + wo) * ldk + h * Ck;

                    double smax = -DBL_MAX;
                    for (int64_t z = z0; z < z1; z++) {
                        const int64_t hi = col_idx[z] / Wi;
                        const int64_t wip = (col_idx[z] % Wi + pscale * wo) % Wi;
                        const float *kp = kx + ((b * Hi + hi) * Wi + wip) * ldk + h * Ck;
                        double s = 0.0;
                        for (int64_t c = 0; c < Ck; c++) s += (double)qp[c] * (double)kp[c];
                        sc[z - z0] = s;
                        if (s > smax) smax = s;
                    }
                    double asum = 0.0;
                    for (int64_t c = 0; c < Cv; c++) acc[c] = 0.0;
                    for (int64_t z = z0; z < z1; z++) {
                        const int64_t hi = col_idx[z] / Wi;
                        const int64_t wip = (col_idx[z] % Wi + pscale * wo) % Wi;
                        const float *vp = vx + ((b * Hi + hi) * Wi + wip) * ldv + h * Cv;
                        const double a = exp(sc[z - z0] - smax) * (double)quad_w[hi];
                        asum += a;
                        for (int64_t c = 0; c < Cv; c++) acc[c] += a * (double)vp[c];
                    }
                    double *yp = y + ((b * Ho + ho) * Wo + wo) * ldv + h * Cv;
                    for (int64_t c = 0; c < Cv; c++) yp[c] = acc[c] / asum;
                }
            }
        }
        free(sc);
        free(acc);
    }
}

/* ------------------------------------------------------------------------- */
/* float64 spec, backward: attention_torch.py:130-390.                         */
/*   p_j = a_j / S,  g_j = <dy, v_j>,  I = sum_j p_j g_j                        */
/*   dv[hi_j, wip_j] += p_j dy                       (attention_torch.py:204) */
/*   dk[hi_j, wip_j] += q p_j (g_j - I)              (attention_torch.py:299) */
/*   dq              = sum_j p_j (g_j - I) k_j       (attention_torch.py:388) */
/* Only queries on rows ho in [ho_lo, ho_hi) are visited: dq is written for    */
/* those rows, dk/dv receive the contributions of those rows only (the caller  */
/* zero-fills them).  Parallel over (batch, head) so scatters never collide.   */
/* ------------------------------------------------------------------------- */
void s2o_bwd_f64(const float *kx, const float *vx, const float *qy, const float *dy, const float *quad_w,
                 const int64_t *col_idx, const int64_t *row_off, double *dk, double *dv, double *dq, int64_t B,
                 int64_t nh, int64_t Hi, int64_t Wi, int64_t Ho, int64_t Wo, int64_t Ck, int64_t Cv, int64_t ho_lo,
                 int64_t ho_hi)
{
    const int64_t pscale = Wi / Wo;
    const int64_t ldk = nh * Ck, ldv = nh * Cv;
    const int64_t BH = B * nh;

    int64_t max_len = 0;
    for (int64_t ho = ho_lo; ho < ho_hi; ho++) {
        const int64_t len = row_off[ho + 1] - row_off[ho];
        if (len > max_len) max_len = len;
    }

#pragma omp parallel
    {
        double *pa = (double *)malloc(sizeof(double) * (size_t)(max_len + 1));
        double *pg = (double *)malloc(sizeof(double) * (size_t)(max_len + 1));
        double *acc = (double *)malloc(sizeof(double) * (size_t)(Ck + 1));

#pragma omp for schedule(dynamic, 1)
        for (int64_t bh = 0; bh < BH; bh++) {
            const int64_t b = bh / nh, h = bh % nh;
            for (int64_t ho = ho_lo; ho < ho_hi; ho++) {
                const int64_t z0 = row_off[ho], z1 = row_off[ho + 1];
                for (int64_t wo = 0; wo < Wo; wo++) {
                    const float *qp = qy + ((b * Ho + ho) * Wo + wo) * ldk + h * Ck;
                    const float *gp = dy + ((b * Ho + ho) * Wo + wo) * ldv + h * Cv;

                    double smax = -DBL_MAX;
                    for (int64_t z = z0; z < z1; z++) {
                        const int64_t hi = col_idx[z] / Wi;
                        const int64_t wip = (col_idx[z] % Wi + pscale * wo) % Wi;
                        const float *kp = kx + ((b * Hi + hi) * Wi + wip) * ldk + h * Ck;
                        const float *vp = vx + ((b * Hi + hi) * Wi + wip) * ldv + h * Cv;
                        double s = 0.0, g = 0.0;
                        for (int64_t c = 0; c < Ck; c++) s += (double)qp[c] * (double)kp[c];
                        for (int64_t c = 0; c < Cv; c++) g += (double)gp[c] * (double)vp[c];
                        pa[z - z0] = s;
                        pg[z - z0] = g;
                        if (s > smax) smax = s;
                    }
                    double asum = 0.0, agv = 0.0;
                    for (int64_t z = z0; z < z1; z++) {
                        const int64_t hi = col_idx[z] / Wi;
                        const double a = exp(pa[z - z0] - smax) * (double)quad_w[hi];
                        pa[z - z0] = a;
                        asum += a;
                        agv += a * pg[z - z0];
                    }
                    const double integral = agv / asum;

                    for (int64_t c = 0; c < Ck; c++) acc[c] = 0.0;
                    for (int64_t z = z0; z < z1; z++) {
                        const int64_t hi = col_idx[z] / Wi;
                        const int64_t wip = (col_idx[z] % Wi + pscale * wo) % Wi;
                        const float *kp = kx + ((b * Hi + hi) * Wi + wip) * ldk + h * Ck;
                        double *dkp = dk + ((b * Hi + hi) * Wi + wip) * ldk + h * Ck;
                        double *dvp = dv + ((b * Hi + hi) * Wi + wip) * ldv + h * Cv;
                        const double p = pa[z - z0] / asum;
                        const double coef = p * (pg[z - z0] - integral);
                        for (int64_t c = 0; c < Cv; c++) dvp[c] += p * (double)gp[c];
                        for (int64_t c = 0; c < Ck; c++) {
                            dkp[c] += coef * (double)qp[c];
                            acc[c] += coef * (double)kp[c];
                        }
                    }
                    double *dqp = dq + ((b * Ho + ho) * Wo + wo) * ldk + h * Ck;
                    for (int64_t c = 0; c < Ck; c++) dqp[c] = acc[c];
                }
            }
        }
        free(pa);
        free(pg);
        free(acc);
    }
}
