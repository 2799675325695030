/*
 * CPU oracle, kernel-level semantics.  TEST INFRASTRUCTURE ONLY: the product
 * never links, loads or calls this file; tests, the smoke check and the
 * benchmark's cpu_baseline leg use it as the checker for the HIP kernels.
 *
 * Plain-C restatement of what the reference's device kernels compute, one
 * function per kernel, including the adaptive translation box ("rule B").
 * Geometry is evaluated in float exactly as the kernels do (build with
 * -ffp-contract=off); sums over translations, bins and edges are accumulated
 * in double so this is the tighter of the two oracles.
 *
 *   ref_translation_ranges   models/kernels/real_enc_fwd.cu:58-85
 *   ref_real_enc_fwd         models/kernels/real_enc_fwd.cu:87-143,
 *                            models/kernels/real_enc_proj_fwd.cu:87-169
 *   ref_real_enc_bwd         models/kernels/real_enc_bwd.cu:80-156,
 *                            models/kernels/real_enc_proj_bwd.cu:88-219
 *   ref_fused_dpa_fwd        models/kernels/fused_dpa_fwd.cu:18-125
 *   ref_fused_dpa_bwd        models/kernels/fused_dpa_bwd.cu:24-125,
 *                            models/kernels/fused_dpa_bwd_q.cu:14-53
 *   ref_irregular_mean       models/kernels/irregular_mean_fwd.cu:4-90
 *   ref_minimum_distance     models/kernels/minimum_distance.cu:4-67
 *   ref_reci_enc_fwd         models/kernels/reci_enc_fwd.cu:3-68
 *   ref_reci_enc_bwd         models/kernels/reci_enc_bwd.cu:3-71
 *
 * Pins: tests/test_oracle_kernels.py checks these against the torch-path
 * oracle under rule A (cutoff 0), against brute force / closed forms, and the
 * range rule against its geometric invariant (every lattice point within the
 * cut-off lies in the box).  The reciprocal-space pair is pinned by the full-cube
 * sum in float64, by the Poisson summation identity against the real-space
 * lattice sum, by the torch-path restatement (other enumeration of the half
 * space) and, for the backward, by finite differences of the forward minus the
 * normalisation term the reference's kernel leaves out.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#define PI_F 3.141592654f

typedef long long i64;

/* Per (atom|edge source, head) translation half-widths R[3].
 * cutoff == 0 selects the fixed cube (rule A). */
static void range_rule(float a, const float *rvl, double cutoff_radius,
                       int lattice_range, int minimum_range, int R[3])
{
    float cutoff = (float)cutoff_radius;
    R[0] = R[1] = R[2] = lattice_range;
    if (cutoff != 0.0f) {
        if (cutoff < 0)
            cutoff = sqrtf(-0.5f / a) * (-cutoff);
        for (int d = 0; d < 3; d++) {
            float num = (cutoff + 0.01f) * rvl[d];
            R[d] = (int)ceil((double)num / (2.0 * (double)PI_F));
            if (minimum_range > 0 && R[d] < minimum_range)
                R[d] = minimum_range;
        }
    }
}

void ref_translation_ranges(const float *a_ik, const float *rvlen_n, const i64 *batch_i,
                            i64 N, i64 H, double cutoff_radius, int lattice_range,
                            int minimum_range, int32_t *R_out)
{
    static const float zero3[3] = {0, 0, 0};
    for (i64 i = 0; i < N; i++)
        for (i64 h = 0; h < H; h++) {
            int R[3];
            const float *rvl = rvlen_n ? rvlen_n + batch_i[i] * 3 : zero3;
            range_rule(a_ik[i * H + h], rvl, rvlen_n ? cutoff_radius : 0.0,
                       lattice_range, minimum_range, R);
            for (int d = 0; d < 3; d++)
                R_out[(i * H + h) * 3 + d] = R[d];
        }
}

static inline float dist2_f(const float *r, const float *t, float n1, float n2, float n3)
{
    float dx = r[0] + t[0] * n1 + t[3] * n2 + t[6] * n3;
    float dy = r[1] + t[1] * n1 + t[4] * n2 + t[7] * n3;
    float dz = r[2] + t[2] * n1 + t[5] * n2 + t[8] * n3;
    return dx * dx + dy * dy + dz * dz;
}

/* Gaussian argument of bin k (0-based) for distance sqrt(d2), built the way the
 * kernels build it: start at -d/mu0/(ws*sqrt2) and add 1/(ws*sqrt2) (k+1) times. */
static inline double gauss_bin(double d, double mu0, double inv_ws_sqrt2, int k)
{
    double b = -d / mu0 * inv_ws_sqrt2 + inv_ws_sqrt2 * (double)(k + 1);
    return exp(-b * b);
}

/* z_ek (E,H); v_ekd (E,H,K) when W_k == NULL else (E,H,D).  W_k is
 * (W_num,H,D,K), W_num in {1,E,N}. */
void ref_real_enc_fwd(const float *a_ik, const float *rpos_ij_e, const float *tvecs_n,
                      const i64 *batch_i, const i64 *edge_ij_e, i64 N, i64 H, i64 E,
                      i64 K, i64 D, double dist_max, double wscale, const float *W_k,
                      i64 W_num, const float *rvlen_n, double cutoff_radius,
                      int lattice_range, int minimum_range, float *z_ek, float *v_ekd)
{
    static const float zero3[3] = {0, 0, 0};
    double *sv = (double *)malloc(sizeof(double) * (size_t)(K > 0 ? K : 1));
    const double inv_ws_sqrt2 = 1.0 / (wscale * sqrt(2.0));
    const double mu0 = K > 0 ? dist_max / (double)K : 1.0;
    for (i64 e = 0; e < E; e++) {
        const i64 i = edge_ij_e[e];
        const i64 n = batch_i[i];
        const float *r = rpos_ij_e + e * 3;
        const float *t = tvecs_n + n * 9;
        const float *rvl = rvlen_n ? rvlen_n + n * 3 : zero3;
        for (i64 h = 0; h < H; h++) {
            const float a = a_ik[i * H + h];
            int R[3];
            range_rule(a, rvl, rvlen_n ? cutoff_radius : 0.0, lattice_range, minimum_range, R);
            float d2min = 1e10f;
            for (int n1 = -R[0]; n1 <= R[0]; n1++)
                for (int n2 = -R[1]; n2 <= R[1]; n2++)
                    for (int n3 = -R[2]; n3 <= R[2]; n3++) {
                        float d2 = dist2_f(r, t, (float)n1, (float)n2, (float)n3);
                        if (d2 < d2min) d2min = d2;
                    }
            double sum = 0;
            for (i64 k = 0; k < K; k++) sv[k] = 0;
            for (int n1 = -R[0]; n1 <= R[0]; n1++)
                for (int n2 = -R[1]; n2 <= R[1]; n2++)
                    for (int n3 = -R[2]; n3 <= R[2]; n3++) {
                        float d2 = dist2_f(r, t, (float)n1, (float)n2, (float)n3);
                        double w = exp((double)a * ((double)d2 - (double)d2min));
                        sum += w;
                        if (K > 0) {
                            double d = sqrt((double)d2);
                            for (i64 k = 0; k < K; k++)
                                sv[k] += gauss_bin(d, mu0, inv_ws_sqrt2, (int)k) * w;
                        }
                    }
            const i64 eh = e * H + h;
            z_ek[eh] = (float)(log(sum) + (double)d2min * (double)a);
            if (K > 0 && v_ekd) {
                if (!W_k) {
                    for (i64 k = 0; k < K; k++)
                        v_ekd[eh * K + k] = (float)(sv[k] / sum);
                } else {
                    i64 w_ind = 0;
                    if (W_num == 1) w_ind = 0;
                    else if (W_num == E) w_ind = e;
                    else if (W_num == N) w_ind = i;
                    const float *W = W_k + (w_ind * H + h) * D * K;
                    for (i64 d = 0; d < D; d++) {
                        double acc = 0;
                        for (i64 k = 0; k < K; k++)
                            acc += (double)W[d * K + k] * sv[k];
                        v_ekd[eh * D + d] = (float)(acc / sum);
                    }
                }
            }
        }
    }
    free(sv);
}

/* First-order float32 conditioning of the Gaussian averages s[e,h,k] = sum_n p_n g_k(d_n):
 *     cond[e,h,k] = sum_n p_n g_k(d_n) * ( 2 |b_k(d_n)| d_n / (sqrt2 ws mu0)  +  |a| d_n^2 )
 * A relative rounding error u in a computed distance moves g_k by g_k 2|b| d/(sqrt2 ws mu0) u
 * (b = Gaussian argument), and one in a d^2 moves the weight p_n by p_n |a| d^2 u: u * cond
 * is the error any float32 evaluation of s carries, whatever its order of operations.  Used by
 * the tests as the element-wise tolerance of narrow Gaussians far from their centre; not a
 * restatement of reference code. */
void ref_real_enc_fwd_cond(const float *a_ik, const float *rpos_ij_e, const float *tvecs_n,
                           const i64 *batch_i, const i64 *edge_ij_e, i64 N, i64 H, i64 E,
                           i64 K, double dist_max, double wscale, const float *rvlen_n,
                           double cutoff_radius, int lattice_range, int minimum_range, float *cond_ehk)
{
    static const float zero3[3] = {0, 0, 0};
    (void)N;
    double *sv = (double *)malloc(sizeof(double) * (size_t)(K > 0 ? K : 1));
    const double inv_ws_sqrt2 = 1.0 / (wscale * sqrt(2.0));
    const double mu0 = K > 0 ? dist_max / (double)K : 1.0;
    for (i64 e = 0; e < E; e++) {
        const i64 i = edge_ij_e[e];
        const i64 n = batch_i[i];
        const float *r = rpos_ij_e + e * 3;
        const float *t = tvecs_n + n * 9;
        const float *rvl = rvlen_n ? rvlen_n + n * 3 : zero3;
        for (i64 h = 0; h < H; h++) {
            const float a = a_ik[i * H + h];
            int R[3];
            range_rule(a, rvl, rvlen_n ? cutoff_radius : 0.0, lattice_range, minimum_range, R);
            float d2min = 1e10f;
            for (int n1 = -R[0]; n1 <= R[0]; n1++)
                for (int n2 = -R[1]; n2 <= R[1]; n2++)
                    for (int n3 = -R[2]; n3 <= R[2]; n3++) {
                        float d2 = dist2_f(r, t, (float)n1, (float)n2, (float)n3);
                        if (d2 < d2min) d2min = d2;
                    }
            double sum = 0;
            for (i64 k = 0; k < K; k++) sv[k] = 0;
            for (int n1 = -R[0]; n1 <= R[0]; n1++)
                for (int n2 = -R[1]; n2 <= R[1]; n2++)
                    for (int n3 = -R[2]; n3 <= R[2]; n3++) {
                        float d2 = dist2_f(r, t, (float)n1, (float)n2, (float)n3);
                        double w = exp((double)a * ((double)d2 - (double)d2min));
                        sum += w;
                        double d = sqrt((double)d2);
                        for (i64 k = 0; k < K; k++) {
                            double b = -d / mu0 * inv_ws_sqrt2 + inv_ws_sqrt2 * (double)(k + 1);
                            sv[k] += exp(-b * b) * w *
                                     (2.0 * fabs(b) * d / mu0 * inv_ws_sqrt2 + fabs((double)a) * (double)d2);
                        }
                    }
            for (i64 k = 0; k < K; k++) cond_ehk[(e * H + h) * K + k] = (float)(sv[k] / sum);
        }
    }
    free(sv);
}

/* Gradient wrt a_ik (N,H) and, when W_k != NULL, wrt W (W_num,H,D,K), already
 * reduced to W's own shape.  gv_ekd is (E,H,K) without W and (E,H,D) with it;
 * gv_ekd may be NULL (treated as zero).  gW_k may be NULL. */
static void real_enc_bwd_impl(const float *a_ik, const float *rpos_ij_e, const float *tvecs_n,
                              const i64 *batch_i, const i64 *edge_ij_e, const i64 *e_start_i,
                              const float *z_ek, const float *gz_ek, const float *gv_ekd,
                              i64 N, i64 H, i64 E, i64 K, i64 D, double dist_max, double wscale,
                              const float *W_k, i64 W_num, const float *rvlen_n,
                              double cutoff_radius, int lattice_range, int minimum_range,
                              float *ga_ik, float *gW_k, int magnitude)
{
    static const float zero3[3] = {0, 0, 0};
    (void)edge_ij_e;   /* rows are walked through e_start_i */
    const size_t Kn = (size_t)(K > 0 ? K : 1);
    double *sgv = (double *)malloc(sizeof(double) * Kn);
    double *sv = (double *)malloc(sizeof(double) * Kn);
    double *gWacc = NULL;
    size_t gWn = 0;
    if (gW_k && W_k && K > 0) {
        gWn = (size_t)(W_num * H * D * K);
        gWacc = (double *)calloc(gWn, sizeof(double));
    }
    const double inv_ws_sqrt2 = 1.0 / (wscale * sqrt(2.0));
    const double mu0 = K > 0 ? dist_max / (double)K : 1.0;
    for (i64 i = 0; i < N; i++) {
        const i64 n = batch_i[i];
        const float *t = tvecs_n + n * 9;
        const float *rvl = rvlen_n ? rvlen_n + n * 3 : zero3;
        for (i64 h = 0; h < H; h++) {
            const float a = a_ik[i * H + h];
            int R[3];
            range_rule(a, rvl, rvlen_n ? cutoff_radius : 0.0, lattice_range, minimum_range, R);
            double total = 0;
            for (i64 e = e_start_i[i]; e < e_start_i[i + 1]; e++) {
                const float *r = rpos_ij_e + e * 3;
                const i64 eh = e * H + h;
                const double z = z_ek[eh];
                const double gz = gz_ek ? (magnitude ? fabs((double)gz_ek[eh]) : gz_ek[eh]) : 0.0;
                i64 w_ind = 0;
                if (W_num == E) w_ind = e;
                else if (W_num == N) w_ind = i;
                const float *W = W_k ? W_k + (w_ind * H + h) * D * K : NULL;
                for (i64 k = 0; k < K; k++) {
                    sv[k] = 0;
                    if (!gv_ekd) sgv[k] = 0;
                    else if (!W) sgv[k] = magnitude ? fabs((double)gv_ekd[eh * K + k]) : gv_ekd[eh * K + k];
                    else {
                        double acc = 0;
                        for (i64 d = 0; d < D; d++) {
                            const double term = (double)W[d * K + k] * (double)gv_ekd[eh * D + d];
                            acc += magnitude ? fabs(term) : term;
                        }
                        sgv[k] = acc;
                    }
                }
                double px_avr = 0, pbg_avr = 0, pxbg = 0;
                for (int n1 = -R[0]; n1 <= R[0]; n1++)
                    for (int n2 = -R[1]; n2 <= R[1]; n2++)
                        for (int n3 = -R[2]; n3 <= R[2]; n3++) {
                            float d2 = dist2_f(r, t, (float)n1, (float)n2, (float)n3);
                            double p = exp((double)a * (double)d2 - z);
                            double px = (double)d2 * p;
                            px_avr += px;
                            if (K > 0) {
                                double d = sqrt((double)d2), bg = 0;
                                for (i64 k = 0; k < K; k++) {
                                    double g = gauss_bin(d, mu0, inv_ws_sqrt2, (int)k);
                                    bg += g * sgv[k];
                                    sv[k] += g * p;
                                }
                                pxbg += px * bg;
                                pbg_avr += p * bg;
                            }
                        }
                total += px_avr * gz + pxbg + (magnitude ? px_avr * pbg_avr : -px_avr * pbg_avr);
                if (gWacc && gv_ekd) {
                    double *gW = gWacc + (w_ind * H + h) * D * K;
                    for (i64 d = 0; d < D; d++)
                        for (i64 k = 0; k < K; k++) {
                            const double g = gv_ekd[eh * D + d];
                            gW[d * K + k] += sv[k] * (magnitude ? fabs(g) : g);
                        }
                }
            }
            ga_ik[i * H + h] = (float)total;
        }
    }
    if (gWacc) {
        for (size_t x = 0; x < gWn; x++) gW_k[x] = (float)gWacc[x];
        free(gWacc);
    }
    free(sgv);
    free(sv);
}

void ref_real_enc_bwd(const float *a_ik, const float *rpos_ij_e, const float *tvecs_n,
                      const i64 *batch_i, const i64 *edge_ij_e, const i64 *e_start_i,
                      const float *z_ek, const float *gz_ek, const float *gv_ekd,
                      i64 N, i64 H, i64 E, i64 K, i64 D, double dist_max, double wscale,
                      const float *W_k, i64 W_num, const float *rvlen_n,
                      double cutoff_radius, int lattice_range, int minimum_range,
                      float *ga_ik, float *gW_k)
{
    real_enc_bwd_impl(a_ik, rpos_ij_e, tvecs_n, batch_i, edge_ij_e, e_start_i, z_ek, gz_ek, gv_ekd, N, H, E, K, D,
                      dist_max, wscale, W_k, W_num, rvlen_n, cutoff_radius, lattice_range, minimum_range, ga_ik,
                      gW_k, 0);
}

/* The same sums with every term replaced by its magnitude (|gz| PX + sum_n p_n (d_n^2 + PX)
 * sum_k g_k |W^T| |gv| for ga, sum_e S |gv| for gW): what a float32 evaluation's rounding error
 * is proportional to, used by the tests as the element-wise tolerance of these gradients.  Not a
 * restatement of reference code. */
void ref_real_enc_bwd_magnitude(const float *a_ik, const float *rpos_ij_e, const float *tvecs_n,
                                const i64 *batch_i, const i64 *edge_ij_e, const i64 *e_start_i,
                                const float *z_ek, const float *gz_ek, const float *gv_ekd,
                                i64 N, i64 H, i64 E, i64 K, i64 D, double dist_max, double wscale,
                                const float *W_k, i64 W_num, const float *rvlen_n,
                                double cutoff_radius, int lattice_range, int minimum_range,
                                float *ga_ik, float *gW_k)
{
    real_enc_bwd_impl(a_ik, rpos_ij_e, tvecs_n, batch_i, edge_ij_e, e_start_i, z_ek, gz_ek, gv_ekd, N, H, E, K, D,
                      dist_max, wscale, W_k, W_num, rvlen_n, cutoff_radius, lattice_range, minimum_range, ga_ik,
                      gW_k, 1);
}

/* que is already divided by sqrt(Dk).  aij_eh / bij_ehd may be NULL. */
void ref_fused_dpa_fwd(const float *que, const float *key, const float *val,
                       const float *aij_eh, const float *bij_ehd, const i64 *edge_ij_e,
                       const i64 *e_start_i, i64 N, i64 H, i64 E, i64 Dk, i64 Dv,
                       float *prob_eh, float *out)
{
    for (i64 i = 0; i < N; i++)
        for (i64 h = 0; h < H; h++) {
            const i64 e0 = e_start_i[i], e1 = e_start_i[i + 1];
            const float *q = que + (i * H + h) * Dk;
            double *lg = (double *)malloc(sizeof(double) * (size_t)(e1 - e0 + 1));
            double mx = -1e300;
            for (i64 e = e0; e < e1; e++) {
                const i64 j = edge_ij_e[E + e];
                const float *kk = key + (j * H + h) * Dk;
                double s = 0;
                for (i64 d = 0; d < Dk; d++) s += (double)q[d] * (double)kk[d];
                if (aij_eh) s += aij_eh[e * H + h];
                lg[e - e0] = s;
                if (s > mx) mx = s;
            }
            double sum = 0;
            for (i64 e = e0; e < e1; e++) { lg[e - e0] = exp(lg[e - e0] - mx); sum += lg[e - e0]; }
            for (i64 d = 0; d < Dv; d++) {
                double acc = 0;
                for (i64 e = e0; e < e1; e++) {
                    const i64 j = edge_ij_e[E + e];
                    double m = val[(j * H + h) * Dv + d];
                    if (bij_ehd) m += bij_ehd[(e * H + h) * Dv + d];
                    acc += m * (lg[e - e0] / sum);
                }
                out[(i * H + h) * Dv + d] = (float)acc;
            }
            for (i64 e = e0; e < e1; e++) prob_eh[e * H + h] = (float)(lg[e - e0] / sum);
            free(lg);
        }
}

/* Analytic backward of the fused attention from the saved prob/out.
 * Outputs gque, gkey, gval (N,H,D*), gaij (E,H), gbij (E,H,Dv) (may be NULL),
 * all in the *untransposed* edge order. */
void ref_fused_dpa_bwd(const float *que, const float *key, const float *val,
                       const float *bij_ehd, const i64 *edge_ij_e, const i64 *e_start_i,
                       i64 N, i64 H, i64 E, i64 Dk, i64 Dv, const float *prob_eh,
                       const float *out, const float *gout, float *gque, float *gkey,
                       float *gval, float *gaij, float *gbij)
{
    double *gk = (double *)calloc((size_t)(N * H * Dk), sizeof(double));
    double *gv = (double *)calloc((size_t)(N * H * Dv), sizeof(double));
    for (i64 i = 0; i < N; i++)
        for (i64 h = 0; h < H; h++) {
            const float *go = gout + (i * H + h) * Dv;
            const float *o = out + (i * H + h) * Dv;
            const float *q = que + (i * H + h) * Dk;
            double gq[1024];
            for (i64 d = 0; d < Dk; d++) gq[d] = 0;
            for (i64 e = e_start_i[i]; e < e_start_i[i + 1]; e++) {
                const i64 j = edge_ij_e[E + e];
                const double p = prob_eh[e * H + h];
                double gs = 0;
                for (i64 d = 0; d < Dv; d++) {
                    double t = (double)go[d] * p;
                    double m = val[(j * H + h) * Dv + d];
                    if (bij_ehd) m += bij_ehd[(e * H + h) * Dv + d];
                    gv[(j * H + h) * Dv + d] += t;
                    if (gbij) gbij[(e * H + h) * Dv + d] = (float)t;
                    gs += (m - (double)o[d]) * t;
                }
                if (gaij) gaij[e * H + h] = (float)gs;
                for (i64 d = 0; d < Dk; d++) {
                    gk[(j * H + h) * Dk + d] += gs * (double)q[d];
                    gq[d] += gs * (double)key[(j * H + h) * Dk + d];
                }
            }
            for (i64 d = 0; d < Dk; d++) gque[(i * H + h) * Dk + d] = (float)gq[d];
        }
    for (i64 x = 0; x < N * H * Dk; x++) gkey[x] = (float)gk[x];
    for (i64 x = 0; x < N * H * Dv; x++) gval[x] = (float)gv[x];
    free(gk);
    free(gv);
}

void ref_irregular_mean(const float *src, const i64 *start_n, i64 B, i64 D, float *dst)
{
    for (i64 n = 0; n < B; n++)
        for (i64 k = 0; k < D; k++) {
            double s = 0;
            for (i64 r = start_n[n]; r < start_n[n + 1]; r++) s += src[r * D + k];
            dst[n * D + k] = (float)(s / (double)(start_n[n + 1] - start_n[n]));
        }
}

/* Per-edge minimum of the squared distance over one box for the whole edge
 * (a positive cut-off sizes the box, otherwise the fixed cube). */
void ref_minimum_distance(const float *rpos_ij_e, const float *tvecs_n, const i64 *batch_i,
                          const i64 *edge_ij_e, i64 E, const float *rvlen_n,
                          double cutoff_radius, int lattice_range, int minimum_range,
                          float *dist2_min_e)
{
    for (i64 e = 0; e < E; e++) {
        const i64 n = batch_i[edge_ij_e[e]];
        const float *r = rpos_ij_e + e * 3;
        const float *t = tvecs_n + n * 9;
        int R[3] = {lattice_range, lattice_range, lattice_range};
        if ((float)cutoff_radius > 0.0f && rvlen_n) {
            for (int d = 0; d < 3; d++) {
                float num = ((float)cutoff_radius + 0.01f) * rvlen_n[n * 3 + d];
                R[d] = (int)ceil((double)num / (2.0 * (double)PI_F));
                if (minimum_range > 0 && R[d] < minimum_range) R[d] = minimum_range;
            }
        }
        float d2min = 1e10f;
        for (int n1 = -R[0]; n1 <= R[0]; n1++)
            for (int n2 = -R[1]; n2 <= R[1]; n2++)
                for (int n3 = -R[2]; n3 <= R[2]; n3++) {
                    float d2 = dist2_f(r, t, (float)n1, (float)n2, (float)n3);
                    if (d2 < d2min) d2min = d2;
                }
        dist2_min_e[e] = d2min;
    }
}

/* Reciprocal-space lattice sum.  z[e,h] = log(max(S, 1e-6)) + 1.5 log(-4 pi a) - log(V) with
 * S = sum over the half space n1 in [0,R] (weight 2 for n1 != 0), n2, n3 in [-R,R] of
 * exp(a |k_n|^2) cos(<kr_base, n>), k_n = n1 b1 + n2 b2 + n3 b3 (rows of rvecs).  k_n, its
 * square and the phase are float expressions as in the kernel; exp, cos and the sum are
 * double here.  sumexp[e,h] = S. */
void ref_reci_enc_fwd(const float *a_ik, const float *kr_base_e, const float *rvecs_n, const float *vcell_n,
                      const i64 *batch_i, const i64 *edge_ij_e, i64 N, i64 H, i64 E, int lattice_range,
                      float *z_ek, float *sumexp_ek)
{
    (void)N;
    const int R = lattice_range;
    for (i64 e = 0; e < E; e++) {
        const i64 i = edge_ij_e[e];
        const i64 n = batch_i[i];
        const float *kr = kr_base_e + e * 3;
        const float *rv = rvecs_n + n * 9;
        for (i64 h = 0; h < H; h++) {
            const float a = a_ik[i * H + h];
            double sum = 0.0;
            for (int m1 = 0; m1 <= R; m1++) {
                const double scale = m1 == 0 ? 1.0 : 2.0;
                for (int m2 = -R; m2 <= R; m2++)
                    for (int m3 = -R; m3 <= R; m3++) {
                        const float n1 = (float)m1, n2 = (float)m2, n3 = (float)m3;
                        const float k1 = rv[0] * n1 + rv[3] * n2 + rv[6] * n3;
                        const float k2 = rv[1] * n1 + rv[4] * n2 + rv[7] * n3;
                        const float k3 = rv[2] * n1 + rv[5] * n2 + rv[8] * n3;
                        const float kk = k1 * k1 + k2 * k2 + k3 * k3;
                        const float ph = kr[0] * n1 + kr[1] * n2 + kr[2] * n3;
                        sum += exp((double)(a * kk)) * cos((double)ph) * scale;
                    }
            }
            const double log_ci = 1.5 * log(-12.5663706144 * (double)a) - log((double)vcell_n[n]);
            z_ek[e * H + h] = (float)(log(sum > 1e-6 ? sum : 1e-6) + log_ci);
            sumexp_ek[e * H + h] = (float)sum;
        }
    }
}

/* ga[i,h] = sum over the edges of row i of gz[e,h] / S[e,h] * sum_n |k_n|^2 exp(a |k_n|^2) cos(.)
 * (zero where S < 1e-6).  As in the reference's kernel, the derivative of the normalisation
 * term 1.5 log(-4 pi a) is NOT part of the result unless normalisation_grad is set (then it is
 * the derivative of z that autograd gives on the reference's PyTorch path). */
void ref_reci_enc_bwd(const float *a_ik, const float *kr_base_e, const float *rvecs_n, const i64 *batch_i,
                      const i64 *e_start_i, const float *gz_ek, const float *sumexp_ek, i64 N, i64 H,
                      int lattice_range, int normalisation_grad, float *ga_ik)
{
    const int R = lattice_range;
    for (i64 i = 0; i < N; i++) {
        const i64 n = batch_i[i];
        const float *rv = rvecs_n + n * 9;
        for (i64 h = 0; h < H; h++) {
            const float a = a_ik[i * H + h];
            double total = 0.0;
            for (i64 e = e_start_i[i]; e < e_start_i[i + 1]; e++) {
                const float *kr = kr_base_e + e * 3;
                double s = 0.0;
                for (int m1 = 0; m1 <= R; m1++) {
                    const double scale = m1 == 0 ? 1.0 : 2.0;
                    for (int m2 = -R; m2 <= R; m2++)
                        for (int m3 = -R; m3 <= R; m3++) {
                            const float n1 = (float)m1, n2 = (float)m2, n3 = (float)m3;
                            const float k1 = rv[0] * n1 + rv[3] * n2 + rv[6] * n3;
                            const float k2 = rv[1] * n1 + rv[4] * n2 + rv[7] * n3;
                            const float k3 = rv[2] * n1 + rv[5] * n2 + rv[8] * n3;
                            const float kk = k1 * k1 + k2 * k2 + k3 * k3;
                            const float ph = kr[0] * n1 + kr[1] * n2 + kr[2] * n3;
                            s += (double)kk * exp((double)(a * kk)) * cos((double)ph) * scale;
                        }
                }
                const float se = sumexp_ek[e * H + h];
                total += s * (double)gz_ek[e * H + h] * (se < 1e-6f ? 0.0 : 1.0 / (double)se);
                if (normalisation_grad) total += (double)gz_ek[e * H + h] * 1.5 / (double)a;
            }
            ga_ik[i * H + h] = (float)total;
        }
    }
}
