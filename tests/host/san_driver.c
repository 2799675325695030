/*
 * Sanitizer run of the CPU-side arithmetic: the C oracle (oracle/kernels_ref.c) and the host build
 * of the kernels' range rule and layout index math (host_rules.cpp), on small inputs generated
 * here, edge cases included (single atoms, empty crystals, K = 0, exponents that are zero, positive,
 * infinite or NaN).  Built with -fsanitize=address,undefined and run by tests/test_host_rules.py: any
 * out-of-bounds access, use of freed memory, signed overflow or misaligned access ends the run with
 * a report and a non-zero status.  Prints a checksum of everything computed so that the run
 * cannot be optimised away.  Test infrastructure only.
 */
#include <math.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>

typedef long long i64;

/* oracle/kernels_ref.c */
void ref_translation_ranges(const float *, const float *, const i64 *, i64, i64, double, int, int, int32_t *);
void ref_real_enc_fwd(const float *, const float *, const float *, const i64 *, const i64 *, i64, i64, i64, i64, i64,
                      double, double, const float *, i64, const float *, double, int, int, float *, float *);
void ref_real_enc_fwd_cond(const float *, const float *, const float *, const i64 *, const i64 *, i64, i64, i64, i64,
                           double, double, const float *, double, int, int, float *);
void ref_real_enc_bwd(const float *, const float *, const float *, const i64 *, const i64 *, const i64 *,
                      const float *, const float *, const float *, i64, i64, i64, i64, i64, double, double,
                      const float *, i64, const float *, double, int, int, float *, float *);
void ref_real_enc_bwd_magnitude(const float *, const float *, const float *, const i64 *, const i64 *, const i64 *,
                                const float *, const float *, const float *, i64, i64, i64, i64, i64, double, double,
                                const float *, i64, const float *, double, int, int, float *, float *);
void ref_fused_dpa_fwd(const float *, const float *, const float *, const float *, const float *, const i64 *,
                       const i64 *, i64, i64, i64, i64, i64, float *, float *);
void ref_fused_dpa_bwd(const float *, const float *, const float *, const float *, const i64 *, const i64 *, i64, i64,
                       i64, i64, i64, const float *, const float *, const float *, float *, float *, float *, float *,
                       float *);
void ref_irregular_mean(const float *, const i64 *, i64, i64, float *);
void ref_minimum_distance(const float *, const float *, const i64 *, const i64 *, i64, const float *, double, int, int,
                          float *);
/* host_rules.cpp */
/* (declared with this file's 64-bit integer type; the definitions use i64, the same size) */
int host_max_range(void);
void host_translation_ranges(const float *, const float *, const i64 *, i64, i64, double, int, int, int32_t *);
int host_batch_layout(const i64 *, i64, i64, i64, i64 *, i64 *, i64 *, i64 *, i64 *, i64 *, i64 *);

static unsigned long long lcg = 88172645463325252ull;
static float unit(void)
{
    lcg = lcg * 6364136223846793005ull + 1442695040888963407ull;
    return (float)((lcg >> 40) & 0xFFFFFF) / 16777216.0f;
}
static float *falloc(size_t n) { return (float *)malloc(sizeof(float) * (n ? n : 1)); }
static double checksum = 0.0;
static void fold(const float *x, size_t n)
{
    for (size_t k = 0; k < n; k++)
        if (x[k] == x[k] && fabsf(x[k]) < 1e30f) checksum += x[k];
}

static int run_case(const i64 *sizes, i64 B, int K, int D, int H, double cutoff, int lr, int mr)
{
    i64 N = 0, E = 0;
    for (i64 b = 0; b < B; b++) { N += sizes[b]; E += sizes[b] * sizes[b]; }
    const i64 U = (E + N) / 2;
    i64 *as = malloc(sizeof(i64) * (B + 1)), *es = malloc(sizeof(i64) * (B + 1)),
        *us = malloc(sizeof(i64) * (B + 1)), *row = malloc(sizeof(i64) * (N + 1)),
        *edges = malloc(sizeof(i64) * (2 * E + 1)), *pairs = malloc(sizeof(i64) * (5 * U + 1)),
        *batch = malloc(sizeof(i64) * (N + 1));
    if (host_batch_layout(sizes, B, N, E, as, es, us, row, edges, pairs, batch) != 0) return 1;
    /* every edge appears in exactly one unit, together with its reverse */
    for (i64 u = 0; u < U; u++) {
        const i64 *d = pairs + 5 * u;
        if (d[0] < 0 || d[0] >= E || d[1] < 0 || d[1] >= E) return 2;
        if (edges[d[0]] != d[2] || edges[E + d[0]] != d[3] || edges[d[1]] != d[3] || edges[E + d[1]] != d[2]) return 3;
        if (batch[d[2]] != d[4]) return 4;
    }
    float *pos = falloc(3 * N), *tv = falloc(9 * B), *rvl = falloc(3 * B), *a = falloc(N * H), *rpos = falloc(3 * E);
    for (i64 x = 0; x < 3 * N; x++) pos[x] = 6.0f * unit();
    for (i64 b = 0; b < B; b++) {
        for (int x = 0; x < 9; x++) tv[9 * b + x] = (x % 4 == 0 ? 4.0f + 3.0f * unit() : 0.7f * (unit() - 0.5f));
        for (int x = 0; x < 3; x++) rvl[3 * b + x] = 6.2831853f / (4.0f + 3.0f * unit());
    }
    for (i64 x = 0; x < N * H; x++) a[x] = -(0.05f + 0.5f * unit());
    for (i64 e = 0; e < E; e++)
        for (int x = 0; x < 3; x++) rpos[3 * e + x] = pos[3 * edges[E + e] + x] - pos[3 * edges[e] + x];
    int32_t *R = malloc(sizeof(int32_t) * (3 * N * H + 1)), *R2 = malloc(sizeof(int32_t) * (3 * N * H + 1));
    ref_translation_ranges(a, rvl, batch, N, H, cutoff, lr, mr, R);
    host_translation_ranges(a, rvl, batch, N, H, cutoff, lr, mr, R2);
    for (i64 x = 0; x < 3 * N * H; x++) {
        if (R[x] != R2[x]) return 5;
        checksum += R[x];
    }
    const int Kn = K > 0 ? K : 1;
    float *W = falloc((size_t)H * D * Kn), *z = falloc(E * H), *v = falloc((size_t)E * H * D), *s = falloc((size_t)E * H * Kn),
          *cond = falloc((size_t)E * H * Kn), *gz = falloc(E * H), *gv = falloc((size_t)E * H * D), *ga = falloc(N * H),
          *gW = falloc((size_t)H * D * Kn), *dmin = falloc(E);
    for (size_t x = 0; x < (size_t)H * D * Kn; x++) W[x] = unit() - 0.5f;
    for (i64 x = 0; x < E * H; x++) gz[x] = unit() - 0.5f;
    for (size_t x = 0; x < (size_t)E * H * D; x++) gv[x] = unit() - 0.5f;
    ref_real_enc_fwd(a, rpos, tv, batch, edges, N, H, E, K, D, 14.0, 1.0, K > 0 ? W : NULL, K > 0 ? 1 : 0, rvl, cutoff, lr, mr,
                     z, K > 0 ? v : NULL);
    fold(z, E * H);
    if (K > 0) {
        fold(v, (size_t)E * H * D);
        ref_real_enc_fwd(a, rpos, tv, batch, edges, N, H, E, K, 0, 14.0, 1.0, NULL, 0, rvl, cutoff, lr, mr, z, s);
        fold(s, (size_t)E * H * K);
        ref_real_enc_fwd_cond(a, rpos, tv, batch, edges, N, H, E, K, 14.0, 1.0, rvl, cutoff, lr, mr, cond);
        fold(cond, (size_t)E * H * K);
    }
    ref_real_enc_bwd(a, rpos, tv, batch, edges, row, z, gz, K > 0 ? gv : NULL, N, H, E, K, D, 14.0, 1.0, K > 0 ? W : NULL,
                     K > 0 ? 1 : 0, rvl, cutoff, lr, mr, ga, K > 0 ? gW : NULL);
    fold(ga, N * H);
    ref_real_enc_bwd_magnitude(a, rpos, tv, batch, edges, row, z, gz, K > 0 ? gv : NULL, N, H, E, K, D, 14.0, 1.0,
                               K > 0 ? W : NULL, K > 0 ? 1 : 0, rvl, cutoff, lr, mr, ga, K > 0 ? gW : NULL);
    fold(ga, N * H);
    ref_minimum_distance(rpos, tv, batch, edges, E, rvl, cutoff < 0 ? 0.0 : cutoff, lr, mr, dmin);
    fold(dmin, E);
    /* attention over the same edge list */
    float *q = falloc((size_t)N * H * D), *k = falloc((size_t)N * H * D), *val = falloc((size_t)N * H * D),
          *prob = falloc(E * H), *out = falloc((size_t)N * H * D), *go = falloc((size_t)N * H * D),
          *gq = falloc((size_t)N * H * D), *gk = falloc((size_t)N * H * D), *gvv = falloc((size_t)N * H * D),
          *gaij = falloc(E * H), *gbij = falloc((size_t)E * H * D), *pooled = falloc((size_t)B * H * D);
    for (size_t x = 0; x < (size_t)N * H * D; x++) { q[x] = unit() - 0.5f; k[x] = unit() - 0.5f; val[x] = unit() - 0.5f; go[x] = unit() - 0.5f; }
    ref_fused_dpa_fwd(q, k, val, z, K > 0 ? v : NULL, edges, row, N, H, E, D, D, prob, out);
    fold(out, (size_t)N * H * D);
    ref_fused_dpa_bwd(q, k, val, K > 0 ? v : NULL, edges, row, N, H, E, D, D, prob, out, go, gq, gk, gvv, gaij,
                      K > 0 ? gbij : NULL);
    fold(gq, (size_t)N * H * D);
    fold(gaij, E * H);
    ref_irregular_mean(out, as, B, (i64)H * D, pooled);
    fold(pooled, (size_t)B * H * D);
    free(as); free(es); free(us); free(row); free(edges); free(pairs); free(batch); free(pos); free(tv); free(rvl);
    free(a); free(rpos); free(R); free(R2); free(W); free(z); free(v); free(s); free(cond); free(gz); free(gv); free(ga);
    free(gW); free(dmin); free(q); free(k); free(val); free(prob); free(out); free(go); free(gq); free(gk); free(gvv);
    free(gaij); free(gbij); free(pooled);
    return 0;
}

int main(void)
{
    /* the range rule on exponents no finite model produces: every half-width stays within bounds */
    const float odd[] = {0.0f, -0.0f, 1.0f, 1e30f, -1e-38f, -1e-45f, -1e30f, INFINITY, -INFINITY, NAN};
    const float rv[] = {0.0f, 1e-30f, 0.9f, 1e30f, INFINITY, NAN, -1.0f};
    const i64 zero = 0;
    for (unsigned x = 0; x < sizeof(odd) / sizeof(odd[0]); x++)
        for (unsigned y = 0; y < sizeof(rv) / sizeof(rv[0]); y++)
            for (int sigma = 0; sigma < 3; sigma++) {
                const float rvl[3] = {rv[y], 0.9f, rv[(y + 1) % 7]};
                int32_t R[3];
                host_translation_ranges(&odd[x], rvl, &zero, 1, 1, sigma == 0 ? -3.5 : (sigma == 1 ? 4.0 : 0.0), 2, sigma, R);
                for (int d = 0; d < 3; d++) {
                    if (R[d] < 0 || R[d] > host_max_range()) { printf("range out of bounds\n"); return 10; }
                    checksum += R[d];
                }
            }
    const i64 s1[] = {1}, s2[] = {3, 1, 5, 2}, s3[] = {2, 0, 4, 0}, s4[] = {7, 7};
    int rc;
    if ((rc = run_case(s1, 1, 0, 4, 2, 0.0, 1, 0))) { printf("case 1 failed: %d\n", rc); return rc; }
    if ((rc = run_case(s2, 4, 8, 4, 4, 0.0, 1, 0))) { printf("case 2 failed: %d\n", rc); return rc; }
    if ((rc = run_case(s2, 4, 6, 3, 2, -3.5, 1, 1))) { printf("case 3 failed: %d\n", rc); return rc; }
    if ((rc = run_case(s3, 4, 5, 2, 1, 3.0, 1, 0))) { printf("case 4 failed: %d\n", rc); return rc; }
    if ((rc = run_case(s4, 2, 16, 8, 8, -3.5, 2, 2))) { printf("case 5 failed: %d\n", rc); return rc; }
    printf("OK %.9e\n", checksum);
    return 0;
}
