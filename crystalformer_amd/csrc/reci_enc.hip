// Reciprocal-space periodic encoding for gfx950:
//     S[e,h] = sum over the half space n1 in [0,R] (weight 2 for n1 != 0), n2, n3 in [-R,R] of
//              exp(a[i,h] |k_n|^2) cos(<kr_base[e], n>),   k_n = n1 b1 + n2 b2 + n3 b3
//     z[e,h] = log(max(S, 1e-6)) + 1.5 log(-4 pi a[i,h]) - log(V)
// and its backward with respect to a.
//
// What is shared is computed once: exp(a |k_n|^2) depends on the query atom and the head only,
// so one wavefront per query atom i first tabulates it for all terms and heads in LDS
// (T * H exponentials instead of T * H per edge), then takes one edge of row i per lane; the
// cosine of a term is the real part of a product of three unit phasors, one per axis, stepped
// by rotations (6 sincos per edge instead of T cosines), and is shared by all heads.
// The backward pass tabulates |k_n|^2 exp(a |k_n|^2) as well, and reduces the edges of the
// row over the wavefront in a fixed order.
#include "cf_common.h"

namespace {

using namespace cf;

constexpr int RECI_TABLE_FLOATS = 8192;    // per table: terms x padded heads

struct ReciArgs {
    const float *a, *kr, *rvecs, *vcell;
    const int64_t *batch, *e_start;
    const float *gz, *sumexp_in;
    int64_t N, E;
    int H, R;
    int norm_grad;             // backward: include d/da of 1.5 log(-4 pi a)
    float *z, *sumexp, *ga;
};

template <int HP, bool BWD>
__global__ __launch_bounds__(WAVE) void reci_enc_kernel(ReciArgs p)
{
    extern __shared__ __align__(16) float lds[];
    const int lane = threadIdx.x;
    const int64_t i = blockIdx.x;
    const int H = p.H, R = p.R;
    const int S = 2 * R + 1;
    const int T = (R + 1) * S * S;
    float *tab = lds;                         // [T][HP]  weight * exp(a kk)
    float *tabk = lds + T * HP;               // [T][HP]  ... * kk (backward)
    const int64_t n = p.batch[i];
    float rv[9];
#pragma unroll
    for (int x = 0; x < 9; x++) rv[x] = p.rvecs[n * 9 + x];

    for (int x = lane; x < T * HP; x += WAVE) {
        const int t = x / HP, h = x - t * HP;
        const int m1 = t / (S * S);
        const int rem = t - m1 * S * S;
        const int q2 = rem / S;
        const float n1 = (float)m1, n2 = (float)(q2 - R), n3 = (float)(rem - q2 * S - R);
        const float k1 = rv[0] * n1 + rv[3] * n2 + rv[6] * n3;
        const float k2 = rv[1] * n1 + rv[4] * n2 + rv[7] * n3;
        const float k3 = rv[2] * n1 + rv[5] * n2 + rv[8] * n3;
        const float kk = k1 * k1 + k2 * k2 + k3 * k3;
        float v = 0.f;
        if (h < H) v = expf(p.a[i * H + h] * kk) * (m1 == 0 ? 1.0f : 2.0f);
        tab[x] = v;
        if (BWD) tabk[x] = v * kk;
    }
    __syncthreads();

    const int64_t e0 = p.e_start[i], e1 = p.e_start[i + 1];
    float part[HP];                           // backward: this lane's share of ga[i, h]
#pragma unroll
    for (int h = 0; h < HP; h++) part[h] = 0.f;
    for (int64_t eb = e0; eb < e1; eb += WAVE) {
        const int64_t e = eb + lane;
        const bool on = e < e1;
        const int64_t el = on ? e : e0;
        const float kr1 = p.kr[el * 3], kr2 = p.kr[el * 3 + 1], kr3 = p.kr[el * 3 + 2];
        // unit phasors: one step along each axis, and the starting points at n2 = n3 = -R
        float st1, ct1, st2, ct2, st3, ct3, s2lo, c2lo, s3lo, c3lo;
        sincosf(kr1, &st1, &ct1);
        sincosf(kr2, &st2, &ct2);
        sincosf(kr3, &st3, &ct3);
        sincosf(-(float)R * kr2, &s2lo, &c2lo);
        sincosf(-(float)R * kr3, &s3lo, &c3lo);
        float acc[HP];
#pragma unroll
        for (int h = 0; h < HP; h++) acc[h] = 0.f;
        const float *row = BWD ? tabk : tab;
        float c1 = 1.f, s1 = 0.f;
        int t = 0;
        for (int m1 = 0; m1 <= R; m1++) {
            float c2 = c2lo, s2 = s2lo;
            for (int m2 = 0; m2 < S; m2++) {
                const float c12 = c1 * c2 - s1 * s2, s12 = s1 * c2 + c1 * s2;
                float c3 = c3lo, s3 = s3lo;
                for (int m3 = 0; m3 < S; m3++, t++) {
                    const float cr = c12 * c3 - s12 * s3;
                    const float4 *w4 = reinterpret_cast<const float4 *>(row + t * HP);
#pragma unroll
                    for (int h4 = 0; h4 < HP / 4; h4++) {
                        const float4 w = w4[h4];           // same address in every lane: LDS broadcast
                        acc[4 * h4] = fmaf(w.x, cr, acc[4 * h4]);
                        acc[4 * h4 + 1] = fmaf(w.y, cr, acc[4 * h4 + 1]);
                        acc[4 * h4 + 2] = fmaf(w.z, cr, acc[4 * h4 + 2]);
                        acc[4 * h4 + 3] = fmaf(w.w, cr, acc[4 * h4 + 3]);
                    }
                    const float c3n = c3 * ct3 - s3 * st3;
                    s3 = s3 * ct3 + c3 * st3;
                    c3 = c3n;
                }
                const float c2n = c2 * ct2 - s2 * st2;
                s2 = s2 * ct2 + c2 * st2;
                c2 = c2n;
            }
            const float c1n = c1 * ct1 - s1 * st1;
            s1 = s1 * ct1 + c1 * st1;
            c1 = c1n;
        }
        if (!BWD) {
            if (on) {
                const float lv = logf(p.vcell[n]);
#pragma unroll
                for (int h = 0; h < HP; h++) {
                    if (h < H) {
                        const float a = p.a[i * H + h];
                        const float log_ci = 1.5f * logf(-12.5663706144f * a) - lv;
                        p.z[e * H + h] = logf(fmaxf(acc[h], 1e-6f)) + log_ci;
                        p.sumexp[e * H + h] = acc[h];
                    }
                }
            }
        } else {
#pragma unroll
            for (int h = 0; h < HP; h++) {
                if (on && h < H) {
                    const float se = p.sumexp_in[e * H + h];
                    const float g = p.gz[e * H + h];
                    part[h] += acc[h] * g * (se < 1e-6f ? 0.f : 1.0f / se);
                    if (p.norm_grad) part[h] += g * (1.5f / p.a[i * H + h]);
                }
            }
        }
    }
    if (BWD) {
#pragma unroll
        for (int h = 0; h < HP; h++) {
            const float s = wave_sum(part[h]);
            if (lane == 0 && h < H) p.ga[i * H + h] = s;
        }
    }
}

__global__ __launch_bounds__(256) void kr_base_kernel(const float *rpos, const float *rvecs, const int64_t *batch,
                                                      const int64_t *edges, int64_t E, float *kr)
{
    const int64_t e = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (e >= E) return;
    const float *rv = rvecs + batch[edges[e]] * 9;
    const float x = rpos[e * 3], y = rpos[e * 3 + 1], z = rpos[e * 3 + 2];
#pragma unroll
    for (int d = 0; d < 3; d++) kr[e * 3 + d] = rv[3 * d] * x + rv[3 * d + 1] * y + rv[3 * d + 2] * z;
}

template <bool BWD>
int launch_reci(const ReciArgs &p, hipStream_t st, const char *what)
{
    const int S = 2 * p.R + 1;
    const int T = (p.R + 1) * S * S;
    const int HP = p.H <= 4 ? 4 : (p.H <= 8 ? 8 : 16);
    CF_REQUIRE((int64_t)T * HP <= RECI_TABLE_FLOATS, CF_ERR_UNSUPPORTED,
               "%s: %d terms x %d heads exceed the table of %d entries", what, T, HP, RECI_TABLE_FLOATS);
    const size_t lds = (size_t)T * HP * sizeof(float) * (BWD ? 2 : 1);
    const dim3 grid((unsigned)p.N);
    switch (HP) {
        case 4: reci_enc_kernel<4, BWD><<<grid, WAVE, lds, st>>>(p); break;
        case 8: reci_enc_kernel<8, BWD><<<grid, WAVE, lds, st>>>(p); break;
        default: reci_enc_kernel<16, BWD><<<grid, WAVE, lds, st>>>(p); break;
    }
    return CF_OK;
}

}  // namespace

extern "C" int cf_kr_base(const float *rpos_ij_e, const float *rvecs_n, const int64_t *batch_i,
                          const int64_t *edge_ij_e, int64_t E, float *kr_base_e, void *stream)
{
    CF_REQUIRE(E >= 0, CF_ERR_INVALID_ARGUMENT, "cf_kr_base: negative edge count");
    if (E == 0) return CF_OK;
    CF_REQUIRE(rpos_ij_e && rvecs_n && batch_i && edge_ij_e && kr_base_e, CF_ERR_INVALID_ARGUMENT,
               "cf_kr_base: null pointer");
    kr_base_kernel<<<(unsigned)((E + 255) / 256), 256, 0, (hipStream_t)stream>>>(rpos_ij_e, rvecs_n, batch_i,
                                                                                 edge_ij_e, E, kr_base_e);
    CF_CHECK_LAUNCH("cf_kr_base");
    return CF_OK;
}

static int reci_check(const char *what, int64_t N, int64_t H, int64_t E, int lattice_range)
{
    CF_REQUIRE(N >= 0 && E >= 0 && N < (1ll << 31), CF_ERR_INVALID_ARGUMENT, "%s: bad sizes N=%lld E=%lld", what,
               (long long)N, (long long)E);
    CF_REQUIRE(H >= 1 && H <= 16, CF_ERR_UNSUPPORTED, "%s: head count %lld not served (1..16)", what, (long long)H);
    CF_REQUIRE(lattice_range >= 0 && lattice_range <= 16, CF_ERR_INVALID_ARGUMENT, "%s: lattice range %d", what,
               lattice_range);
    return CF_OK;
}

extern "C" int cf_reci_enc_fwd(const float *a_ik, const float *kr_base_e, const float *rvecs_n,
                               const float *vcell_n, const int64_t *batch_i, const int64_t *e_start_i, int64_t N,
                               int64_t H, int64_t E, int lattice_range, float *z_ek, float *sumexp_ek,
                               void *stream)
{
    int rc = reci_check("cf_reci_enc_fwd", N, H, E, lattice_range);
    if (rc) return rc;
    if (N == 0 || E == 0) return CF_OK;
    CF_REQUIRE(a_ik && kr_base_e && rvecs_n && vcell_n && batch_i && e_start_i && z_ek && sumexp_ek,
               CF_ERR_INVALID_ARGUMENT, "cf_reci_enc_fwd: null pointer");
    ReciArgs p{};
    p.a = a_ik; p.kr = kr_base_e; p.rvecs = rvecs_n; p.vcell = vcell_n; p.batch = batch_i; p.e_start = e_start_i;
    p.N = N; p.E = E; p.H = (int)H; p.R = lattice_range; p.z = z_ek; p.sumexp = sumexp_ek;
    rc = launch_reci<false>(p, (hipStream_t)stream, "cf_reci_enc_fwd");
    if (rc) return rc;
    CF_CHECK_LAUNCH("cf_reci_enc_fwd");
    return CF_OK;
}

extern "C" int cf_reci_enc_bwd(const float *a_ik, const float *kr_base_e, const float *rvecs_n,
                               const int64_t *batch_i, const int64_t *e_start_i, const float *gz_ek,
                               const float *sumexp_ek, int64_t N, int64_t H, int64_t E, int lattice_range,
                               int normalisation_grad, float *ga_ik, void *stream)
{
    int rc = reci_check("cf_reci_enc_bwd", N, H, E, lattice_range);
    if (rc) return rc;
    if (N == 0) return CF_OK;
    CF_REQUIRE(a_ik && rvecs_n && batch_i && e_start_i && ga_ik && (E == 0 || (kr_base_e && gz_ek && sumexp_ek)),
               CF_ERR_INVALID_ARGUMENT, "cf_reci_enc_bwd: null pointer");
    ReciArgs p{};
    p.a = a_ik; p.kr = kr_base_e; p.rvecs = rvecs_n; p.batch = batch_i; p.e_start = e_start_i;
    p.gz = gz_ek; p.sumexp_in = sumexp_ek;
    p.N = N; p.E = E; p.H = (int)H; p.R = lattice_range; p.norm_grad = normalisation_grad; p.ga = ga_ik;
    rc = launch_reci<true>(p, (hipStream_t)stream, "cf_reci_enc_bwd");
    if (rc) return rc;
    CF_CHECK_LAUNCH("cf_reci_enc_bwd");
    return CF_OK;
}
