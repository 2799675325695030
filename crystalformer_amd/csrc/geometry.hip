// Small per-crystal / per-atom preparation kernels for gfx950 that replace
// chains of tiny elementwise launches in front of the periodic encoding:
//   * lattice geometry: cell volume, reciprocal vectors and their lengths;
//   * Gaussian exponents: per-head tail-length logits from the query, their
//     normalisation over the batch, the positive map and the final
//     a = -rho / (2 r0^2), plus the scaled query for the attention.
#include "cf_common.h"

namespace {

using namespace cf;

// One thread per crystal.  Products and sums are kept un-contracted and in the
// term order of models/indexed_latticeformer_encoder.py:34-44 so the volume is
// the one the stock elementwise expression gives.
__global__ void lattice_geometry_kernel(const float *trans, int64_t B, float *vcell, float *recip,
                                        float *rvlen)
{
#pragma clang fp contract(off)
    const int64_t b = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (b >= B) return;
    const float *m = trans + b * 9;
    const float m00 = m[0], m01 = m[1], m02 = m[2];
    const float m10 = m[3], m11 = m[4], m12 = m[5];
    const float m20 = m[6], m21 = m[7], m22 = m[8];
    float det = m00 * m11 * m22;
    det = det + m01 * m12 * m20;
    det = det + m02 * m10 * m21;
    det = det - m02 * m11 * m20;
    det = det - m00 * m12 * m21;
    det = det - m01 * m10 * m22;
    if (vcell) vcell[b] = det;
    // b1 = 2 pi (a2 x a3) / V and cyclic (models/indexed_latticeformer_encoder.py:206-212)
    const float s = (1.0f / det) * 6.283185307179586f;
    float c[9];
    c[0] = m11 * m22 - m12 * m21;
    c[1] = m12 * m20 - m10 * m22;
    c[2] = m10 * m21 - m11 * m20;
    c[3] = m21 * m02 - m22 * m01;
    c[4] = m22 * m00 - m20 * m02;
    c[5] = m20 * m01 - m21 * m00;
    c[6] = m01 * m12 - m02 * m11;
    c[7] = m02 * m10 - m00 * m12;
    c[8] = m00 * m11 - m01 * m10;
#pragma unroll
    for (int r = 0; r < 3; r++) {
        const float x = c[3 * r] * s, y = c[3 * r + 1] * s, z = c[3 * r + 2] * s;
        if (recip) {
            recip[b * 9 + 3 * r] = x;
            recip[b * 9 + 3 * r + 1] = y;
            recip[b * 9 + 3 * r + 2] = z;
        }
        if (rvlen) rvlen[b * 3 + r] = sqrtf(x * x + y * y + z * z);
    }
}

// ---- Gaussian exponents -----------------------------------------------------
constexpr int GE_THREADS = 256;

struct GaussArgs {
    const float *q, *w;
    float *gauss_scale;
    int64_t N, H, D, total;
    int normalize, update_stats, func;
    float beta, lb, coef, q_scale;
    float *part;       // (blocks, 3): count, mean, sum of squared deviations; then (scale, shift) used and stored
    int blocks;
    float *alpha_n, *a, *q_scaled;
    const int64_t *live_N;   // nullable: the live atom count on the device (N is then the capacity)
};

// Live element count and the number of blocks that hold an element (the statistics are merged over
// exactly those, so a launch sized for a capacity gives the bits of a launch sized for the live count).
__device__ __forceinline__ int64_t live_total(const GaussArgs &p, int &blocks)
{
    if (!p.live_N) {
        blocks = p.blocks;
        return p.total;
    }
    const int64_t total = live_count(p.live_N, p.N) * p.H;
    blocks = (int)((total + GE_THREADS - 1) / GE_THREADS);
    return total;
}

__device__ __forceinline__ float positive_map(float x, int func, float beta, float lb)
{
    // models/indexed_lattice_multi_head_attention_cuda.py:675-692
    if (func == 0) {            // elu
        const float t = x * (beta / (1.0f - lb));
        return (1.0f - lb) * (t > 0.f ? t : expf(t) - 1.0f) + 1.0f;
    }
    if (func == 1) return (1.0f - lb) * fabsf(x) + lb;           // abs
    return (1.0f - lb) * expf(x * (beta / (1.0f - lb))) + lb;   // exp
}

// Chan's pairwise update of (count, mean, M2).
__device__ __forceinline__ void stat_merge(float &n, float &mean, float &m2, float nb, float meanb, float m2b)
{
    const float nt = n + nb;
    if (nt == 0.f) return;
    const float delta = meanb - mean;
    mean += delta * (nb / nt);
    m2 += m2b + delta * delta * (n * nb / nt);
    n = nt;
}

// One thread per (atom, head): alpha = <q, w_head>; the block leaves its
// (count, mean, M2).  Without normalisation the positive map is applied here.
__global__ __launch_bounds__(GE_THREADS) void gauss_exponents_alpha_kernel(GaussArgs p)
{
    __shared__ float red[GE_THREADS / WAVE][2];
    const int64_t t = (int64_t)blockIdx.x * GE_THREADS + threadIdx.x;
    int live_blocks;
    const int64_t total = live_total(p, live_blocks);
    if ((int)blockIdx.x >= live_blocks) return;
    const bool live = t < total;
    float alpha = 0.f;
    if (live) {
        const int64_t h = t % p.H;
        const float *qr = p.q + t * p.D;
        const float *wr = p.w + h * p.D;
        float *qs = p.q_scaled ? p.q_scaled + t * p.D : nullptr;
        if ((p.D & 3) == 0) {
            for (int64_t d = 0; d < p.D; d += 4) {
                const float4 qv = *reinterpret_cast<const float4 *>(qr + d);
                const float4 wv = *reinterpret_cast<const float4 *>(wr + d);
                alpha += (qv.x * wv.x + qv.y * wv.y) + (qv.z * wv.z + qv.w * wv.w);
                if (qs) *reinterpret_cast<float4 *>(qs + d) =
                    make_float4(qv.x * p.q_scale, qv.y * p.q_scale, qv.z * p.q_scale, qv.w * p.q_scale);
            }
        } else {
            for (int64_t d = 0; d < p.D; d++) {
                alpha += qr[d] * wr[d];
                if (qs) qs[d] = qr[d] * p.q_scale;
            }
        }
    }
    if (!p.normalize) {
        if (live) {
            if (p.alpha_n) p.alpha_n[t] = alpha;
            p.a[t] = positive_map(alpha, p.func, p.beta, p.lb) * p.coef;
        }
        return;
    }
    if (live) p.a[t] = alpha;
    // block statistics: mean first, then squared deviations from it
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int64_t first = (int64_t)blockIdx.x * GE_THREADS;
    const float cnt = (float)min((int64_t)GE_THREADS, total - first);
    float s = wave_sum(live ? alpha : 0.f);
    if (lane == 0) red[wave][0] = s;
    __syncthreads();
    float mean = 0.f;
    for (int w = 0; w < GE_THREADS / WAVE; w++) mean += red[w][0];
    mean /= cnt;
    const float dv = live ? alpha - mean : 0.f;
    s = wave_sum(dv * dv);
    if (lane == 0) red[wave][1] = s;
    __syncthreads();
    if (threadIdx.x == 0) {
        if (blockIdx.x == 0) {
            // snapshot of the stored statistics: the second kernel may overwrite them
            // while other blocks still need the old values
            p.part[3 * p.blocks + 2] = p.gauss_scale[0];
            p.part[3 * p.blocks + 3] = p.gauss_scale[1];
        }
        float m2 = 0.f;
        for (int w = 0; w < GE_THREADS / WAVE; w++) m2 += red[w][1];
        p.part[3 * blockIdx.x] = cnt;
        p.part[3 * blockIdx.x + 1] = mean;
        p.part[3 * blockIdx.x + 2] = m2;
    }
}

// Every block merges the block statistics in the same fixed order, picks the
// stored or the batch statistics and finishes its own elements.
__global__ __launch_bounds__(GE_THREADS) void gauss_exponents_final_kernel(GaussArgs p)
{
    __shared__ float sh[2];
    int live_blocks;
    const int64_t total = live_total(p, live_blocks);
    if ((int)blockIdx.x >= live_blocks) return;
    if (threadIdx.x < WAVE) {
        const int lane = threadIdx.x;
        float n = 0.f, mean = 0.f, m2 = 0.f;
        for (int b = lane; b < live_blocks; b += WAVE)
            stat_merge(n, mean, m2, p.part[3 * b], p.part[3 * b + 1], p.part[3 * b + 2]);
#pragma unroll
        for (int off = 1; off < WAVE; off <<= 1) {
            const float nb = __shfl_xor(n, off, WAVE), mb = __shfl_xor(mean, off, WAVE),
                        qb = __shfl_xor(m2, off, WAVE);
            // lower lane first on both sides so partners agree bit for bit
            float n0 = (lane & off) ? nb : n, m0 = (lane & off) ? mb : mean, q0 = (lane & off) ? qb : m2;
            const float n1 = (lane & off) ? n : nb, m1 = (lane & off) ? mean : mb, q1 = (lane & off) ? m2 : qb;
            stat_merge(n0, m0, q0, n1, m1, q1);
            n = n0; mean = m0; m2 = q0;
        }
        if (lane == 0) {
            const float stored_scale = p.part[3 * p.blocks + 2], stored_shift = p.part[3 * p.blocks + 3];
            const bool stored = stored_scale > 0.f;
            const float scale = stored ? stored_scale : 1.0f / sqrtf(m2 / (n - 1.0f));
            const float shift = stored ? stored_shift : -mean;
            sh[0] = scale;
            sh[1] = shift;
            if (blockIdx.x == 0) {
                p.part[3 * p.blocks] = scale;       // the pair used, for a backward pass
                p.part[3 * p.blocks + 1] = shift;
                if (p.update_stats) {
                    p.gauss_scale[0] = scale;
                    p.gauss_scale[1] = shift;
                }
            }
        }
    }
    __syncthreads();
    const float scale = sh[0], shift = sh[1];
    const int64_t t = (int64_t)blockIdx.x * GE_THREADS + threadIdx.x;
    if (t >= total) return;
    const float x = (p.a[t] + shift) * scale;
    if (p.alpha_n) p.alpha_n[t] = x;
    p.a[t] = positive_map(x, p.func, p.beta, p.lb) * p.coef;
}

// ---- Gaussian exponents, backward --------------------------------------------
struct GaussBwdArgs {
    const float *ga, *gqs, *q, *w, *alpha_n, *used_scale;
    int64_t N, H, D, total;
    int func;
    float beta, lb, coef, q_scale;
    float *part;       // (blocks, H, D) partial weight gradients
    int blocks;
    float *gq, *gw;
};

__device__ __forceinline__ float positive_map_slope(float x, int func, float beta, float lb)
{
    if (func == 0) {            // elu
        const float t = x * (beta / (1.0f - lb));
        return (t > 0.f ? 1.0f : expf(t)) * beta;
    }
    if (func == 1) return (x > 0.f ? 1.0f : (x < 0.f ? -1.0f : 0.f)) * (1.0f - lb);   // abs
    return expf(x * (beta / (1.0f - lb))) * beta;                                      // exp
}

// One thread per (atom, head): g_alpha = ga * rho'(alpha_n) * coef * scale;
// gq = g_alpha w_head + gqs * q_scale; the block leaves sum_atoms g_alpha q per (head, d),
// 16 columns of d at a time through LDS, atoms added in ascending order.
__global__ __launch_bounds__(GE_THREADS) void gauss_exponents_bwd_kernel(GaussBwdArgs p)
{
    __shared__ float prod[GE_THREADS][17];
    const int64_t first = (int64_t)blockIdx.x * GE_THREADS;
    const int64_t t = first + threadIdx.x;
    const bool live = t < p.total;
    const int64_t h = live ? t % p.H : 0;
    float g_alpha = 0.f;
    if (live && p.ga) {
        g_alpha = p.ga[t] * positive_map_slope(p.alpha_n[t], p.func, p.beta, p.lb) * p.coef;
        if (p.used_scale) g_alpha *= p.used_scale[0];
    }
    const float *qr = p.q + (live ? t : 0) * p.D;
    const float *wr = p.w + h * p.D;
    for (int64_t d0 = 0; d0 < p.D; d0 += 16) {
        const int nd = (int)min((int64_t)16, p.D - d0);
        if ((p.D & 3) == 0) {
            // rows are 16-byte aligned: four components per load and store
            typedef float float4_t __attribute__((ext_vector_type(4)));
            const float4_t zero4 = {0.f, 0.f, 0.f, 0.f};
            float4_t qv[4], wv[4], sv[4];
#pragma unroll
            for (int c4 = 0; c4 < 4; c4++) {
                const bool on = live && 4 * c4 < nd;
                qv[c4] = on ? *reinterpret_cast<const float4_t *>(qr + d0 + 4 * c4) : zero4;
                wv[c4] = on && p.gq ? *reinterpret_cast<const float4_t *>(wr + d0 + 4 * c4) : zero4;
                sv[c4] = on && p.gq && p.gqs ? *reinterpret_cast<const float4_t *>(p.gqs + t * p.D + d0 + 4 * c4) : zero4;
            }
#pragma unroll
            for (int c4 = 0; c4 < 4; c4++) {
#pragma unroll
                for (int r = 0; r < 4; r++) prod[threadIdx.x][4 * c4 + r] = g_alpha * qv[c4][r];
                if (live && p.gq && 4 * c4 < nd)
                    *reinterpret_cast<float4_t *>(p.gq + t * p.D + d0 + 4 * c4) = wv[c4] * g_alpha + sv[c4] * p.q_scale;
            }
        } else {
            for (int d = 0; d < nd; d++) {
                const float qv = live ? qr[d0 + d] : 0.f;
                prod[threadIdx.x][d] = g_alpha * qv;
                if (live && p.gq) {
                    float g = g_alpha * wr[d0 + d];
                    if (p.gqs) g += p.gqs[t * p.D + d0 + d] * p.q_scale;
                    p.gq[t * p.D + d0 + d] = g;
                }
            }
        }
        __syncthreads();
        if (p.part) {
            for (int64_t j = threadIdx.x; j < p.H * 16; j += GE_THREADS) {
                const int64_t hh = j >> 4;
                const int d = (int)(j & 15);
                if (d < nd) {
                    // first thread of this block whose head is hh
                    int tid = (int)((hh - first % p.H + p.H) % p.H);
                    float s = 0.f;
                    for (; tid < GE_THREADS; tid += (int)p.H) s += prod[tid][d];
                    p.part[((int64_t)blockIdx.x * p.H + hh) * p.D + d0 + d] = s;
                }
            }
        }
        __syncthreads();
    }
}

__global__ __launch_bounds__(256) void gauss_exponents_bwd_reduce_kernel(const float *part, int blocks, int64_t hd,
                                                                        float *gw)
{
    const int64_t x = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (x >= hd) return;
    float s0 = 0.f, s1 = 0.f;
    int b = 0;
    // 8 loads in flight; even blocks go to one running sum, odd blocks to the other
    for (; b + 7 < blocks; b += 8) {
        float v[8];
#pragma unroll
        for (int u = 0; u < 8; u++) v[u] = part[(int64_t)(b + u) * hd + x];
#pragma unroll
        for (int u = 0; u < 8; u += 2) {
            s0 += v[u];
            s1 += v[u + 1];
        }
    }
    for (; b + 1 < blocks; b += 2) {
        s0 += part[(int64_t)b * hd + x];
        s1 += part[(int64_t)(b + 1) * hd + x];
    }
    if (b < blocks) s0 += part[(int64_t)b * hd + x];
    gw[x] = s0 + s1;
}

}  // namespace

extern "C" int64_t cf_gauss_exponents_bwd_workspace(int64_t N, int64_t H, int64_t D)
{
    if (N < 0 || H < 1 || D < 1) return -1;
    const int64_t blocks = (N * H + GE_THREADS - 1) / GE_THREADS;
    return (blocks > 0 ? blocks : 1) * H * D * (int64_t)sizeof(float);
}

extern "C" int cf_gauss_exponents_bwd(const float *ga, const float *gqs, const float *q, const float *w,
                                      const float *alpha_n, const float *used_scale, int64_t N, int64_t H,
                                      int64_t D, int positive_func, float beta, float lower_bound, float coef,
                                      float q_scale, void *workspace, int64_t workspace_bytes, float *gq,
                                      float *gw, void *stream_)
{
    hipStream_t stream = (hipStream_t)stream_;
    CF_REQUIRE(N >= 0 && H >= 1 && D >= 1 && H <= 4096, CF_ERR_INVALID_ARGUMENT,
               "cf_gauss_exponents_bwd: bad sizes N=%lld H=%lld D=%lld", (long long)N, (long long)H, (long long)D);
    CF_REQUIRE(positive_func >= 0 && positive_func <= 2, CF_ERR_UNSUPPORTED,
               "cf_gauss_exponents_bwd: positive map %d not served (0 elu, 1 abs, 2 exp)", positive_func);
    CF_REQUIRE(lower_bound < 1.0f, CF_ERR_INVALID_ARGUMENT, "cf_gauss_exponents_bwd: lower bound must be < 1");
    CF_REQUIRE(gq || gw, CF_ERR_INVALID_ARGUMENT, "cf_gauss_exponents_bwd: no output requested");
    if (N == 0) {
        if (gw) {                                  // no atoms: zero gradient (the sum over zero blocks)
            gauss_exponents_bwd_reduce_kernel<<<(int)((H * D + 255) / 256), 256, 0, stream>>>(nullptr, 0, H * D, gw);
            CF_CHECK_LAUNCH("cf_gauss_exponents_bwd: zero");
        }
        return CF_OK;
    }
    CF_REQUIRE(q && w && (!ga || alpha_n), CF_ERR_INVALID_ARGUMENT, "cf_gauss_exponents_bwd: NULL operand");
    const int64_t blocks = (N * H + GE_THREADS - 1) / GE_THREADS;
    CF_REQUIRE(blocks < (1ll << 31), CF_ERR_INVALID_ARGUMENT, "cf_gauss_exponents_bwd: too many atoms");
    if (gw)
        CF_REQUIRE(workspace && workspace_bytes >= cf_gauss_exponents_bwd_workspace(N, H, D), CF_ERR_INVALID_ARGUMENT,
                   "cf_gauss_exponents_bwd: workspace of %lld bytes needed",
                   (long long)cf_gauss_exponents_bwd_workspace(N, H, D));
    GaussBwdArgs p;
    p.ga = ga; p.gqs = gqs; p.q = q; p.w = w; p.alpha_n = alpha_n; p.used_scale = used_scale;
    p.N = N; p.H = H; p.D = D; p.total = N * H;
    p.func = positive_func; p.beta = beta; p.lb = lower_bound; p.coef = coef; p.q_scale = q_scale;
    p.part = gw ? (float *)workspace : nullptr;
    p.blocks = (int)blocks;
    p.gq = gq; p.gw = gw;
    gauss_exponents_bwd_kernel<<<(int)blocks, GE_THREADS, 0, stream>>>(p);
    CF_CHECK_LAUNCH("cf_gauss_exponents_bwd");
    if (gw) {
        const int64_t hd = H * D;
        gauss_exponents_bwd_reduce_kernel<<<(int)((hd + 255) / 256), 256, 0, stream>>>(p.part, (int)blocks, hd, gw);
        CF_CHECK_LAUNCH("cf_gauss_exponents_bwd: reduce");
    }
    return CF_OK;
}

extern "C" int cf_lattice_geometry(const float *trans, int64_t B, float *vcell, float *recip, float *rvlen,
                                   void *stream_)
{
    hipStream_t stream = (hipStream_t)stream_;
    CF_REQUIRE(B >= 0, CF_ERR_INVALID_ARGUMENT, "cf_lattice_geometry: negative crystal count");
    if (B == 0) return CF_OK;
    CF_REQUIRE(trans, CF_ERR_INVALID_ARGUMENT, "cf_lattice_geometry: trans is NULL");
    CF_REQUIRE(vcell || recip || rvlen, CF_ERR_INVALID_ARGUMENT, "cf_lattice_geometry: no output requested");
    const int threads = 128;
    lattice_geometry_kernel<<<(int)((B + threads - 1) / threads), threads, 0, stream>>>(trans, B, vcell, recip,
                                                                                         rvlen);
    CF_CHECK_LAUNCH("cf_lattice_geometry");
    return CF_OK;
}

extern "C" int64_t cf_gauss_exponents_workspace(int64_t N, int64_t H)
{
    if (N < 0 || H < 0) return -1;
    const int64_t blocks = (N * H + GE_THREADS - 1) / GE_THREADS;
    return (blocks * 3 + 4) * (int64_t)sizeof(float);
}

extern "C" int cf_gauss_exponents(const float *q, const float *w, float *gauss_scale, int64_t N, int64_t H,
                                  int64_t D, int normalize, int update_stats, int positive_func, float beta,
                                  float lower_bound, float coef, float q_scale, void *workspace,
                                  int64_t workspace_bytes, float *alpha_n, float *a, float *q_scaled,
                                  void *stream_)
{
    hipStream_t stream = (hipStream_t)stream_;
    CF_REQUIRE(N >= 0 && H >= 1 && D >= 1, CF_ERR_INVALID_ARGUMENT,
               "cf_gauss_exponents: bad sizes N=%lld H=%lld D=%lld", (long long)N, (long long)H, (long long)D);
    if (N == 0) return CF_OK;
    CF_REQUIRE(q && w && a, CF_ERR_INVALID_ARGUMENT, "cf_gauss_exponents: NULL operand");
    CF_REQUIRE(positive_func >= 0 && positive_func <= 2, CF_ERR_UNSUPPORTED,
               "cf_gauss_exponents: positive map %d not served (0 elu, 1 abs, 2 exp)", positive_func);
    CF_REQUIRE(lower_bound < 1.0f, CF_ERR_INVALID_ARGUMENT, "cf_gauss_exponents: lower bound must be < 1");
    const int64_t total = N * H;
    const int64_t blocks = (total + GE_THREADS - 1) / GE_THREADS;
    CF_REQUIRE(blocks < (1ll << 31), CF_ERR_INVALID_ARGUMENT, "cf_gauss_exponents: too many atoms");
    if (normalize) {
        CF_REQUIRE(gauss_scale, CF_ERR_INVALID_ARGUMENT, "cf_gauss_exponents: gauss_scale is NULL");
        CF_REQUIRE(workspace && workspace_bytes >= cf_gauss_exponents_workspace(N, H), CF_ERR_INVALID_ARGUMENT,
                   "cf_gauss_exponents: workspace of %lld bytes needed",
                   (long long)cf_gauss_exponents_workspace(N, H));
    }
    GaussArgs p;
    p.q = q; p.w = w; p.gauss_scale = gauss_scale;
    p.N = N; p.H = H; p.D = D; p.total = total;
    p.normalize = normalize; p.update_stats = update_stats; p.func = positive_func;
    p.beta = beta; p.lb = lower_bound; p.coef = coef; p.q_scale = q_scale;
    p.part = (float *)workspace; p.blocks = (int)blocks;
    p.alpha_n = alpha_n; p.a = a; p.q_scaled = q_scaled;
    p.live_N = cf::live_atoms(N);
    gauss_exponents_alpha_kernel<<<(int)blocks, GE_THREADS, 0, stream>>>(p);
    CF_CHECK_LAUNCH("cf_gauss_exponents: alpha");
    if (normalize) {
        gauss_exponents_final_kernel<<<(int)blocks, GE_THREADS, 0, stream>>>(p);
        CF_CHECK_LAUNCH("cf_gauss_exponents: normalise");
    }
    return CF_OK;
}
