// Real-space periodic encoding for gfx950: the lattice sum of Gaussian distance
// decay (attention bias z) and the K-bin Gaussian value position encoding (v),
// forward and backward.
//
// Work decomposition (wave64):
//   * one wavefront owns one edge (i -> j) and walks the translation box in
//     chunks of 64 translations;
//   * "wide" phase, lane = translation: geometry d^2(n), sqrt, and the H
//     per-head weights exp(a_h (d^2 - d^2_min)) are evaluated once per
//     translation and shared by all bins;
//   * "deep" phase, lane = Gaussian bin: the 64 translations of the chunk are
//     replayed one by one, their distance and head weights broadcast out of the
//     owning lane with v_readlane, each lane evaluating its own bin's Gaussian
//     once and feeding H accumulators;
//   * epilogue: the H x K sums are staged in LDS and multiplied by the D x K
//     projection (also LDS resident) with lane = (head, output row).
//
// All exponentials go through v_exp_f32 with log2(e) folded into the operands.
#include "cf_common.h"

#include <mutex>

namespace {

using namespace cf;

struct EncArgs {
    const float *a_ik;
    const float *rpos;
    const float *tvecs;
    const int64_t *batch;
    const int64_t *edges;
    const int64_t *e_start;
    const float *W;
    const float *rvlen;
    const float *z_in;
    const float *gz;
    const float *gv;
    float *z;
    float *v;
    float *ga_edge;   // (E,H) per-edge contributions to ga
    float *sv_out;    // (E,H,K) normalised Gaussian averages (for gW)
    int64_t N, E;
    int64_t W_num;
    int K, D;
    float cutoff;
    int lattice_range, min_range;
    float bin_step;   // sqrt(log2 e) / (ws*sqrt 2): Gaussian argument per bin index
    float s_scale;    // bin_step / mu0: distance -> Gaussian argument
};

// Geometry of one translation.
struct Cell {
    float rx, ry, rz;
    float t[9];
};

__device__ __forceinline__ float dist2(const Cell &c, float n1, float n2, float n3)
{
    float dx = c.rx + c.t[0] * n1 + c.t[3] * n2 + c.t[6] * n3;
    float dy = c.ry + c.t[1] * n1 + c.t[4] * n2 + c.t[7] * n3;
    float dz = c.rz + c.t[2] * n1 + c.t[5] * n2 + c.t[8] * n3;
    return dx * dx + dy * dy + dz * dz;
}

// Translation box of one edge: union over heads, plus the per-head boxes when
// they differ.
template <int H>
struct Box {
    int U1, U2, U3;      // union half-widths
    int S2, S3, T;       // strides and translation count of the union box
    bool uniform;        // every head uses the union box
    int R1[H], R2[H], R3[H];
};

template <int H>
__device__ __forceinline__ void make_box(Box<H> &box, const float *a, float cutoff,
                                         const float *rvl, int lattice_range, int min_range)
{
    box.U1 = box.U2 = box.U3 = 0;
    bool uni = true;
#pragma unroll
    for (int h = 0; h < H; h++) {
        range_rule(a[h], cutoff, rvl, lattice_range, min_range, box.R1[h], box.R2[h], box.R3[h]);
        box.U1 = max(box.U1, box.R1[h]);
        box.U2 = max(box.U2, box.R2[h]);
        box.U3 = max(box.U3, box.R3[h]);
    }
#pragma unroll
    for (int h = 0; h < H; h++)
        uni = uni && box.R1[h] == box.U1 && box.R2[h] == box.U2 && box.R3[h] == box.U3;
    box.uniform = uni;
    box.S3 = 2 * box.U3 + 1;
    box.S2 = 2 * box.U2 + 1;
    box.T = (2 * box.U1 + 1) * box.S2 * box.S3;
}

template <int H>
__device__ __forceinline__ void decode(const Box<H> &box, int idx, int &n1, int &n2, int &n3)
{
    int plane = box.S2 * box.S3;
    int q1 = idx / plane;
    int rem = idx - q1 * plane;
    int q2 = rem / box.S3;
    n1 = q1 - box.U1;
    n2 = q2 - box.U2;
    n3 = rem - q2 * box.S3 - box.U3;
}

template <int H>
__device__ __forceinline__ bool inside(const Box<H> &box, int h, int n1, int n2, int n3)
{
    return abs(n1) <= box.R1[h] && abs(n2) <= box.R2[h] && abs(n3) <= box.R3[h];
}

__device__ __forceinline__ void load_cell(Cell &c, const EncArgs &p, int64_t e, int64_t n)
{
    const float *r = p.rpos + e * 3;
    c.rx = r[0];
    c.ry = r[1];
    c.rz = r[2];
    const float *t = p.tvecs + n * 9;
#pragma unroll
    for (int x = 0; x < 9; x++) c.t[x] = t[x];
}

// Per-head minimum of d^2 over the head's own box (wave-uniform result).
template <int H>
__device__ __forceinline__ void box_minimum(const Box<H> &box, const Cell &c, int lane,
                                            float *d2min)
{
    float m[H];
#pragma unroll
    for (int h = 0; h < H; h++) m[h] = 1e10f;
    for (int c0 = 0; c0 < box.T; c0 += WAVE) {
        int idx = c0 + lane;
        if (idx < box.T) {
            int n1, n2, n3;
            decode(box, idx, n1, n2, n3);
            float d2 = dist2(c, (float)n1, (float)n2, (float)n3);
            if (box.uniform) {
                m[0] = fminf(m[0], d2);
            } else {
#pragma unroll
                for (int h = 0; h < H; h++)
                    if (inside(box, h, n1, n2, n3)) m[h] = fminf(m[h], d2);
            }
        }
    }
    if (box.uniform) {
        float v = wave_min(m[0]);
#pragma unroll
        for (int h = 0; h < H; h++) d2min[h] = v;
    } else {
#pragma unroll
        for (int h = 0; h < H; h++) d2min[h] = wave_min(m[h]);
    }
}

// ---------------------------------------------------------------------------
// forward, K == 0: bias only.  lane = translation.
// ---------------------------------------------------------------------------
template <int H>
__global__ __launch_bounds__(256) void real_enc_fwd_bias_kernel(EncArgs p)
{
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int wpb = blockDim.x >> 6;
    for (int64_t e = (int64_t)blockIdx.x * wpb + wave; e < p.E; e += (int64_t)gridDim.x * wpb) {
        const int64_t i = p.edges[e];
        const int64_t n = p.batch[i];
        Cell c;
        load_cell(c, p, e, n);
        float a[H];
#pragma unroll
        for (int h = 0; h < H; h++) a[h] = p.a_ik[i * H + h];
        float rvl[3] = {0.f, 0.f, 0.f};
        if (p.rvlen) {
            rvl[0] = p.rvlen[n * 3 + 0];
            rvl[1] = p.rvlen[n * 3 + 1];
            rvl[2] = p.rvlen[n * 3 + 2];
        }
        Box<H> box;
        make_box(box, a, p.cutoff, rvl, p.lattice_range, p.min_range);
        float d2min[H];
        box_minimum(box, c, lane, d2min);
        float sum[H];
#pragma unroll
        for (int h = 0; h < H; h++) sum[h] = 0.f;
        for (int c0 = 0; c0 < box.T; c0 += WAVE) {
            int idx = c0 + lane;
            if (idx < box.T) {
                int n1, n2, n3;
                decode(box, idx, n1, n2, n3);
                float d2 = dist2(c, (float)n1, (float)n2, (float)n3);
#pragma unroll
                for (int h = 0; h < H; h++) {
                    float w = exp2_hw(a[h] * LOG2E * (d2 - d2min[h]));
                    if (!box.uniform && !inside(box, h, n1, n2, n3)) w = 0.f;
                    sum[h] += w;
                }
            }
        }
#pragma unroll
        for (int h = 0; h < H; h++) {
            float s = wave_sum(sum[h]);
            if (lane == h) p.z[e * H + h] = log2_hw(s) * LN2 + d2min[h] * a[h];
        }
    }
}

// ---------------------------------------------------------------------------
// forward, K == 0, fused with the attention that consumes the bias: one work-group per query
// atom.  Phase 1 (a wavefront per edge of the row, lane = translation) forms the lattice-sum
// bias z of the row exactly as the kernel above does and leaves it in LDS; phase 2 adds the
// scaled dot products q_i . k_j (thread = (key, head)); phase 3 is the softmax over the row's
// keys (a wavefront per head); phase 4 aggregates the values (thread = (head, component)).
// Neither z nor the probabilities ever reach HBM.  The unordered-pair trick of the matrix-core
// kernel buys nothing here: without Gaussian bins the exponentials are per (edge, head) anyway
// and only the distance of a translation would be shared.
// LDS: logits / probabilities [row length][H], key atoms [row length].
// ---------------------------------------------------------------------------
struct RowArgs {
    const float *que, *key, *val;
    float *out;
    int Dk, Dv;
    int max_row;
};

template <int H>
__global__ __launch_bounds__(1024) void enc_dpa_row_kernel(EncArgs p, RowArgs r)
{
    extern __shared__ float lds[];
    float *zl = lds;                                            // [row][H]
    int *jl = reinterpret_cast<int *>(lds + (size_t)r.max_row * H);   // [row]
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int wpb = blockDim.x >> 6;
    const int64_t i = blockIdx.x;
    const int64_t e0 = p.e_start[i];
    const int n = (int)(p.e_start[i + 1] - e0);
    const int Dk = r.Dk, Dv = r.Dv;
    if (n == 0) {                                               // an atom without edges: zero row
        for (int x = threadIdx.x; x < H * Dv; x += blockDim.x) r.out[i * H * Dv + x] = 0.f;
        return;
    }
    if (n > r.max_row) {
        // a row longer than the bound the caller gave (the LDS was sized with it): nothing of the
        // row may be staged; the output row is NaN so that the broken promise cannot pass for a result
        for (int x = threadIdx.x; x < H * Dv; x += blockDim.x) r.out[i * H * Dv + x] = __builtin_nanf("");
        return;
    }
    // ---- phase 1: lattice sums of the row
    {
        const int64_t nb = p.batch[i];
        float a[H];
#pragma unroll
        for (int h = 0; h < H; h++) a[h] = p.a_ik[i * H + h];
        float rvl[3] = {0.f, 0.f, 0.f};
        if (p.rvlen) {
            rvl[0] = p.rvlen[nb * 3 + 0];
            rvl[1] = p.rvlen[nb * 3 + 1];
            rvl[2] = p.rvlen[nb * 3 + 2];
        }
        Box<H> box;
        make_box(box, a, p.cutoff, rvl, p.lattice_range, p.min_range);
        // The box belongs to the row's atom: boxes of up to 128 translations (the default cube has
        // 125) are decoded once, two translations per lane, with the heads whose own box holds
        // them as a bit set; every edge of the row then costs two distance evaluations per lane.
        const bool small = box.T <= 2 * WAVE;
        float nf[2][3] = {{0.f, 0.f, 0.f}, {0.f, 0.f, 0.f}};
        int hbits[2] = {0, 0};
        if (small) {
#pragma unroll
            for (int ch = 0; ch < 2; ch++) {
                const int idx = ch * WAVE + lane;
                if (idx < box.T) {
                    int n1, n2, n3;
                    decode(box, idx, n1, n2, n3);
                    nf[ch][0] = (float)n1;
                    nf[ch][1] = (float)n2;
                    nf[ch][2] = (float)n3;
#pragma unroll
                    for (int h = 0; h < H; h++)
                        if (box.uniform || inside(box, h, n1, n2, n3)) hbits[ch] |= 1 << h;
                }
            }
        }
        for (int jj = wave; jj < n; jj += wpb) {
            const int64_t e = e0 + jj;
            Cell c;
            load_cell(c, p, e, nb);
            float d2min[H];
            float sum[H];
#pragma unroll
            for (int h = 0; h < H; h++) sum[h] = 0.f;
            if (small) {
                float d2[2];
#pragma unroll
                for (int ch = 0; ch < 2; ch++) d2[ch] = dist2(c, nf[ch][0], nf[ch][1], nf[ch][2]);
                if (box.uniform) {
                    const float m = wave_min(fminf(hbits[0] ? d2[0] : 1e10f, hbits[1] ? d2[1] : 1e10f));
#pragma unroll
                    for (int h = 0; h < H; h++) d2min[h] = m;
                } else {
#pragma unroll
                    for (int h = 0; h < H; h++)
                        d2min[h] = wave_min(fminf((hbits[0] >> h) & 1 ? d2[0] : 1e10f,
                                                  (hbits[1] >> h) & 1 ? d2[1] : 1e10f));
                }
#pragma unroll
                for (int ch = 0; ch < 2; ch++)
#pragma unroll
                    for (int h = 0; h < H; h++) {
                        const float w = exp2_hw(a[h] * LOG2E * (d2[ch] - d2min[h]));
                        sum[h] += ((hbits[ch] >> h) & 1) ? w : 0.f;
                    }
            } else {
                box_minimum(box, c, lane, d2min);
                for (int c0 = 0; c0 < box.T; c0 += WAVE) {
                    int idx = c0 + lane;
                    if (idx < box.T) {
                        int n1, n2, n3;
                        decode(box, idx, n1, n2, n3);
                        float d2 = dist2(c, (float)n1, (float)n2, (float)n3);
#pragma unroll
                        for (int h = 0; h < H; h++) {
                            float w = exp2_hw(a[h] * LOG2E * (d2 - d2min[h]));
                            if (!box.uniform && !inside(box, h, n1, n2, n3)) w = 0.f;
                            sum[h] += w;
                        }
                    }
                }
            }
#pragma unroll
            for (int h = 0; h < H; h++) {
                float s = wave_sum(sum[h]);
                if (lane == h) zl[jj * H + h] = log2_hw(s) * LN2 + d2min[h] * a[h];
            }
            if (lane == 0) jl[jj] = (int)p.edges[p.E + e];
        }
    }
    __syncthreads();
    // ---- phase 2: logits q_i . k_j + z (the query comes pre-divided by sqrt(Dk))
    for (int x = threadIdx.x; x < n * H; x += blockDim.x) {
        const int jj = x / H, h = x - jj * H;
        const float *qp = r.que + (i * H + h) * Dk;
        const float *kp = r.key + ((int64_t)jl[jj] * H + h) * Dk;
        float s = 0.f;
        for (int d = 0; d < Dk; d++) s = fmaf(qp[d], kp[d], s);
        zl[x] += s;
    }
    __syncthreads();
    // ---- phase 3: softmax over the keys of the row, a wavefront per head
    for (int h = wave; h < H; h += wpb) {
        float m = -3.0e38f;
        for (int jj = lane; jj < n; jj += WAVE) m = fmaxf(m, zl[jj * H + h]);
        m = wave_max(m);
        float sum = 0.f;
        for (int jj = lane; jj < n; jj += WAVE) {
            const float w = exp2_hw((zl[jj * H + h] - m) * LOG2E);
            zl[jj * H + h] = w;
            sum += w;
        }
        const float inv = 1.0f / wave_sum(sum);
        for (int jj = lane; jj < n; jj += WAVE) zl[jj * H + h] *= inv;
    }
    __syncthreads();
    // ---- phase 4: out[i,h,:] = sum_j p_ij v_j
    for (int x = threadIdx.x; x < H * Dv; x += blockDim.x) {
        const int h = x / Dv;
        float acc0 = 0.f, acc1 = 0.f;
        int jj = 0;
        for (; jj + 1 < n; jj += 2) {
            acc0 = fmaf(zl[jj * H + h], r.val[(int64_t)jl[jj] * H * Dv + x], acc0);
            acc1 = fmaf(zl[(jj + 1) * H + h], r.val[(int64_t)jl[jj + 1] * H * Dv + x], acc1);
        }
        if (jj < n) acc0 = fmaf(zl[jj * H + h], r.val[(int64_t)jl[jj] * H * Dv + x], acc0);
        r.out[i * H * Dv + x] = acc0 + acc1;
    }
}

// ---------------------------------------------------------------------------
// forward, K > 0.  NB = bins per lane (K <= 64*NB).
// LDS: [W: H*D*KP floats if PROJ && W_num==1][per wave: H*KP floats]
// ---------------------------------------------------------------------------
template <int H, int NB, bool PROJ>
__global__ __launch_bounds__(256) void real_enc_fwd_kernel(EncArgs p)
{
    extern __shared__ float lds[];
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int wpb = blockDim.x >> 6;
    const int K = p.K, D = p.D;
    const int KP = NB * WAVE + 1;
    const bool w_shared = PROJ && p.W_num == 1;
    float *Wl = lds;
    float *Sl = lds + (w_shared ? H * D * KP : 0) + wave * H * KP;
    if (w_shared) {
        for (int x = threadIdx.x; x < H * D * K; x += blockDim.x) {
            int hd = x / K, k = x - hd * K;
            Wl[hd * KP + k] = p.W[x];
        }
        __syncthreads();
    }
    // Gaussian argument of this lane's bins at distance 0: bin_step * (k+1).
    float ck[NB];
#pragma unroll
    for (int nb = 0; nb < NB; nb++) ck[nb] = p.bin_step * (float)(lane + nb * WAVE + 1);

    for (int64_t e = (int64_t)blockIdx.x * wpb + wave; e < p.E; e += (int64_t)gridDim.x * wpb) {
        const int64_t i = p.edges[e];
        const int64_t n = p.batch[i];
        Cell c;
        load_cell(c, p, e, n);
        float a[H];
#pragma unroll
        for (int h = 0; h < H; h++) a[h] = p.a_ik[i * H + h];
        float rvl[3] = {0.f, 0.f, 0.f};
        if (p.rvlen) {
            rvl[0] = p.rvlen[n * 3 + 0];
            rvl[1] = p.rvlen[n * 3 + 1];
            rvl[2] = p.rvlen[n * 3 + 2];
        }
        Box<H> box;
        make_box(box, a, p.cutoff, rvl, p.lattice_range, p.min_range);
        float d2min[H];
        box_minimum(box, c, lane, d2min);

        float sum[H];
        float S[H][NB];
#pragma unroll
        for (int h = 0; h < H; h++) {
            sum[h] = 0.f;
#pragma unroll
            for (int nb = 0; nb < NB; nb++) S[h][nb] = 0.f;
        }
        for (int c0 = 0; c0 < box.T; c0 += WAVE) {
            // wide phase: lane = translation
            int idx = c0 + lane;
            bool valid = idx < box.T;
            int n1, n2, n3;
            decode(box, valid ? idx : 0, n1, n2, n3);
            float d2 = dist2(c, (float)n1, (float)n2, (float)n3);
            float s = sqrt_hw(d2) * p.s_scale;
            float w[H];
#pragma unroll
            for (int h = 0; h < H; h++) {
                float x = exp2_hw(a[h] * LOG2E * (d2 - d2min[h]));
                bool on = valid && (box.uniform || inside(box, h, n1, n2, n3));
                w[h] = on ? x : 0.f;
                sum[h] += w[h];
            }
            // deep phase: lane = bin
            // (translations past the end of the box carry zero weight, so the
            // replay may run to the next multiple of 4)
            const int cnt = min(WAVE, (box.T - c0 + 3) & ~3);
            for (int t0 = 0; t0 < cnt; t0 += 4) {
#pragma unroll
                for (int u = 0; u < 4; u++) {
                    const int t = t0 + u;
                    float st = readlane_f(s, t);
                    float g[NB];
#pragma unroll
                    for (int nb = 0; nb < NB; nb++) {
                        float b = ck[nb] - st;
                        g[nb] = exp2_hw(-(b * b));
                    }
#pragma unroll
                    for (int h = 0; h < H; h++) {
                        float wt = readlane_f(w[h], t);
#pragma unroll
                        for (int nb = 0; nb < NB; nb++) S[h][nb] = fmaf(wt, g[nb], S[h][nb]);
                    }
                }
            }
        }
        float inv[H];
#pragma unroll
        for (int h = 0; h < H; h++) {
            float tot = wave_sum(sum[h]);
            inv[h] = 1.0f / tot;
            if (lane == h) p.z[e * H + h] = log2_hw(tot) * LN2 + d2min[h] * a[h];
        }
        if (!PROJ) {
#pragma unroll
            for (int h = 0; h < H; h++)
#pragma unroll
                for (int nb = 0; nb < NB; nb++) {
                    int k = lane + nb * WAVE;
                    if (k < K) p.v[(e * H + h) * K + k] = S[h][nb] * inv[h];
                }
        } else {
            // stage the normalised H x K sums, then lane = (head, output row)
#pragma unroll
            for (int h = 0; h < H; h++)
#pragma unroll
                for (int nb = 0; nb < NB; nb++) {
                    int k = lane + nb * WAVE;
                    Sl[h * KP + k] = (k < K) ? S[h][nb] * inv[h] : 0.f;
                }
            wave_mem_sync();
            int64_t w_ind = 0;
            if (p.W_num == 1) w_ind = 0;
            else if (p.W_num == p.E) w_ind = e;
            else if (p.W_num == p.N) w_ind = i;
            const float *Wg = p.W + w_ind * (int64_t)H * D * K;
            for (int x = lane; x < H * D; x += WAVE) {
                int h = x / D;
                const float *srow = Sl + h * KP;
                float acc = 0.f;
                if (w_shared) {
                    const float *wrow = Wl + x * KP;
                    for (int k = 0; k < K; k++) acc = fmaf(wrow[k], srow[k], acc);
                } else {
                    const float *wrow = Wg + (int64_t)x * K;
                    for (int k = 0; k < K; k++) acc = fmaf(wrow[k], srow[k], acc);
                }
                p.v[e * (int64_t)H * D + x] = acc;
            }
            wave_mem_sync();
        }
    }
}

// ---------------------------------------------------------------------------
// backward.  Per edge and head:
//   p_n = exp(a d2_n - z), PX = sum_n p_n d2_n,
//   S_k = sum_n p_n g_k(n), Q_k = sum_n p_n d2_n g_k(n),
//   ga_e = gz PX + sum_k sgv_k Q_k - PX sum_k sgv_k S_k,
//   sgv_k = sum_d W[d,k] gv_d (or gv_k without projection).
// S is also written out (normalised Gaussian averages) for the gW reduction.
// LDS: [W: H*D*KP floats if PROJ && W_num==1]
// ---------------------------------------------------------------------------
template <int H, int NB, bool PROJ>
__global__ __launch_bounds__(256) void real_enc_bwd_kernel(EncArgs p)
{
    extern __shared__ float lds[];
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int wpb = blockDim.x >> 6;
    const int K = p.K, D = p.D;
    const int KP = NB * WAVE + 1;
    const bool w_shared = PROJ && p.W_num == 1;
    float *Wl = lds;
    if (w_shared) {
        for (int x = threadIdx.x; x < H * D * K; x += blockDim.x) {
            int hd = x / K, k = x - hd * K;
            Wl[hd * KP + k] = p.W[x];
        }
        __syncthreads();
    }
    float ck[NB];
#pragma unroll
    for (int nb = 0; nb < NB; nb++) ck[nb] = p.bin_step * (float)(lane + nb * WAVE + 1);

    for (int64_t e = (int64_t)blockIdx.x * wpb + wave; e < p.E; e += (int64_t)gridDim.x * wpb) {
        const int64_t i = p.edges[e];
        const int64_t n = p.batch[i];
        Cell c;
        load_cell(c, p, e, n);
        float a[H], zl[H];
#pragma unroll
        for (int h = 0; h < H; h++) {
            a[h] = p.a_ik[i * H + h];
            zl[h] = p.z_in[e * H + h] * LOG2E;
        }
        float rvl[3] = {0.f, 0.f, 0.f};
        if (p.rvlen) {
            rvl[0] = p.rvlen[n * 3 + 0];
            rvl[1] = p.rvlen[n * 3 + 1];
            rvl[2] = p.rvlen[n * 3 + 2];
        }
        Box<H> box;
        make_box(box, a, p.cutoff, rvl, p.lattice_range, p.min_range);

        // sgv[h][nb]: upstream gradient folded onto this lane's bins
        float sgv[H][NB];
        if (!p.gv) {
#pragma unroll
            for (int h = 0; h < H; h++)
#pragma unroll
                for (int nb = 0; nb < NB; nb++) sgv[h][nb] = 0.f;
        } else if (!PROJ) {
#pragma unroll
            for (int h = 0; h < H; h++)
#pragma unroll
                for (int nb = 0; nb < NB; nb++) {
                    int k = lane + nb * WAVE;
                    sgv[h][nb] = (k < K) ? p.gv[(e * H + h) * K + k] : 0.f;
                }
        } else {
            int64_t w_ind = 0;
            if (p.W_num == 1) w_ind = 0;
            else if (p.W_num == p.E) w_ind = e;
            else if (p.W_num == p.N) w_ind = i;
            const float *Wg = p.W + w_ind * (int64_t)H * D * K;
            const float *gve = p.gv + e * (int64_t)H * D;
#pragma unroll
            for (int h = 0; h < H; h++) {
#pragma unroll
                for (int nb = 0; nb < NB; nb++) sgv[h][nb] = 0.f;
                for (int d = 0; d < D; d++) {
                    float g = gve[h * D + d];   // wave-uniform load
#pragma unroll
                    for (int nb = 0; nb < NB; nb++) {
                        int k = lane + nb * WAVE;
                        float wv = 0.f;
                        if (k < K)
                            wv = w_shared ? Wl[(h * D + d) * KP + k] : Wg[((int64_t)h * D + d) * K + k];
                        sgv[h][nb] = fmaf(wv, g, sgv[h][nb]);
                    }
                }
            }
        }

        float px[H];
        float S[H][NB], Q[H][NB];
#pragma unroll
        for (int h = 0; h < H; h++) {
            px[h] = 0.f;
#pragma unroll
            for (int nb = 0; nb < NB; nb++) S[h][nb] = Q[h][nb] = 0.f;
        }
        for (int c0 = 0; c0 < box.T; c0 += WAVE) {
            int idx = c0 + lane;
            bool valid = idx < box.T;
            int n1, n2, n3;
            decode(box, valid ? idx : 0, n1, n2, n3);
            float d2 = dist2(c, (float)n1, (float)n2, (float)n3);
            float s = sqrt_hw(d2) * p.s_scale;
            float w[H], wq[H];
#pragma unroll
            for (int h = 0; h < H; h++) {
                float x = exp2_hw(a[h] * LOG2E * d2 - zl[h]);
                bool on = valid && (box.uniform || inside(box, h, n1, n2, n3));
                w[h] = on ? x : 0.f;
                wq[h] = w[h] * d2;
                px[h] += wq[h];
            }
            if (K > 0) {
                const int cnt = min(WAVE, (box.T - c0 + 1) & ~1);
                for (int t0 = 0; t0 < cnt; t0 += 2) {
#pragma unroll
                    for (int u = 0; u < 2; u++) {
                        const int t = t0 + u;
                        float st = readlane_f(s, t);
                        float g[NB];
#pragma unroll
                        for (int nb = 0; nb < NB; nb++) {
                            float b = ck[nb] - st;
                            g[nb] = exp2_hw(-(b * b));
                        }
#pragma unroll
                        for (int h = 0; h < H; h++) {
                            float wt = readlane_f(w[h], t);
                            float qt = readlane_f(wq[h], t);
#pragma unroll
                            for (int nb = 0; nb < NB; nb++) {
                                S[h][nb] = fmaf(wt, g[nb], S[h][nb]);
                                Q[h][nb] = fmaf(qt, g[nb], Q[h][nb]);
                            }
                        }
                    }
                }
            }
        }
#pragma unroll
        for (int h = 0; h < H; h++) {
            float PX = wave_sum(px[h]);
            float A = 0.f, Bv = 0.f;
#pragma unroll
            for (int nb = 0; nb < NB; nb++) {
                A = fmaf(sgv[h][nb], Q[h][nb], A);
                Bv = fmaf(sgv[h][nb], S[h][nb], Bv);
            }
            A = wave_sum(A);
            Bv = wave_sum(Bv);
            if (lane == h) {
                float gz = p.gz ? p.gz[e * H + h] : 0.f;
                p.ga_edge[e * H + h] = PX * gz + (A - PX * Bv);
            }
            if (p.sv_out) {
#pragma unroll
                for (int nb = 0; nb < NB; nb++) {
                    int k = lane + nb * WAVE;
                    if (k < K) p.sv_out[(e * H + h) * K + k] = S[h][nb];
                }
            }
        }
    }
}

// backward, K == 0: ga_e = gz * sum_n p_n d2_n.  lane = translation.
template <int H>
__global__ __launch_bounds__(256) void real_enc_bwd_bias_kernel(EncArgs p)
{
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int wpb = blockDim.x >> 6;
    for (int64_t e = (int64_t)blockIdx.x * wpb + wave; e < p.E; e += (int64_t)gridDim.x * wpb) {
        const int64_t i = p.edges[e];
        const int64_t n = p.batch[i];
        Cell c;
        load_cell(c, p, e, n);
        float a[H], zl[H];
#pragma unroll
        for (int h = 0; h < H; h++) {
            a[h] = p.a_ik[i * H + h];
            zl[h] = p.z_in[e * H + h] * LOG2E;
        }
        float rvl[3] = {0.f, 0.f, 0.f};
        if (p.rvlen) {
            rvl[0] = p.rvlen[n * 3 + 0];
            rvl[1] = p.rvlen[n * 3 + 1];
            rvl[2] = p.rvlen[n * 3 + 2];
        }
        Box<H> box;
        make_box(box, a, p.cutoff, rvl, p.lattice_range, p.min_range);
        float px[H];
#pragma unroll
        for (int h = 0; h < H; h++) px[h] = 0.f;
        for (int c0 = 0; c0 < box.T; c0 += WAVE) {
            int idx = c0 + lane;
            if (idx < box.T) {
                int n1, n2, n3;
                decode(box, idx, n1, n2, n3);
                float d2 = dist2(c, (float)n1, (float)n2, (float)n3);
#pragma unroll
                for (int h = 0; h < H; h++) {
                    float x = exp2_hw(a[h] * LOG2E * d2 - zl[h]) * d2;
                    if (!box.uniform && !inside(box, h, n1, n2, n3)) x = 0.f;
                    px[h] += x;
                }
            }
        }
#pragma unroll
        for (int h = 0; h < H; h++) {
            float PX = wave_sum(px[h]);
            if (lane == h) p.ga_edge[e * H + h] = PX * (p.gz ? p.gz[e * H + h] : 0.f);
        }
    }
}

// ga[i,h] = sum over the atom's edge row of ga_edge, fixed order (8 interleaved
// partial sums, then a tree), one thread per (atom, head).
__global__ void reduce_ga_kernel(const float *ga_edge, const int64_t *e_start, int64_t N, int H,
                                 float *ga)
{
    int64_t tid = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (tid >= N * H) return;
    int64_t i = tid / H;
    int h = (int)(tid - i * H);
    int64_t e0 = e_start[i], e1 = e_start[i + 1];
    float acc[8] = {0, 0, 0, 0, 0, 0, 0, 0};
    int64_t e = e0;
    for (; e + 8 <= e1; e += 8)
#pragma unroll
        for (int u = 0; u < 8; u++) acc[u] += ga_edge[(e + u) * H + h];
    for (int u = 0; e < e1; e++, u++) acc[u] += ga_edge[e * H + h];
    ga[tid] = ((acc[0] + acc[1]) + (acc[2] + acc[3])) + ((acc[4] + acc[5]) + (acc[6] + acc[7]));
}

// gW partial sums: block (h, split) accumulates gv[e,h,d] * sv[e,h,k] over its
// slice of edges, thread = (d,k) pairs.  part is (splits,H,D,K).
__global__ __launch_bounds__(256) void gw_partial_kernel(const float *gv, const float *sv,
                                                         int64_t E, int H, int D, int K,
                                                         int splits, float *part)
{
    const int h = blockIdx.x % H;
    const int sp = blockIdx.x / H;
    const int64_t per = (E + splits - 1) / splits;
    const int64_t e0 = sp * per, e1 = min(E, e0 + per);
    const int DK = D * K;
    for (int x0 = 0; x0 < DK; x0 += 256 * 4) {
        float acc[4] = {0, 0, 0, 0};
        int d[4], k[4];
#pragma unroll
        for (int u = 0; u < 4; u++) {
            int x = x0 + threadIdx.x + u * 256;
            d[u] = x < DK ? x / K : 0;
            k[u] = x < DK ? x - d[u] * K : 0;
        }
        for (int64_t e = e0; e < e1; e++) {
            const float *g = gv + (e * H + h) * D;
            const float *s = sv + (e * H + h) * K;
#pragma unroll
            for (int u = 0; u < 4; u++) acc[u] = fmaf(g[d[u]], s[k[u]], acc[u]);
        }
#pragma unroll
        for (int u = 0; u < 4; u++) {
            int x = x0 + threadIdx.x + u * 256;
            if (x < DK) part[((int64_t)sp * H + h) * DK + x] = acc[u];
        }
    }
}

__global__ void gw_final_kernel(const float *part, int splits, int64_t HDK, float *gW)
{
    int64_t x = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (x >= HDK) return;
    float acc = 0.f;
    for (int s = 0; s < splits; s++) acc += part[(int64_t)s * HDK + x];
    gW[x] = acc;
}

// per-edge / per-atom W: gW[w,h,d,k] = sum over the edges that use slot w.
// W_num == E: one edge per slot.  W_num == N: the atom's edge row.
__global__ void gw_indexed_kernel(const float *gv, const float *sv, const int64_t *e_start,
                                  int64_t W_num, int64_t E, int H, int D, int K, float *gW)
{
    int64_t x = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    int64_t total = W_num * H * D * K;
    if (x >= total) return;
    int k = (int)(x % K);
    int d = (int)((x / K) % D);
    int h = (int)((x / ((int64_t)K * D)) % H);
    int64_t w = x / ((int64_t)K * D * H);
    int64_t e0 = w, e1 = w + 1;
    if (W_num != E) {
        e0 = e_start[w];
        e1 = e_start[w + 1];
    }
    float acc = 0.f;
    for (int64_t e = e0; e < e1; e++) acc = fmaf(gv[(e * H + h) * D + d], sv[(e * H + h) * K + k], acc);
    gW[x] = acc;
}

__global__ void fill_zero_kernel(float *dst, int64_t n)
{
    int64_t x = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (x < n) dst[x] = 0.f;
}

__global__ void translation_ranges_kernel(const float *a_ik, const float *rvlen, const int64_t *batch,
                                          int64_t N, int H, float cutoff, int lattice_range,
                                          int min_range, int32_t *R_out)
{
    int64_t tid = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (tid >= N * H) return;
    int64_t i = tid / H;
    float rvl[3] = {0.f, 0.f, 0.f};
    if (rvlen) {
        int64_t n = batch[i];
        rvl[0] = rvlen[n * 3];
        rvl[1] = rvlen[n * 3 + 1];
        rvl[2] = rvlen[n * 3 + 2];
    }
    int R1, R2, R3;
    range_rule(a_ik[tid], rvlen ? cutoff : 0.f, rvl, lattice_range, min_range, R1, R2, R3);
    R_out[tid * 3 + 0] = R1;
    R_out[tid * 3 + 1] = R2;
    R_out[tid * 3 + 2] = R3;
}

__global__ void minimum_distance_kernel(const float *rpos, const float *tvecs, const int64_t *batch,
                                        const int64_t *edges, int64_t E, const float *rvlen,
                                        float cutoff, int lattice_range, int min_range, float *out)
{
    int64_t e = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (e >= E) return;
    const int64_t n = batch[edges[e]];
    Cell c;
    c.rx = rpos[e * 3];
    c.ry = rpos[e * 3 + 1];
    c.rz = rpos[e * 3 + 2];
    for (int x = 0; x < 9; x++) c.t[x] = tvecs[n * 9 + x];
    int R1 = lattice_range, R2 = lattice_range, R3 = lattice_range;
    if (cutoff > 0.f && rvlen) {
        R1 = range_axis(cutoff, rvlen[n * 3 + 0], min_range);
        R2 = range_axis(cutoff, rvlen[n * 3 + 1], min_range);
        R3 = range_axis(cutoff, rvlen[n * 3 + 2], min_range);
    }
    float m = 1e10f;
    for (int n1 = -R1; n1 <= R1; n1++)
        for (int n2 = -R2; n2 <= R2; n2++)
            for (int n3 = -R3; n3 <= R3; n3++) m = fminf(m, dist2(c, (float)n1, (float)n2, (float)n3));
    out[e] = m;
}

constexpr int GW_SPLITS = 64;

inline int64_t align256(int64_t x) { return (x + 255) / 256 * 256; }

int fill_args(EncArgs &p, const char *who, const float *a_ik, const float *rpos, const float *tvecs,
              const int64_t *batch, const int64_t *edges, int64_t N, int64_t H, int64_t E, int64_t B,
              int64_t K, int64_t D, double dist_max, double wscale, const float *W, int64_t W_num,
              const float *rvlen, double cutoff, int lattice_range, int min_range)
{
    CF_REQUIRE(N >= 0 && E >= 0 && B >= 0, CF_ERR_INVALID_ARGUMENT, "%s: negative size", who);
    CF_REQUIRE(H == 1 || H == 2 || H == 4 || H == 8 || H == 16, CF_ERR_UNSUPPORTED,
               "%s: head count %lld not supported (1,2,4,8,16)", who, (long long)H);
    CF_REQUIRE(K >= 0 && K <= 128, CF_ERR_UNSUPPORTED, "%s: K=%lld outside 0..128", who, (long long)K);
    CF_REQUIRE(lattice_range >= 0 && lattice_range <= MAX_RANGE, CF_ERR_INVALID_ARGUMENT,
               "%s: lattice_range %d outside 0..%d", who, lattice_range, MAX_RANGE);
    CF_REQUIRE(min_range >= 0 && min_range <= MAX_RANGE, CF_ERR_INVALID_ARGUMENT,
               "%s: minimum_range %d outside 0..%d", who, min_range, MAX_RANGE);
    if (E > 0)
        CF_REQUIRE(a_ik && rpos && tvecs && batch && edges, CF_ERR_INVALID_ARGUMENT,
                   "%s: null input pointer", who);
    CF_REQUIRE((float)cutoff == 0.0f || rvlen, CF_ERR_INVALID_ARGUMENT,
               "%s: non-zero cutoff_radius needs rvlen_n", who);
    if (K > 0) {
        CF_REQUIRE(dist_max > 0 && wscale > 0, CF_ERR_INVALID_ARGUMENT,
                   "%s: dist_max and wscale must be positive", who);
        if (W) {
            CF_REQUIRE(D >= 1 && D <= 64, CF_ERR_UNSUPPORTED, "%s: D=%lld outside 1..64", who, (long long)D);
            CF_REQUIRE(W_num == 1 || W_num == E || W_num == N, CF_ERR_INVALID_ARGUMENT,
                       "%s: W_num=%lld must be 1, E or N", who, (long long)W_num);
        }
    }
    p = EncArgs{};
    p.a_ik = a_ik;
    p.rpos = rpos;
    p.tvecs = tvecs;
    p.batch = batch;
    p.edges = edges;
    p.W = (K > 0) ? W : nullptr;
    p.rvlen = rvlen;
    p.N = N;
    p.E = E;
    p.W_num = W_num;
    p.K = (int)K;
    p.D = (int)D;
    p.cutoff = rvlen ? (float)cutoff : 0.0f;
    p.lattice_range = lattice_range;
    p.min_range = min_range;
    if (K > 0) {
        const float reci_ws_sqrt2 = 1.0f / ((float)wscale * sqrtf(2.0f));
        const float mu0 = (float)dist_max / (float)K;
        p.bin_step = reci_ws_sqrt2 * sqrtf(LOG2E);
        p.s_scale = p.bin_step / mu0;
    }
    return CF_OK;
}

int grid_for(int64_t E, int wpb, int waves_per_cu)
{
    int64_t blocks = (E + wpb - 1) / wpb;
    int64_t cap = (int64_t)device_cu_count() * waves_per_cu / wpb;
    if (cap < 1) cap = 1;
    return (int)(blocks < cap ? blocks : cap);
}

template <int H>
int launch_fwd(const EncArgs &p, hipStream_t st)
{
    const int wpb = 4;
    if (p.K == 0) {
        int grid = grid_for(p.E, wpb, 32);
        real_enc_fwd_bias_kernel<H><<<grid, wpb * WAVE, 0, st>>>(p);
        return CF_OK;
    }
    const int NB = p.K <= 64 ? 1 : 2;
    const int KP = NB * WAVE + 1;
    const bool proj = p.W != nullptr;
    size_t lds = 0;
    if (proj) lds = sizeof(float) * ((p.W_num == 1 ? (size_t)H * p.D * KP : 0) + (size_t)wpb * H * KP);
    CF_REQUIRE(lds <= 160 * 1024, CF_ERR_UNSUPPORTED, "cf_real_enc_fwd: H*D*K too large for LDS");
    int grid = grid_for(p.E, wpb, lds > 40 * 1024 ? 8 : 12);
#define CF_FWD(NBV, PROJV)                                                                            \
    do {                                                                                              \
        if (lds > 64 * 1024)                                                                          \
            (void)hipFuncSetAttribute((const void *)real_enc_fwd_kernel<H, NBV, PROJV>,               \
                                      hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);          \
        real_enc_fwd_kernel<H, NBV, PROJV><<<grid, wpb * WAVE, lds, st>>>(p);                         \
    } while (0)
    if (NB == 1) {
        if (proj) CF_FWD(1, true); else CF_FWD(1, false);
    } else {
        if (proj) CF_FWD(2, true); else CF_FWD(2, false);
    }
#undef CF_FWD
    return CF_OK;
}

template <int H>
int launch_bwd(const EncArgs &p, hipStream_t st)
{
    const int wpb = 4;
    if (p.K == 0) {
        int grid = grid_for(p.E, wpb, 32);
        real_enc_bwd_bias_kernel<H><<<grid, wpb * WAVE, 0, st>>>(p);
        return CF_OK;
    }
    const int NB = p.K <= 64 ? 1 : 2;
    const int KP = NB * WAVE + 1;
    const bool proj = p.W != nullptr;
    size_t lds = 0;
    if (proj && p.W_num == 1) lds = sizeof(float) * (size_t)H * p.D * KP;
    CF_REQUIRE(lds <= 160 * 1024, CF_ERR_UNSUPPORTED, "cf_real_enc_bwd: H*D*K too large for LDS");
    int grid = grid_for(p.E, wpb, 8);
#define CF_BWD(NBV, PROJV)                                                                            \
    do {                                                                                              \
        if (lds > 64 * 1024)                                                                          \
            (void)hipFuncSetAttribute((const void *)real_enc_bwd_kernel<H, NBV, PROJV>,               \
                                      hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);          \
        real_enc_bwd_kernel<H, NBV, PROJV><<<grid, wpb * WAVE, lds, st>>>(p);                         \
    } while (0)
    if (NB == 1) {
        if (proj) CF_BWD(1, true); else CF_BWD(1, false);
    } else {
        if (proj) CF_BWD(2, true); else CF_BWD(2, false);
    }
#undef CF_BWD
    return CF_OK;
}

#define CF_DISPATCH_H(H, fn, ...)                    \
    ((H) == 1 ? fn<1>(__VA_ARGS__)                   \
     : (H) == 2 ? fn<2>(__VA_ARGS__)                 \
     : (H) == 4 ? fn<4>(__VA_ARGS__)                 \
     : (H) == 8 ? fn<8>(__VA_ARGS__)                 \
                : fn<16>(__VA_ARGS__))

}  // namespace

extern "C" int cf_real_enc_fwd(const float *a_ik, const float *rpos_ij_e, const float *tvecs_n,
                               const int64_t *batch_i, const int64_t *edge_ij_e, int64_t N, int64_t H,
                               int64_t E, int64_t B, int64_t K, int64_t D, double dist_max,
                               double wscale, const float *W_k, int64_t W_num, const float *rvlen_n,
                               double cutoff_radius, int lattice_range, int minimum_range,
                               const int64_t *pairs_u, int64_t U, int32_t *sched_2, float *z_ek, float *v_ekd,
                               void *stream)
{
    EncArgs p;
    int rc = fill_args(p, "cf_real_enc_fwd", a_ik, rpos_ij_e, tvecs_n, batch_i, edge_ij_e, N, H, E, B, K,
                       D, dist_max, wscale, W_k, W_num, rvlen_n, cutoff_radius, lattice_range,
                       minimum_range);
    if (rc) return rc;
    if (E == 0) return CF_OK;
    CF_REQUIRE(z_ek, CF_ERR_INVALID_ARGUMENT, "cf_real_enc_fwd: z_ek is null");
    CF_REQUIRE(K == 0 || v_ekd, CF_ERR_INVALID_ARGUMENT, "cf_real_enc_fwd: v_ekd is null with K>0");
    CF_REQUIRE(!pairs_u || 2 * U == E + N, CF_ERR_INVALID_ARGUMENT,
               "cf_real_enc_fwd: a pair list over dense crystal blocks has (E+N)/2 = %lld entries, got %lld",
               (long long)((E + N) / 2), (long long)U);
    p.z = z_ek;
    p.v = v_ekd;
    if (pairs_u) {
        rc = launch_real_enc_fwd_pairs(a_ik, rpos_ij_e, tvecs_n, batch_i, edge_ij_e, pairs_u, U, N, H, E, K, D,
                                       p.bin_step, p.s_scale, p.W, W_num, rvlen_n, p.cutoff, lattice_range,
                                       minimum_range, reinterpret_cast<unsigned int *>(sched_2), nullptr, nullptr,
                                       z_ek, v_ekd, (hipStream_t)stream);
        if (rc == CF_OK) {
            CF_CHECK_LAUNCH("cf_real_enc_fwd (pairs)");
            return CF_OK;
        }
        if (rc != CF_ERR_UNSUPPORTED) return rc;   // otherwise: shape not instantiated, use the per-edge kernel
    }
    CF_REQUIRE(!cf::live_edges(E), CF_ERR_UNSUPPORTED,
               "cf_real_enc_fwd: with a size header set only the pair-evaluated kernels are served "
               "(pair list, K <= 128, shared projection with D <= 32)");
    rc = CF_DISPATCH_H(H, launch_fwd, p, (hipStream_t)stream);
    if (rc) return rc;
    CF_CHECK_LAUNCH("cf_real_enc_fwd");
    return CF_OK;
}

extern "C" int64_t cf_real_enc_bwd_workspace(int64_t N, int64_t H, int64_t E, int64_t K, int64_t D,
                                             int64_t W_num, int want_gW)
{
    int64_t bytes = align256(E * H * 4);                       // per-edge ga
    if (K > 0 && want_gW) {
        // per-edge kernels: normalised Gaussian averages + split partial sums of gW
        int64_t generic = align256(E * H * K * 4);
        if (W_num == 1) generic += align256((int64_t)GW_SPLITS * H * D * K * 4);
        // pair kernel: one H x D x K block per work-group
        int64_t paired = 0;
        if (W_num == 1) paired = align256((int64_t)real_enc_bwd_pairs_blocks((E + N) / 2, H) * H * D * K * 4);
        bytes += generic > paired ? generic : paired;
    }
    return bytes;
}

// cf_real_enc_bwd and cf_real_enc_bwd_rings (rings != nullptr: the pair kernel starts from the
// staged translations; shapes and gradient sets the pair kernel does not take go to the other
// kernels, which have no use for the rings).
static int real_enc_bwd_entry(const float *a_ik, const float *rpos_ij_e, const float *tvecs_n,
                              const int64_t *batch_i, const int64_t *edge_ij_e,
                              const int64_t *e_start_i, const float *z_ek, const float *gz_ek,
                              const float *gv_ekd, int64_t N, int64_t H, int64_t E, int64_t B, int64_t K,
                              int64_t D, double dist_max, double wscale, const float *W_k, int64_t W_num,
                              const float *rvlen_n, double cutoff_radius, int lattice_range,
                              int minimum_range, const int64_t *pairs_u, int64_t U, void *workspace,
                              int64_t workspace_bytes, float *ga_ik, float *gW_k, const float *rings,
                              void *stream)
{
    EncArgs p;
    int rc = fill_args(p, "cf_real_enc_bwd", a_ik, rpos_ij_e, tvecs_n, batch_i, edge_ij_e, N, H, E, B, K,
                       D, dist_max, wscale, W_k, W_num, rvlen_n, cutoff_radius, lattice_range,
                       minimum_range);
    if (rc) return rc;
    CF_REQUIRE(N == 0 || (ga_ik && e_start_i), CF_ERR_INVALID_ARGUMENT,
               "cf_real_enc_bwd: ga_ik / e_start_i is null");
    const bool want_gW = gW_k != nullptr && W_k != nullptr && K > 0;
    hipStream_t st = (hipStream_t)stream;
    if (want_gW && !gv_ekd) {
        int64_t total = W_num * H * D * K;
        fill_zero_kernel<<<(int)((total + 255) / 256), 256, 0, st>>>(gW_k, total);
        CF_CHECK_LAUNCH("cf_real_enc_bwd: clearing gW");
    }
    if (N == 0) return CF_OK;
    const int64_t need = cf_real_enc_bwd_workspace(N, H, E, K, D, W_num, want_gW && gv_ekd);
    CF_REQUIRE(E == 0 || (workspace && workspace_bytes >= need), CF_ERR_INVALID_ARGUMENT,
               "cf_real_enc_bwd: workspace of %lld bytes needed, %lld given", (long long)need,
               (long long)workspace_bytes);
    CF_REQUIRE(E == 0 || z_ek, CF_ERR_INVALID_ARGUMENT, "cf_real_enc_bwd: z_ek is null");
    CF_REQUIRE(!pairs_u || 2 * U == E + N, CF_ERR_INVALID_ARGUMENT,
               "cf_real_enc_bwd: a pair list over dense crystal blocks has (E+N)/2 = %lld entries, got %lld",
               (long long)((E + N) / 2), (long long)U);
    char *ws = (char *)workspace;
    if (pairs_u && E > 0 && K > 0 && W_k && W_num == 1 && gv_ekd) {
        float *ga_edge = (float *)ws;
        float *gW_part = want_gW ? (float *)(ws + align256(E * H * 4)) : nullptr;
        if (gW_part && H > 8) {     // a work-group only writes the head groups it visits
            int64_t total = (int64_t)real_enc_bwd_pairs_blocks(U, H) * H * D * K;
            fill_zero_kernel<<<(int)((total + 255) / 256), 256, 0, st>>>(gW_part, total);
        }
        rc = launch_real_enc_bwd_pairs(a_ik, rpos_ij_e, tvecs_n, batch_i, edge_ij_e, pairs_u, U, z_ek, gz_ek,
                                       gv_ekd, N, H, E, K, D, p.bin_step, p.s_scale, W_k, rvlen_n, p.cutoff,
                                       lattice_range, minimum_range, ga_edge, gW_part, gW_k, e_start_i, ga_ik,
                                       rings, st);
        if (rc == CF_OK) {
            CF_CHECK_LAUNCH("cf_real_enc_bwd (pairs)");     // the pair kernel and its two reductions
            return CF_OK;
        }
        if (rc != CF_ERR_UNSUPPORTED) return rc;
    }
    p.e_start = e_start_i;
    p.z_in = z_ek;
    p.gz = gz_ek;
    p.gv = (K > 0) ? gv_ekd : nullptr;
    p.ga_edge = (float *)ws;
    ws += align256(E * H * 4);
    float *part = nullptr;
    if (want_gW && gv_ekd) {
        p.sv_out = (float *)ws;
        ws += align256(E * H * K * 4);
        part = (float *)ws;
    }
    if (E > 0) {
        rc = CF_DISPATCH_H(H, launch_bwd, p, st);
        if (rc) return rc;
        CF_CHECK_LAUNCH("cf_real_enc_bwd");
    }
    {
        int64_t total = N * H;
        reduce_ga_kernel<<<(int)((total + 255) / 256), 256, 0, st>>>(p.ga_edge, e_start_i, N, (int)H, ga_ik);
        CF_CHECK_LAUNCH("cf_real_enc_bwd: reduce_ga");
    }
    if (want_gW && gv_ekd) {
        if (W_num == 1) {
            gw_partial_kernel<<<(int)(H * GW_SPLITS), 256, 0, st>>>(gv_ekd, p.sv_out, E, (int)H, (int)D,
                                                                     (int)K, GW_SPLITS, part);
            CF_CHECK_LAUNCH("cf_real_enc_bwd: gw_partial");
            int64_t HDK = H * D * K;
            gw_final_kernel<<<(int)((HDK + 255) / 256), 256, 0, st>>>(part, GW_SPLITS, HDK, gW_k);
            CF_CHECK_LAUNCH("cf_real_enc_bwd: gw_final");
        } else {
            int64_t total = W_num * H * D * K;
            gw_indexed_kernel<<<(int)((total + 255) / 256), 256, 0, st>>>(gv_ekd, p.sv_out, e_start_i, W_num,
                                                                          E, (int)H, (int)D, (int)K, gW_k);
            CF_CHECK_LAUNCH("cf_real_enc_bwd: gw_indexed");
        }
    }
    return CF_OK;
}

extern "C" int cf_real_enc_bwd(const float *a_ik, const float *rpos_ij_e, const float *tvecs_n,
                               const int64_t *batch_i, const int64_t *edge_ij_e,
                               const int64_t *e_start_i, const float *z_ek, const float *gz_ek,
                               const float *gv_ekd, int64_t N, int64_t H, int64_t E, int64_t B, int64_t K,
                               int64_t D, double dist_max, double wscale, const float *W_k, int64_t W_num,
                               const float *rvlen_n, double cutoff_radius, int lattice_range,
                               int minimum_range, const int64_t *pairs_u, int64_t U, void *workspace,
                               int64_t workspace_bytes, float *ga_ik, float *gW_k, void *stream)
{
    return real_enc_bwd_entry(a_ik, rpos_ij_e, tvecs_n, batch_i, edge_ij_e, e_start_i, z_ek, gz_ek, gv_ekd, N, H, E,
                              B, K, D, dist_max, wscale, W_k, W_num, rvlen_n, cutoff_radius, lattice_range,
                              minimum_range, pairs_u, U, workspace, workspace_bytes, ga_ik, gW_k, nullptr, stream);
}

extern "C" int cf_real_enc_bwd_rings(const float *a_ik, const float *rpos_ij_e, const float *tvecs_n,
                                     const int64_t *batch_i, const int64_t *edge_ij_e,
                                     const int64_t *e_start_i, const float *z_ek, const float *gz_ek,
                                     const float *gv_ekd, int64_t N, int64_t H, int64_t E, int64_t B, int64_t K,
                                     int64_t D, double dist_max, double wscale, const float *W_k,
                                     int lattice_range, const int64_t *pairs_u, int64_t U, const float *rings,
                                     void *workspace, int64_t workspace_bytes, float *ga_ik, float *gW_k,
                                     void *stream)
{
    CF_REQUIRE(rings && pairs_u, CF_ERR_INVALID_ARGUMENT, "cf_real_enc_bwd_rings: rings / pairs_u is null");
    return real_enc_bwd_entry(a_ik, rpos_ij_e, tvecs_n, batch_i, edge_ij_e, e_start_i, z_ek, gz_ek, gv_ekd, N, H, E,
                              B, K, D, dist_max, wscale, W_k, 1, nullptr, 0.0, lattice_range, 0, pairs_u, U,
                              workspace, workspace_bytes, ga_ik, gW_k, rings, stream);
}

// ---- backward without a caller-provided workspace ----------------------------------
// Scratch of cf_real_enc_bwd (per-edge ga, per-work-group gW blocks, or the per-edge kernels'
// Gaussian averages) in a fixed array that every GPU running this library holds until the
// process ends.  The array's name is a host-side stand-in for the symbol: the device address
// is looked up once per device, with that device current, and only that address is ever
// handed to a kernel.
#define CF_STATIC_SCRATCH_BYTES (32ll << 20)
static __device__ __align__(256) unsigned char scratch[CF_STATIC_SCRATCH_BYTES];

namespace {
constexpr int MAX_DEVICES = 64;
std::mutex g_scratch_mutex;
void *g_scratch_ptr[MAX_DEVICES] = {};

int static_scratch(void **out)
{
    int dev = -1;
    hipError_t err = hipGetDevice(&dev);
    if (err != hipSuccess) return cf::hip_failed(err, "cf_real_enc_bwd_static: hipGetDevice");
    CF_REQUIRE(dev >= 0 && dev < MAX_DEVICES, CF_ERR_INVALID_ARGUMENT,
               "cf_real_enc_bwd_static: device %d outside 0..%d", dev, MAX_DEVICES - 1);
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (!g_scratch_ptr[dev]) {
        void *ptr = nullptr;
        err = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
        if (err != hipSuccess) return cf::hip_failed(err, "cf_real_enc_bwd_static: hipGetSymbolAddress");
        CF_REQUIRE(ptr != nullptr, CF_ERR_HIP, "cf_real_enc_bwd_static: no device address for the scratch array");
        g_scratch_ptr[dev] = ptr;
    }
    *out = g_scratch_ptr[dev];
    return CF_OK;
}
}  // namespace

extern "C" int64_t cf_static_scratch_bytes(void) { return CF_STATIC_SCRATCH_BYTES; }

extern "C" int cf_real_enc_bwd_static(const float *a_ik, const float *rpos_ij_e, const float *tvecs_n,
                                      const int64_t *batch_i, const int64_t *edge_ij_e,
                                      const int64_t *e_start_i, const float *z_ek, const float *gz_ek,
                                      const float *gv_ekd, int64_t N, int64_t H, int64_t E, int64_t B, int64_t K,
                                      int64_t D, double dist_max, double wscale, const float *W_k, int64_t W_num,
                                      const float *rvlen_n, double cutoff_radius, int lattice_range,
                                      int minimum_range, const int64_t *pairs_u, int64_t U, float *ga_ik,
                                      float *gW_k, void *stream)
{
    CF_REQUIRE(N >= 0 && H >= 1 && E >= 0 && K >= 0 && D >= 0 && W_num >= 0, CF_ERR_INVALID_ARGUMENT,
               "cf_real_enc_bwd_static: negative size");
    const bool want_gW = gW_k != nullptr && W_k != nullptr && K > 0 && gv_ekd != nullptr;
    const int64_t need = cf_real_enc_bwd_workspace(N, H, E, K, D, W_num, want_gW);
    CF_REQUIRE(need <= CF_STATIC_SCRATCH_BYTES, CF_ERR_INVALID_ARGUMENT,
               "cf_real_enc_bwd_static: these sizes need %lld bytes of scratch, the built-in buffer holds %lld; "
               "use cf_real_enc_bwd with a workspace", (long long)need, (long long)CF_STATIC_SCRATCH_BYTES);
    void *ws = nullptr;
    int rc = static_scratch(&ws);
    if (rc) return rc;
    return cf_real_enc_bwd(a_ik, rpos_ij_e, tvecs_n, batch_i, edge_ij_e, e_start_i, z_ek, gz_ek, gv_ekd, N, H, E,
                           B, K, D, dist_max, wscale, W_k, W_num, rvlen_n, cutoff_radius, lattice_range,
                           minimum_range, pairs_u, U, ws, CF_STATIC_SCRATCH_BYTES, ga_ik, gW_k, stream);
}

namespace {
template <int H>
int launch_enc_dpa_rows(const EncArgs &p, const RowArgs &r, int64_t N, hipStream_t st)
{
    const size_t lds = sizeof(float) * (size_t)r.max_row * (H + 1);
    // a wavefront per edge of the longest row, 4 to 16 of them
    const int waves = r.max_row <= 4 ? 4 : r.max_row <= 8 ? 8 : 16;
    enc_dpa_row_kernel<H><<<(int)N, waves * WAVE, lds, st>>>(p, r);
    return CF_OK;
}
}  // namespace

extern "C" int cf_fused_enc_dpa_fwd(const float *a_ik, const float *rpos_ij_e, const float *tvecs_n,
                                    const int64_t *batch_i, const int64_t *edge_ij_e, const int64_t *e_start_i,
                                    const float *que, const float *key, const float *val, int64_t N, int64_t H,
                                    int64_t E, int64_t B, int64_t Dk, int64_t Dv, const float *rvlen_n,
                                    double cutoff_radius, int lattice_range, int minimum_range, int64_t max_row,
                                    float *out, void *stream)
{
    EncArgs p;
    int rc = fill_args(p, "cf_fused_enc_dpa_fwd", a_ik, rpos_ij_e, tvecs_n, batch_i, edge_ij_e, N, H, E, B, 0, 0,
                       1.0, 1.0, nullptr, 0, rvlen_n, cutoff_radius, lattice_range, minimum_range);
    if (rc) return rc;
    CF_REQUIRE(Dk >= 1 && Dv >= 1 && Dk <= 256 && Dv <= 256, CF_ERR_INVALID_ARGUMENT,
               "cf_fused_enc_dpa_fwd: head widths %lld / %lld outside 1..256", (long long)Dk, (long long)Dv);
    CF_REQUIRE(N < (1ll << 31), CF_ERR_UNSUPPORTED, "cf_fused_enc_dpa_fwd: more than 2^31 atoms");
    if (N == 0) return CF_OK;
    CF_REQUIRE(que && key && val && out && e_start_i, CF_ERR_INVALID_ARGUMENT, "cf_fused_enc_dpa_fwd: null pointer");
    CF_REQUIRE(max_row >= 0 && max_row * (H + 1) * 4 <= 64 * 1024, CF_ERR_UNSUPPORTED,
               "cf_fused_enc_dpa_fwd: rows of up to %lld edges; this kernel keeps a row's %lld logits in 64 KB of "
               "LDS (use cf_real_enc_fwd + cf_fused_dpa_fwd)", (long long)max_row, (long long)(max_row * H));
    p.e_start = e_start_i;
    RowArgs r{que, key, val, out, (int)Dk, (int)Dv, (int)(max_row < 1 ? 1 : max_row)};
    rc = CF_DISPATCH_H(H, launch_enc_dpa_rows, p, r, N, (hipStream_t)stream);
    if (rc) return rc;
    CF_CHECK_LAUNCH("cf_fused_enc_dpa_fwd");
    return CF_OK;
}

extern "C" int cf_translation_ranges(const float *a_ik, const float *rvlen_n, const int64_t *batch_i,
                                     int64_t N, int64_t H, double cutoff_radius, int lattice_range,
                                     int minimum_range, int32_t *R_out, void *stream)
{
    CF_REQUIRE(N >= 0 && H >= 1, CF_ERR_INVALID_ARGUMENT, "cf_translation_ranges: bad sizes");
    if (N == 0) return CF_OK;
    CF_REQUIRE(a_ik && R_out && (!rvlen_n || batch_i), CF_ERR_INVALID_ARGUMENT,
               "cf_translation_ranges: null pointer");
    int64_t total = N * H;
    translation_ranges_kernel<<<(int)((total + 255) / 256), 256, 0, (hipStream_t)stream>>>(
        a_ik, rvlen_n, batch_i, N, (int)H, (float)cutoff_radius, lattice_range, minimum_range, R_out);
    CF_CHECK_LAUNCH("cf_translation_ranges");
    return CF_OK;
}

extern "C" int cf_minimum_distance(const float *rpos_ij_e, const float *tvecs_n, const int64_t *batch_i,
                                   const int64_t *edge_ij_e, int64_t E, const float *rvlen_n,
                                   double cutoff_radius, int lattice_range, int minimum_range,
                                   float *dist2_min_e, void *stream)
{
    CF_REQUIRE(E >= 0, CF_ERR_INVALID_ARGUMENT, "cf_minimum_distance: negative E");
    CF_REQUIRE(cutoff_radius >= 0, CF_ERR_INVALID_ARGUMENT, "cf_minimum_distance: cutoff_radius must be >= 0");
    CF_REQUIRE(lattice_range >= 0 && lattice_range <= MAX_RANGE, CF_ERR_INVALID_ARGUMENT,
               "cf_minimum_distance: lattice_range out of bounds");
    if (E == 0) return CF_OK;
    CF_REQUIRE(rpos_ij_e && tvecs_n && batch_i && edge_ij_e && dist2_min_e, CF_ERR_INVALID_ARGUMENT,
               "cf_minimum_distance: null pointer");
    minimum_distance_kernel<<<(int)((E + 255) / 256), 256, 0, (hipStream_t)stream>>>(
        rpos_ij_e, tvecs_n, batch_i, edge_ij_e, E, rvlen_n, (float)cutoff_radius, lattice_range,
        minimum_range, dist2_min_e);
    CF_CHECK_LAUNCH("cf_minimum_distance");
    return CF_OK;
}
