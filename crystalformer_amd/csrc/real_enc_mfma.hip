// Real-space periodic encoding, forward, matrix-core version for gfx950.
//
// Unit of work: an unordered edge pair {(i->j), (j->i)} (or one self edge).
// Both directions see the same set of image distances, d_ji(n) = d_ij(-n), and
// every translation box is symmetric, so the K Gaussians of a translation are
// evaluated ONCE and feed 16 weight columns: 8 heads of atom i and 8 heads of
// atom j.  The accumulation
//        S[bin, column] += g_bin(d_t) * w_column(d_t)        over translations t
// is a GEMM with the translations as the reduction dimension and runs on
// v_mfma_f32_16x16x4_f32: 4 translations per instruction, 16 bins x 16 columns
// per tile, K/16 tiles.
//
// Lane roles inside a wavefront (q = lane / 16, c = lane % 16):
//   wide phase   lane = translation (64 at a time): decode, d^2, sqrt, in-box
//                bits of the 16 columns -> a 1 KB LDS ring per wave;
//   deep phase   for each group of 4 translations, lane (q, c) reads translation
//                q of the group, forms column c's weight exp(a_c (d^2 - d^2min_c))
//                (B operand) and the Gaussians of bins 16m + c (A operands);
//   epilogue     lane (q, c) owns bins 16m + 4q + r of column c (the MFMA
//                accumulator layout); the D x K projection is applied from LDS
//                and reduced over q with two cross-lane adds.
#include "cf_common.h"

namespace {

using namespace cf;

typedef float float4_t __attribute__((ext_vector_type(4)));

struct PairArgs {
    const float *a_ik;
    const float *rpos;
    const float *tvecs;
    const int64_t *batch;
    const int64_t *edges;
    const int64_t *pairs;   // (U,2): edge (i->j) with i <= j and its reverse
    const float *W;
    const float *rvlen;
    float *z;
    float *v;
    int64_t N, E, U;
    int64_t W_num;
    int H, K, D;
    int head_groups;        // ceil(H / 8)
    float cutoff;
    int lattice_range, min_range;
    float bin_step, s_scale;
};

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

__device__ __forceinline__ void decode(int idx, int S2, int S3, int U1, int U2, int U3, int &n1, int &n2,
                                       int &n3)
{
    int plane = S2 * S3;
    int q1 = idx / plane;
    int rem = idx - q1 * plane;
    int q2 = rem / S3;
    n1 = q1 - U1;
    n2 = q2 - U2;
    n3 = rem - q2 * S3 - U3;
}

// max over the 16 lanes that share q (xor 1,2,4,8) and then over q (xor 16,32)
__device__ __forceinline__ int wave_max_int(int v)
{
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v = max(v, __shfl_xor(v, off, WAVE));
    return v;
}

// W staged as [h][d][KP] with KP = 16*NT + 4 floats (16-byte aligned rows).
template <int NT, bool UNIFORM, bool PROJ>
__global__ __launch_bounds__(256) void real_enc_fwd_pair_kernel(PairArgs p)
{
    extern __shared__ __align__(16) float lds[];
    constexpr int KP = 16 * NT + 4;
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int wpb = blockDim.x >> 6;
    const int q = lane >> 4;
    const int c = lane & 15;
    const int H = p.H, K = p.K, D = p.D;
    const bool w_shared = PROJ && p.W_num == 1;
    float *Wl = lds;
    float4_t *ring = reinterpret_cast<float4_t *>(lds + (w_shared ? H * D * KP : 0)) + wave * WAVE;

    if (w_shared) {
        for (int x = threadIdx.x; x < H * D * KP; x += blockDim.x) {
            int hd = x / KP, k = x - hd * KP;
            Wl[x] = (k < K) ? p.W[hd * K + k] : 0.f;
        }
        __syncthreads();
    }
    // Gaussian argument of bin 16m + c at distance 0
    float ck[NT];
#pragma unroll
    for (int m = 0; m < NT; m++) ck[m] = p.bin_step * (float)(16 * m + c + 1);

    const int64_t items = p.U * p.head_groups;
    for (int64_t it = (int64_t)blockIdx.x * wpb + wave; it < items; it += (int64_t)gridDim.x * wpb) {
        const int64_t u = it / p.head_groups;
        const int hg = (int)(it - u * p.head_groups);
        const int64_t e_ij = p.pairs[2 * u], e_ji = p.pairs[2 * u + 1];
        const int64_t i = p.edges[e_ij], j = p.edges[p.E + e_ij];
        const int64_t n = p.batch[i];
        Cell cell;
        cell.rx = p.rpos[e_ij * 3 + 0];
        cell.ry = p.rpos[e_ij * 3 + 1];
        cell.rz = p.rpos[e_ij * 3 + 2];
#pragma unroll
        for (int x = 0; x < 9; x++) cell.t[x] = p.tvecs[n * 9 + x];

        // column c: head (hg*8 + c%8) of atom i (c < 8) or atom j (c >= 8)
        const int h = hg * 8 + (c & 7);
        const bool col_on = h < H && (c < 8 || e_ji != e_ij);
        const int64_t atom = (c < 8) ? i : j;
        const float a = col_on ? p.a_ik[atom * H + h] : -1.0f;
        const float a2 = a * LOG2E;

        // translation box: union over the 16 columns; per-column boxes when they differ
        int U1 = p.lattice_range, U2 = U1, U3 = U1;
        int R1 = U1, R2 = U1, R3 = U1;
        if (!UNIFORM) {
            float rvl[3] = {p.rvlen[n * 3 + 0], p.rvlen[n * 3 + 1], p.rvlen[n * 3 + 2]};
            range_rule(a, p.cutoff, rvl, p.lattice_range, p.min_range, R1, R2, R3);
            if (!col_on) R1 = R2 = R3 = 0;
            U1 = wave_max_int(R1);
            U2 = wave_max_int(R2);
            U3 = wave_max_int(R3);
        }
        const int S3 = 2 * U3 + 1, S2 = 2 * U2 + 1;
        const int T = (2 * U1 + 1) * S2 * S3;

        // pass 1: minimum of d^2 over each column's own box
        float d2min;
        {
            float mloc[UNIFORM ? 1 : 16];
#pragma unroll
            for (int x = 0; x < (UNIFORM ? 1 : 16); x++) mloc[x] = 1e10f;
            for (int c0 = 0; c0 < T; c0 += WAVE) {
                int idx = c0 + lane;
                if (idx < T) {
                    int n1, n2, n3;
                    decode(idx, S2, S3, U1, U2, U3, n1, n2, n3);
                    float d2 = dist2(cell, (float)n1, (float)n2, (float)n3);
                    if (UNIFORM) {
                        mloc[0] = fminf(mloc[0], d2);
                    } else {
#pragma unroll
                        for (int x = 0; x < 16; x++) {
                            int r1 = __builtin_amdgcn_readlane(R1, x);
                            int r2 = __builtin_amdgcn_readlane(R2, x);
                            int r3 = __builtin_amdgcn_readlane(R3, x);
                            if (abs(n1) <= r1 && abs(n2) <= r2 && abs(n3) <= r3) mloc[x] = fminf(mloc[x], d2);
                        }
                    }
                }
            }
            if (UNIFORM) {
                d2min = wave_min(mloc[0]);
            } else {
                d2min = 1e10f;
#pragma unroll
                for (int x = 0; x < 16; x++) {
                    float mx = wave_min(mloc[x]);
                    if (c == x) d2min = mx;
                }
            }
        }

        // pass 2: accumulate
        float4_t acc[NT];
#pragma unroll
        for (int m = 0; m < NT; m++) acc[m] = float4_t{0.f, 0.f, 0.f, 0.f};
        float sum = 0.f;
        for (int c0 = 0; c0 < T; c0 += WAVE) {
            {   // wide phase: lane = translation
                int idx = c0 + lane;
                bool valid = idx < T;
                int n1, n2, n3;
                decode(valid ? idx : 0, S2, S3, U1, U2, U3, n1, n2, n3);
                float d2 = dist2(cell, (float)n1, (float)n2, (float)n3);
                float s = sqrt_hw(d2) * p.s_scale;
                int bits = 0;
                if (valid) {
                    if (UNIFORM) {
                        bits = 0xFFFF;
                    } else {
#pragma unroll
                        for (int x = 0; x < 16; x++) {
                            int r1 = __builtin_amdgcn_readlane(R1, x);
                            int r2 = __builtin_amdgcn_readlane(R2, x);
                            int r3 = __builtin_amdgcn_readlane(R3, x);
                            if (abs(n1) <= r1 && abs(n2) <= r2 && abs(n3) <= r3) bits |= (1 << x);
                        }
                    }
                }
                ring[lane] = float4_t{d2, s, __int_as_float(bits), 0.f};
            }
            wave_mem_sync();
            const int groups = (min(WAVE, T - c0) + 3) >> 2;
            for (int g = 0; g < groups; g++) {
                const float4_t rec = ring[4 * g + q];
                const int bits = __float_as_int(rec.z);
                float w = exp2_hw(a2 * (rec.x - d2min));
                w = (col_on && ((bits >> c) & 1)) ? w : 0.f;
                sum += w;
#pragma unroll
                for (int m = 0; m < NT; m++) {
                    float b = ck[m] - rec.y;
                    float gm = exp2_hw(-(b * b));
                    acc[m] = __builtin_amdgcn_mfma_f32_16x16x4f32(gm, w, acc[m], 0, 0, 0);
                }
            }
            wave_mem_sync();
        }
        // column totals: the 4 lanes sharing c hold partial sums
        sum += __shfl_xor(sum, 16, WAVE);
        sum += __shfl_xor(sum, 32, WAVE);
        const float inv = 1.0f / sum;
        const int64_t e_col = (c < 8) ? e_ij : e_ji;
        if (col_on && q == 0) p.z[e_col * H + h] = log2_hw(sum) * LN2 + d2min * a;

        // epilogue: lane (q,c) holds S[bin = 16m + 4q + r][column c] in acc[m][r]
        if (!PROJ) {
            if (col_on) {
#pragma unroll
                for (int m = 0; m < NT; m++) {
                    int k0 = 16 * m + 4 * q;
                    float *dst = p.v + (e_col * H + h) * K + k0;
#pragma unroll
                    for (int r = 0; r < 4; r++)
                        if (k0 + r < K) dst[r] = acc[m][r] * inv;
                }
            }
        } else {
            int64_t w_ind = 0;
            if (p.W_num == 1) w_ind = 0;
            else if (p.W_num == p.E) w_ind = e_col;
            else if (p.W_num == p.N) w_ind = atom;
            const float *Wg = p.W + (w_ind * H + (col_on ? h : 0)) * (int64_t)D * K;
            const float *Wh = Wl + (col_on ? h : 0) * D * KP;
            for (int d0 = 0; d0 < D; d0 += 16) {
                float out[16];
#pragma unroll
                for (int dd = 0; dd < 16; dd++) {
                    float o = 0.f;
                    if (d0 + dd < D) {
#pragma unroll
                        for (int m = 0; m < NT; m++) {
                            const int k0 = 16 * m + 4 * q;
                            if (w_shared) {
                                const float4_t wv = *reinterpret_cast<const float4_t *>(Wh + (d0 + dd) * KP + k0);
                                o = fmaf(wv.x, acc[m][0], o);
                                o = fmaf(wv.y, acc[m][1], o);
                                o = fmaf(wv.z, acc[m][2], o);
                                o = fmaf(wv.w, acc[m][3], o);
                            } else {
#pragma unroll
                                for (int r = 0; r < 4; r++)
                                    if (k0 + r < K) o = fmaf(Wg[(int64_t)(d0 + dd) * K + k0 + r], acc[m][r], o);
                            }
                        }
                    }
                    o += __shfl_xor(o, 16, WAVE);
                    o += __shfl_xor(o, 32, WAVE);
                    out[dd] = o * inv;
                }
                // lane q writes components d0 + 4q .. d0 + 4q + 3
                if (col_on) {
                    float *dst = p.v + (e_col * H + h) * D + d0 + 4 * q;
#pragma unroll
                    for (int r = 0; r < 4; r++) {
                        float val = q == 0 ? out[r] : q == 1 ? out[4 + r] : q == 2 ? out[8 + r] : out[12 + r];
                        if (d0 + 4 * q + r < D) dst[r] = val;
                    }
                }
            }
        }
    }
}

// (i <= j) edges of every crystal's dense block and their reverses.
__global__ void edge_pairs_kernel(const int64_t *atom_start, const int64_t *edge_start,
                                  const int64_t *unit_start, int64_t B, int64_t E, int64_t *pairs)
{
    int64_t e = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (e >= E) return;
    int64_t lo = 0, hi = B;
    while (hi - lo > 1) {
        int64_t mid = (lo + hi) >> 1;
        if (edge_start[mid] <= e) lo = mid; else hi = mid;
    }
    const int64_t n = atom_start[lo + 1] - atom_start[lo];
    const int64_t e0 = edge_start[lo];
    const int64_t local = e - e0;
    const int64_t il = local / n, jl = local - il * n;
    if (il > jl) return;
    // row il of the upper triangle starts after il*n - il*(il-1)/2 units
    const int64_t u = unit_start[lo] + il * n - (il * (il - 1)) / 2 + (jl - il);
    pairs[2 * u] = e;
    pairs[2 * u + 1] = e0 + jl * n + il;
}

}  // namespace

namespace cf {

// Launches the pair kernel; returns CF_ERR_UNSUPPORTED (without setting an
// error) when the shape is outside what it instantiates so that the caller can
// use the per-edge kernel.
int launch_real_enc_fwd_pairs(const float *a_ik, const float *rpos, const float *tvecs, const int64_t *batch,
                              const int64_t *edges, const int64_t *pairs, int64_t U, int64_t N, int64_t H,
                              int64_t E, int64_t K, int64_t D, float bin_step, float s_scale, const float *W,
                              int64_t W_num, const float *rvlen, float cutoff, int lattice_range,
                              int min_range, float *z, float *v, hipStream_t st)
{
    if (K < 1 || K > 128 || (K > 64 && W)) return CF_ERR_UNSUPPORTED;
    if (W && (D < 1 || D > 64 || (D % 4) != 0)) return CF_ERR_UNSUPPORTED;
    PairArgs p{};
    p.a_ik = a_ik; p.rpos = rpos; p.tvecs = tvecs; p.batch = batch; p.edges = edges; p.pairs = pairs;
    p.W = W; p.rvlen = rvlen; p.z = z; p.v = v;
    p.N = N; p.E = E; p.U = U; p.W_num = W_num;
    p.H = (int)H; p.K = (int)K; p.D = (int)D;
    p.head_groups = (int)((H + 7) / 8);
    p.cutoff = cutoff; p.lattice_range = lattice_range; p.min_range = min_range;
    p.bin_step = bin_step; p.s_scale = s_scale;
    const int NT = K <= 16 ? 1 : K <= 32 ? 2 : K <= 64 ? 4 : 8;
    const int KP = 16 * NT + 4;
    const int wpb = 4;
    const bool proj = W != nullptr;
    const bool uniform = cutoff == 0.0f;
    size_t lds = sizeof(float) * ((proj && W_num == 1 ? (size_t)H * D * KP : 0) + (size_t)wpb * WAVE * 4);
    if (lds > 64 * 1024) return CF_ERR_UNSUPPORTED;
    const int64_t items = U * p.head_groups;
    int64_t blocks = (items + wpb - 1) / wpb;
    int64_t cap = (int64_t)device_cu_count() * 4;      // 16 waves per CU
    if (blocks > cap) blocks = cap;
    if (blocks < 1) return CF_OK;
#define CF_PAIR(NTV, UNI, PRJ) \
    real_enc_fwd_pair_kernel<NTV, UNI, PRJ><<<(int)blocks, wpb * WAVE, lds, st>>>(p)
#define CF_PAIR_NT(NTV)                                     \
    do {                                                    \
        if (uniform) {                                      \
            if (proj) CF_PAIR(NTV, true, true);             \
            else CF_PAIR(NTV, true, false);                 \
        } else {                                            \
            if (proj) CF_PAIR(NTV, false, true);            \
            else CF_PAIR(NTV, false, false);                \
        }                                                   \
    } while (0)
    switch (NT) {
        case 1: CF_PAIR_NT(1); break;
        case 2: CF_PAIR_NT(2); break;
        case 4: CF_PAIR_NT(4); break;
        default: CF_PAIR_NT(8); break;
    }
#undef CF_PAIR_NT
#undef CF_PAIR
    return CF_OK;
}

}  // namespace cf

extern "C" int cf_edge_pairs(const int64_t *atom_start_n, const int64_t *edge_start_n,
                             const int64_t *unit_start_n, int64_t B, int64_t E, int64_t *pairs_u,
                             void *stream)
{
    CF_REQUIRE(B >= 0 && E >= 0, CF_ERR_INVALID_ARGUMENT, "cf_edge_pairs: negative size");
    if (E == 0) return CF_OK;
    CF_REQUIRE(B > 0 && atom_start_n && edge_start_n && unit_start_n && pairs_u, CF_ERR_INVALID_ARGUMENT,
               "cf_edge_pairs: null pointer or no crystals");
    edge_pairs_kernel<<<(int)((E + 255) / 256), 256, 0, (hipStream_t)stream>>>(atom_start_n, edge_start_n,
                                                                              unit_start_n, B, E, pairs_u);
    CF_CHECK_LAUNCH("cf_edge_pairs");
    return CF_OK;
}
