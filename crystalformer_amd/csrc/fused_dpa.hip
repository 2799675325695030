// Fused edge-indexed dot-product attention for gfx950, forward and backward.
//
// Forward: one wavefront per query atom.
//   * logits, lane = key: each lane forms q_i . k_j + a_ij for all heads of
//     its keys and parks them in prob[e,h]; per-head max and sum are wave
//     reductions, so a crystal of any size is handled (no per-crystal limit);
//   * aggregation, lane = (head, value component): the wave streams the edge
//     row once, reading b_ij with fully coalesced 4*H*Dv-byte rows.
// Backward: three gather-by-owner kernels (no atomics, fixed summation order):
//   rows    (per query): gb_ij = go_i p_ij, gs_ij = sum_d (v_j + b_ij - o_i) gb_ij
//   queries (per query): gq_i = sum_j gs_ij k_j
//   keys    (per key)  : gv_j = sum_i gb_ij, gk_j = sum_i gs_ij q_i, walking a
//                        column of the crystal's dense n x n edge block.
#include "cf_common.h"

namespace {

using namespace cf;

struct DpaArgs {
    const float *que, *key, *val, *aij, *bij;
    const int64_t *edges, *e_start, *batch, *atom_start, *edge_start;
    const float *prob_in, *out_in, *gout;
    float *prob, *out;
    float *gque, *gkey, *gval, *gaij, *gbij;
    int64_t N, E;
    int H, Dk, Dv;
};

constexpr int MAXH = 16;

// ------------------------------------------------------------------ forward
template <int H>
__global__ __launch_bounds__(256) void fused_dpa_fwd_kernel(DpaArgs p)
{
    const int lane = threadIdx.x & 63;
    const int64_t i = (int64_t)blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
    if (i >= p.N) return;   // whole wave exits together
    const int Dk = p.Dk, Dv = p.Dv;
    const int64_t e0 = p.e_start[i], e1 = p.e_start[i + 1];
    const int64_t *dst = p.edges + p.E;
    const float *q = p.que + i * H * Dk;

    // pass 1: raw logits -> prob, running max
    float mx[H];
#pragma unroll
    for (int h = 0; h < H; h++) mx[h] = -3.0e38f;
    for (int64_t e = e0 + lane; e < e1; e += WAVE) {
        const float *kj = p.key + dst[e] * H * Dk;
#pragma unroll
        for (int h = 0; h < H; h++) {
            float s = 0.f;
            for (int d = 0; d < Dk; d++) s = fmaf(q[h * Dk + d], kj[h * Dk + d], s);
            if (p.aij) s += p.aij[e * H + h];
            p.prob[e * H + h] = s;
            mx[h] = fmaxf(mx[h], s);
        }
    }
    float sm[H];
#pragma unroll
    for (int h = 0; h < H; h++) {
        mx[h] = wave_max(mx[h]);
        sm[h] = 0.f;
    }
    // pass 2: exponentials (each lane re-reads only what it wrote)
    for (int64_t e = e0 + lane; e < e1; e += WAVE) {
#pragma unroll
        for (int h = 0; h < H; h++) {
            float x = exp2_hw((p.prob[e * H + h] - mx[h]) * LOG2E);
            p.prob[e * H + h] = x;
            sm[h] += x;
        }
    }
    float inv[H];
#pragma unroll
    for (int h = 0; h < H; h++) inv[h] = 1.0f / wave_sum(sm[h]);
    // pass 3: normalise
    for (int64_t e = e0 + lane; e < e1; e += WAVE) {
#pragma unroll
        for (int h = 0; h < H; h++) p.prob[e * H + h] *= inv[h];
    }
    wave_mem_sync();

    // aggregation: lane = (head, component)
    const int HD = H * Dv;
    for (int x = lane; x < HD; x += WAVE) {
        const int h = x / Dv;
        float acc0 = 0.f, acc1 = 0.f, acc2 = 0.f, acc3 = 0.f;
        int64_t e = e0;
        if (p.bij) {
            for (; e + 4 <= e1; e += 4) {
                float m0 = p.val[dst[e] * HD + x] + p.bij[e * HD + x];
                float m1 = p.val[dst[e + 1] * HD + x] + p.bij[(e + 1) * HD + x];
                float m2 = p.val[dst[e + 2] * HD + x] + p.bij[(e + 2) * HD + x];
                float m3 = p.val[dst[e + 3] * HD + x] + p.bij[(e + 3) * HD + x];
                acc0 = fmaf(p.prob[e * H + h], m0, acc0);
                acc1 = fmaf(p.prob[(e + 1) * H + h], m1, acc1);
                acc2 = fmaf(p.prob[(e + 2) * H + h], m2, acc2);
                acc3 = fmaf(p.prob[(e + 3) * H + h], m3, acc3);
            }
            for (; e < e1; e++)
                acc0 = fmaf(p.prob[e * H + h], p.val[dst[e] * HD + x] + p.bij[e * HD + x], acc0);
        } else {
            for (; e + 4 <= e1; e += 4) {
                acc0 = fmaf(p.prob[e * H + h], p.val[dst[e] * HD + x], acc0);
                acc1 = fmaf(p.prob[(e + 1) * H + h], p.val[dst[e + 1] * HD + x], acc1);
                acc2 = fmaf(p.prob[(e + 2) * H + h], p.val[dst[e + 2] * HD + x], acc2);
                acc3 = fmaf(p.prob[(e + 3) * H + h], p.val[dst[e + 3] * HD + x], acc3);
            }
            for (; e < e1; e++) acc0 = fmaf(p.prob[e * H + h], p.val[dst[e] * HD + x], acc0);
        }
        p.out[i * HD + x] = (acc0 + acc1) + (acc2 + acc3);
    }
}

// ----------------------------------------------------------------- backward
// rows: per query i, lane = (head, value component); Dv is a power of two <= 64
// so that the lanes of one head form an aligned group.
__global__ __launch_bounds__(256) void fused_dpa_bwd_rows_kernel(DpaArgs p)
{
    const int lane = threadIdx.x & 63;
    const int64_t i = (int64_t)blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
    if (i >= p.N) return;
    const int H = p.H, Dv = p.Dv, HD = H * Dv;
    const int64_t e0 = p.e_start[i], e1 = p.e_start[i + 1];
    const int64_t *dst = p.edges + p.E;
    for (int x0 = 0; x0 < HD; x0 += WAVE) {
        const int x = x0 + lane;
        const bool on = x < HD;
        const int h = on ? x / Dv : 0;
        const float go = on ? p.gout[i * HD + x] : 0.f;
        const float o = on ? p.out_in[i * HD + x] : 0.f;
        for (int64_t e = e0; e < e1; e++) {
            float part = 0.f;
            if (on) {
                float t = go * p.prob_in[e * H + h];
                float m = p.val[dst[e] * HD + x];
                if (p.bij) m += p.bij[e * HD + x];
                if (p.gbij) p.gbij[e * HD + x] = t;
                part = (m - o) * t;
            }
            for (int off = Dv >> 1; off > 0; off >>= 1) part += __shfl_xor(part, off, WAVE);
            if (on && (x % Dv) == 0) p.gaij[e * H + h] = part;
        }
    }
}

// queries: gq[i,h,:] = sum_j gs_ij k_j ; lane = (head, key component)
__global__ __launch_bounds__(256) void fused_dpa_bwd_que_kernel(DpaArgs p)
{
    const int lane = threadIdx.x & 63;
    const int64_t i = (int64_t)blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
    if (i >= p.N) return;
    const int H = p.H, Dk = p.Dk, HD = H * Dk;
    const int64_t e0 = p.e_start[i], e1 = p.e_start[i + 1];
    const int64_t *dst = p.edges + p.E;
    for (int x = lane; x < HD; x += WAVE) {
        const int h = x / Dk;
        float acc0 = 0.f, acc1 = 0.f, acc2 = 0.f, acc3 = 0.f;
        int64_t e = e0;
        for (; e + 4 <= e1; e += 4) {
            acc0 = fmaf(p.gaij[e * H + h], p.key[dst[e] * HD + x], acc0);
            acc1 = fmaf(p.gaij[(e + 1) * H + h], p.key[dst[e + 1] * HD + x], acc1);
            acc2 = fmaf(p.gaij[(e + 2) * H + h], p.key[dst[e + 2] * HD + x], acc2);
            acc3 = fmaf(p.gaij[(e + 3) * H + h], p.key[dst[e + 3] * HD + x], acc3);
        }
        for (; e < e1; e++) acc0 = fmaf(p.gaij[e * H + h], p.key[dst[e] * HD + x], acc0);
        p.gque[i * HD + x] = (acc0 + acc1) + (acc2 + acc3);
    }
}

// keys: per key atom j, walk the column (i, j) of the crystal's dense block.
__global__ __launch_bounds__(256) void fused_dpa_bwd_keys_kernel(DpaArgs p)
{
    const int lane = threadIdx.x & 63;
    const int64_t j = (int64_t)blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
    if (j >= p.N) return;
    const int H = p.H, Dk = p.Dk, Dv = p.Dv;
    const int64_t b = p.batch[j];
    const int64_t ab = p.atom_start[b];
    const int64_t n = p.atom_start[b + 1] - ab;
    const int64_t eb = p.edge_start[b] + (j - ab);
    const int HDv = H * Dv, HDk = H * Dk;
    for (int x = lane; x < HDv; x += WAVE) {
        const int h = x / Dv;
        float acc0 = 0.f, acc1 = 0.f;
        int64_t il = 0;
        for (; il + 2 <= n; il += 2) {
            acc0 = fmaf(p.gout[(ab + il) * HDv + x], p.prob_in[(eb + il * n) * H + h], acc0);
            acc1 = fmaf(p.gout[(ab + il + 1) * HDv + x], p.prob_in[(eb + (il + 1) * n) * H + h], acc1);
        }
        if (il < n) acc0 = fmaf(p.gout[(ab + il) * HDv + x], p.prob_in[(eb + il * n) * H + h], acc0);
        p.gval[j * HDv + x] = acc0 + acc1;
    }
    for (int x = lane; x < HDk; x += WAVE) {
        const int h = x / Dk;
        float acc0 = 0.f, acc1 = 0.f;
        int64_t il = 0;
        for (; il + 2 <= n; il += 2) {
            acc0 = fmaf(p.que[(ab + il) * HDk + x], p.gaij[(eb + il * n) * H + h], acc0);
            acc1 = fmaf(p.que[(ab + il + 1) * HDk + x], p.gaij[(eb + (il + 1) * n) * H + h], acc1);
        }
        if (il < n) acc0 = fmaf(p.que[(ab + il) * HDk + x], p.gaij[(eb + il * n) * H + h], acc0);
        p.gkey[j * HDk + x] = acc0 + acc1;
    }
}

int check_dims(const char *who, int64_t N, int64_t H, int64_t E, int64_t Dk, int64_t Dv)
{
    CF_REQUIRE(N >= 0 && E >= 0, CF_ERR_INVALID_ARGUMENT, "%s: negative size", who);
    CF_REQUIRE(H >= 1 && H <= MAXH, CF_ERR_UNSUPPORTED, "%s: head count %lld outside 1..%d", who,
               (long long)H, MAXH);
    CF_REQUIRE(Dk >= 1 && Dk <= 256 && Dv >= 1 && Dv <= 256, CF_ERR_UNSUPPORTED,
               "%s: head dims (%lld,%lld) outside 1..256", who, (long long)Dk, (long long)Dv);
    return CF_OK;
}

template <int H>
void launch_fwd(const DpaArgs &p, hipStream_t st)
{
    const int wpb = 4;
    fused_dpa_fwd_kernel<H><<<(int)((p.N + wpb - 1) / wpb), wpb * WAVE, 0, st>>>(p);
}

}  // namespace

extern "C" int cf_fused_dpa_fwd(const float *que, const float *key, const float *val,
                                const float *aij_eh, const float *bij_ehd, const int64_t *edge_ij_e,
                                const int64_t *e_start_i, int64_t N, int64_t H, int64_t E, int64_t Dk,
                                int64_t Dv, float *prob_eh, float *out, void *stream)
{
    int rc = check_dims("cf_fused_dpa_fwd", N, H, E, Dk, Dv);
    if (rc) return rc;
    if (N == 0) return CF_OK;
    CF_REQUIRE(que && key && val && e_start_i && out && (E == 0 || (edge_ij_e && prob_eh)),
               CF_ERR_INVALID_ARGUMENT, "cf_fused_dpa_fwd: null pointer");
    DpaArgs p{};
    p.que = que; p.key = key; p.val = val; p.aij = aij_eh; p.bij = bij_ehd;
    p.edges = edge_ij_e; p.e_start = e_start_i;
    p.prob = prob_eh; p.out = out;
    p.N = N; p.E = E; p.H = (int)H; p.Dk = (int)Dk; p.Dv = (int)Dv;
    hipStream_t st = (hipStream_t)stream;
    switch (H) {
        case 1: launch_fwd<1>(p, st); break;
        case 2: launch_fwd<2>(p, st); break;
        case 4: launch_fwd<4>(p, st); break;
        case 8: launch_fwd<8>(p, st); break;
        case 16: launch_fwd<16>(p, st); break;
        default:
            CF_REQUIRE(false, CF_ERR_UNSUPPORTED, "cf_fused_dpa_fwd: head count %lld not supported (1,2,4,8,16)",
                       (long long)H);
    }
    CF_CHECK_LAUNCH("cf_fused_dpa_fwd");
    return CF_OK;
}

extern "C" int cf_fused_dpa_bwd(const float *que, const float *key, const float *val,
                                const float *bij_ehd, const int64_t *batch_i, const int64_t *edge_ij_e,
                                const int64_t *e_start_i, const int64_t *atom_start_n,
                                const int64_t *edge_start_n, int64_t N, int64_t H, int64_t E, int64_t B,
                                int64_t Dk, int64_t Dv, const float *prob_eh, const float *out,
                                const float *gout, float *gque, float *gkey, float *gval, float *gaij,
                                float *gbij, void *stream)
{
    int rc = check_dims("cf_fused_dpa_bwd", N, H, E, Dk, Dv);
    if (rc) return rc;
    CF_REQUIRE(B >= 0, CF_ERR_INVALID_ARGUMENT, "cf_fused_dpa_bwd: negative B");
    CF_REQUIRE(Dv <= 64 && (Dv & (Dv - 1)) == 0, CF_ERR_UNSUPPORTED,
               "cf_fused_dpa_bwd: value head dim %lld must be a power of two <= 64", (long long)Dv);
    if (N == 0) return CF_OK;
    CF_REQUIRE(que && key && val && batch_i && e_start_i && atom_start_n && edge_start_n && out && gout &&
                   gque && gkey && gval && (E == 0 || (edge_ij_e && prob_eh && gaij)),
               CF_ERR_INVALID_ARGUMENT, "cf_fused_dpa_bwd: null pointer");
    DpaArgs p{};
    p.que = que; p.key = key; p.val = val; p.bij = bij_ehd;
    p.batch = batch_i; p.edges = edge_ij_e; p.e_start = e_start_i;
    p.atom_start = atom_start_n; p.edge_start = edge_start_n;
    p.prob_in = prob_eh; p.out_in = out; p.gout = gout;
    p.gque = gque; p.gkey = gkey; p.gval = gval; p.gaij = gaij; p.gbij = gbij;
    p.N = N; p.E = E; p.H = (int)H; p.Dk = (int)Dk; p.Dv = (int)Dv;
    hipStream_t st = (hipStream_t)stream;
    const int wpb = 4;
    const int grid = (int)((N + wpb - 1) / wpb);
    fused_dpa_bwd_rows_kernel<<<grid, wpb * WAVE, 0, st>>>(p);
    CF_CHECK_LAUNCH("cf_fused_dpa_bwd: rows");
    fused_dpa_bwd_que_kernel<<<grid, wpb * WAVE, 0, st>>>(p);
    CF_CHECK_LAUNCH("cf_fused_dpa_bwd: queries");
    fused_dpa_bwd_keys_kernel<<<grid, wpb * WAVE, 0, st>>>(p);
    CF_CHECK_LAUNCH("cf_fused_dpa_bwd: keys");
    return CF_OK;
}
