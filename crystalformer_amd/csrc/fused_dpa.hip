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


// ------------------------------------------------- forward, streaming version
// One work-group of 4 wavefronts per query atom, single pass over the edge row
// with a running (max, sum, output) per head ("online" softmax).  Lane = (edge
// slot, head, 4 components): the H*Dv/4 lanes of a slot read one edge's key row,
// value row and b_ij row as consecutive 16-byte pieces (fully coalesced);
// 4*ES = 4*64/(H*Dv/4) edges are in flight per step, the loop is unrolled 4x and
// the key indices of the next step are fetched one step ahead.  The partial
// (max, sum, output) of slots and wavefronts are merged through shuffles and LDS.
// Raw logits are parked in prob[e,h] and normalised by a second, cheap sweep
// (4*H bytes per edge).  Needs Dk == Dv, Dv/4 a power of two, H*Dv/4 <= 64.
typedef float float4_v __attribute__((ext_vector_type(4)));

constexpr int DPA_WPQ = 4;     // wavefronts per query row

__global__ __launch_bounds__(256) void fused_dpa_fwd_stream_kernel(DpaArgs p, int DV4, int LPE)
{
    __shared__ float part[DPA_WPQ][WAVE][6];
    __shared__ float fin[2][MAXH];
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int64_t i = blockIdx.x;
    const int H = p.H;
    const int HD4 = LPE;                       // float4 pieces per edge row
    const int ES = WAVE / LPE;                 // edge slots per wavefront
    const int es = lane / LPE;
    const int piece = lane - es * LPE;         // which float4 of the (H,Dv) row
    const int h = piece / DV4;
    const bool lead = (piece - h * DV4) == 0;  // first piece of its head: owns the logit
    const int64_t e0 = p.e_start[i], e1 = p.e_start[i + 1];
    const int64_t *dst = p.edges + p.E;
    const float4_v *key4 = reinterpret_cast<const float4_v *>(p.key);
    const float4_v *val4 = reinterpret_cast<const float4_v *>(p.val);
    const float4_v *bij4 = reinterpret_cast<const float4_v *>(p.bij);
    const float4_v q4 = reinterpret_cast<const float4_v *>(p.que)[i * HD4 + piece];

    float m = -1.0e30f, l = 0.f;
    float4_v acc = {0.f, 0.f, 0.f, 0.f};
    // Raw logits of the main loop are parked in prob[] and normalised by the closing sweep; those of
    // the last (for most rows: the only) partial step stay in registers and are written once,
    // normalised, so that a short row never reads its own stores back.
    auto step = [&](int64_t e, int64_t j, bool park) -> float {
        const float4_v k4 = key4[j * HD4 + piece];
        float4_v v4 = val4[j * HD4 + piece];
        if (bij4) {
            const float4_v b4 = bij4[e * HD4 + piece];
            v4 += b4;
        }
        float s = q4.x * k4.x + q4.y * k4.y + q4.z * k4.z + q4.w * k4.w;
        for (int off = DV4 >> 1; off > 0; off >>= 1) s += __shfl_xor(s, off, WAVE);
        if (p.aij) s += p.aij[e * H + h];
        if (park && lead) p.prob[e * H + h] = s;
        const float m_new = fmaxf(m, s);
        const float sc = exp2_hw((m - m_new) * LOG2E);
        const float pe = exp2_hw((s - m_new) * LOG2E);
        l = l * sc + pe;
        acc = acc * sc + v4 * pe;
        m = m_new;
        return s;
    };
    const int stride = DPA_WPQ * ES;
    // the main loop takes whole steps of 4 * stride edges (the same number in every lane), the
    // rest of the row (fewer than 4 * stride edges) is the partial step
    int64_t eb = e0;
    int64_t e = eb + wave * ES + es;
    // key indices one step (4 edges per slot) ahead
    int64_t jn[4];
#pragma unroll
    for (int u = 0; u < 4; u++) jn[u] = (e + u * stride < e1) ? dst[e + u * stride] : 0;
    for (; eb + 4 * stride <= e1; eb += 4 * stride, e += 4 * stride) {
        int64_t jc[4];
#pragma unroll
        for (int u = 0; u < 4; u++) jc[u] = jn[u];
#pragma unroll
        for (int u = 0; u < 4; u++) {
            const int64_t en = e + (4 + u) * stride;
            jn[u] = (en < e1) ? dst[en] : 0;
        }
#pragma unroll
        for (int u = 0; u < 4; u++) step(e + u * stride, jc[u], true);
    }
    const int64_t e_tail = e;                      // first edge of this lane's slot in the last step
    const int64_t parked = (eb - e0) * H;          // logits parked by the main loop
    float s_tail[4];
#pragma unroll
    for (int u = 0; u < 4; u++) {
        s_tail[u] = 0.f;
        if (e_tail + u * stride < e1) s_tail[u] = step(e_tail + u * stride, jn[u], false);
    }
    // merge the edge slots of this wavefront
    auto merge = [&](float mo, float lo, float4_v ao) {
        const float m_new = fmaxf(m, mo);
        const float s1 = exp2_hw((m - m_new) * LOG2E), s2 = exp2_hw((mo - m_new) * LOG2E);
        l = l * s1 + lo * s2;
        acc = acc * s1 + ao * s2;
        m = m_new;
    };
    for (int off = LPE; off < WAVE; off <<= 1) {
        const float mo = __shfl_xor(m, off, WAVE);
        const float lo = __shfl_xor(l, off, WAVE);
        float4_v ao;
        ao.x = __shfl_xor(acc.x, off, WAVE);
        ao.y = __shfl_xor(acc.y, off, WAVE);
        ao.z = __shfl_xor(acc.z, off, WAVE);
        ao.w = __shfl_xor(acc.w, off, WAVE);
        merge(mo, lo, ao);
    }
    // merge the wavefronts (fixed order 0,1,2,3) in wavefront 0
    if (es == 0) {
        float *dstp = part[wave][piece];
        dstp[0] = m; dstp[1] = l; dstp[2] = acc.x; dstp[3] = acc.y; dstp[4] = acc.z; dstp[5] = acc.w;
    }
    __syncthreads();
    if (wave == 0 && es == 0) {
        for (int w = 1; w < DPA_WPQ; w++) {
            const float *src = part[w][piece];
            merge(src[0], src[1], float4_v{src[2], src[3], src[4], src[5]});
        }
        const float inv = l > 0.f ? 1.0f / l : 0.f;     // an atom without edges yields zeros
        reinterpret_cast<float4_v *>(p.out)[i * HD4 + piece] = acc * inv;
        if (lead) {
            fin[0][h] = m;
            fin[1][h] = inv;
        }
    }
    __syncthreads();
    // normalise the parked logits: element x of the row's (n,H) block belongs to head x % H
    if (lead) {
        const float mt = fin[0][h], it = fin[1][h];
#pragma unroll
        for (int u = 0; u < 4; u++)
            if (e_tail + u * stride < e1)
                p.prob[(e_tail + u * stride) * H + h] = exp2_hw((s_tail[u] - mt) * LOG2E) * it;
    }
    const int hx = threadIdx.x % H;
    const float mh = fin[0][hx], ih = fin[1][hx];
    float *row = p.prob + e0 * H;
    for (int64_t x = threadIdx.x; x < parked; x += blockDim.x) row[x] = exp2_hw((row[x] - mh) * LOG2E) * ih;
}

// ------------------------------------------------- backward, streaming version
// Same lane layout as the streaming forward (work-group of 4 wavefronts per atom,
// lane = (edge slot, head, 4 components)), two kernels, fixed summation order:
//   query side  per query i over its edge row: gb_ij = go_i p_ij (stored),
//               gs_ij = sum_d (v_j + b_ij - o_i) gb_ij (stored as gaij),
//               gq_i = sum_j gs_ij k_j;
//   key side    per key j over the column (i, j) of the crystal's dense block:
//               gv_j = sum_i go_i p_ij, gk_j = sum_i gs_ij q_i.
__global__ __launch_bounds__(256) void fused_dpa_bwd_query_stream_kernel(DpaArgs p, int DV4, int LPE)
{
    __shared__ float part[DPA_WPQ][WAVE][4];
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int64_t i = blockIdx.x;
    const int H = p.H;
    const int HD4 = LPE;
    const int ES = WAVE / LPE;
    const int es = lane / LPE;
    const int piece = lane - es * LPE;
    const int h = piece / DV4;
    const bool lead = (piece - h * DV4) == 0;
    const int64_t e0 = p.e_start[i], e1 = p.e_start[i + 1];
    const int64_t *dst = p.edges + p.E;
    const float4_v *key4 = reinterpret_cast<const float4_v *>(p.key);
    const float4_v *val4 = reinterpret_cast<const float4_v *>(p.val);
    const float4_v *bij4 = reinterpret_cast<const float4_v *>(p.bij);
    float4_v *gb4 = reinterpret_cast<float4_v *>(p.gbij);
    const float4_v go4 = reinterpret_cast<const float4_v *>(p.gout)[i * HD4 + piece];
    const float4_v o4 = reinterpret_cast<const float4_v *>(p.out_in)[i * HD4 + piece];
    float4_v gq = {0.f, 0.f, 0.f, 0.f};
    const int stride = DPA_WPQ * ES;
    for (int64_t e = e0 + wave * ES + es; e < e1; e += stride) {
        const int64_t j = dst[e];
        const float pr = p.prob_in[e * H + h];
        const float4_v k4 = key4[j * HD4 + piece];
        float4_v m4 = val4[j * HD4 + piece];
        if (bij4) m4 += bij4[e * HD4 + piece];
        const float4_v t4 = go4 * pr;
        if (gb4) gb4[e * HD4 + piece] = t4;
        m4 -= o4;
        float gs = m4.x * t4.x + m4.y * t4.y + m4.z * t4.z + m4.w * t4.w;
        for (int off = DV4 >> 1; off > 0; off >>= 1) gs += __shfl_xor(gs, off, WAVE);
        if (lead) p.gaij[e * H + h] = gs;
        gq += k4 * gs;
    }
    for (int off = LPE; off < WAVE; off <<= 1) {
        gq.x += __shfl_xor(gq.x, off, WAVE);
        gq.y += __shfl_xor(gq.y, off, WAVE);
        gq.z += __shfl_xor(gq.z, off, WAVE);
        gq.w += __shfl_xor(gq.w, off, WAVE);
    }
    if (es == 0) {
        float *d = part[wave][piece];
        d[0] = gq.x; d[1] = gq.y; d[2] = gq.z; d[3] = gq.w;
    }
    __syncthreads();
    if (wave == 0 && es == 0) {
        for (int w = 1; w < DPA_WPQ; w++) {
            const float *s = part[w][piece];
            gq += float4_v{s[0], s[1], s[2], s[3]};
        }
        reinterpret_cast<float4_v *>(p.gque)[i * HD4 + piece] = gq;
    }
}

__global__ __launch_bounds__(256) void fused_dpa_bwd_key_stream_kernel(DpaArgs p, int DV4, int LPE)
{
    __shared__ float part[DPA_WPQ][WAVE][8];
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int64_t j = blockIdx.x;
    const int H = p.H;
    const int HD4 = LPE;
    const int ES = WAVE / LPE;
    const int es = lane / LPE;
    const int piece = lane - es * LPE;
    const int h = piece / DV4;
    const int64_t b = p.batch[j];
    const int64_t ab = p.atom_start[b];
    const int64_t n = p.atom_start[b + 1] - ab;
    const int64_t eb = p.edge_start[b] + (j - ab);
    const float4_v *que4 = reinterpret_cast<const float4_v *>(p.que);
    const float4_v *go4 = reinterpret_cast<const float4_v *>(p.gout);
    float4_v gv = {0.f, 0.f, 0.f, 0.f}, gk = {0.f, 0.f, 0.f, 0.f};
    const int stride = DPA_WPQ * ES;
    for (int64_t il = wave * ES + es; il < n; il += stride) {
        const int64_t e = eb + il * n;
        const float pr = p.prob_in[e * H + h];
        const float gs = p.gaij[e * H + h];
        gv += go4[(ab + il) * HD4 + piece] * pr;
        gk += que4[(ab + il) * HD4 + piece] * gs;
    }
    for (int off = LPE; off < WAVE; off <<= 1) {
        gv.x += __shfl_xor(gv.x, off, WAVE); gv.y += __shfl_xor(gv.y, off, WAVE);
        gv.z += __shfl_xor(gv.z, off, WAVE); gv.w += __shfl_xor(gv.w, off, WAVE);
        gk.x += __shfl_xor(gk.x, off, WAVE); gk.y += __shfl_xor(gk.y, off, WAVE);
        gk.z += __shfl_xor(gk.z, off, WAVE); gk.w += __shfl_xor(gk.w, off, WAVE);
    }
    if (es == 0) {
        float *d = part[wave][piece];
        d[0] = gv.x; d[1] = gv.y; d[2] = gv.z; d[3] = gv.w;
        d[4] = gk.x; d[5] = gk.y; d[6] = gk.z; d[7] = gk.w;
    }
    __syncthreads();
    if (wave == 0 && es == 0) {
        for (int w = 1; w < DPA_WPQ; w++) {
            const float *s = part[w][piece];
            gv += float4_v{s[0], s[1], s[2], s[3]};
            gk += float4_v{s[4], s[5], s[6], s[7]};
        }
        reinterpret_cast<float4_v *>(p.gval)[j * HD4 + piece] = gv;
        reinterpret_cast<float4_v *>(p.gkey)[j * HD4 + piece] = gk;
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
    // streaming kernel when a head's components split into 16-byte pieces that tile a wavefront
    const int64_t dv4 = Dv / 4, lpe = H * dv4;
    const bool pow2 = (dv4 & (dv4 - 1)) == 0 && (H & (H - 1)) == 0;
    if (Dk == Dv && Dv % 4 == 0 && pow2 && lpe >= 1 && lpe <= 64) {
        fused_dpa_fwd_stream_kernel<<<(int)N, DPA_WPQ * WAVE, 0, st>>>(p, (int)dv4, (int)lpe);
        CF_CHECK_LAUNCH("cf_fused_dpa_fwd");
        return CF_OK;
    }
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
    {
        const int64_t dv4 = Dv / 4, lpe = H * dv4;
        const bool pow2 = (dv4 & (dv4 - 1)) == 0 && (H & (H - 1)) == 0;
        if (Dk == Dv && Dv % 4 == 0 && pow2 && lpe >= 1 && lpe <= 64) {
            fused_dpa_bwd_query_stream_kernel<<<(int)N, DPA_WPQ * WAVE, 0, st>>>(p, (int)dv4, (int)lpe);
            CF_CHECK_LAUNCH("cf_fused_dpa_bwd: query side");
            fused_dpa_bwd_key_stream_kernel<<<(int)N, DPA_WPQ * WAVE, 0, st>>>(p, (int)dv4, (int)lpe);
            CF_CHECK_LAUNCH("cf_fused_dpa_bwd: key side");
            return CF_OK;
        }
    }
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
