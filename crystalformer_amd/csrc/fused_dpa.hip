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
    const int64_t *live_N;   // forward only, nullable: live atom count on the device (N is then the capacity)
};

constexpr int MAXH = 16;

// ------------------------------------------------------------------ forward
template <int H>
__global__ __launch_bounds__(256) void fused_dpa_fwd_kernel(DpaArgs p)
{
    const int lane = threadIdx.x & 63;
    const int64_t i = (int64_t)blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
    if (i >= live_count(p.live_N, p.N)) return;   // whole wave exits together
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
// value row and b_ij row as consecutive 16-byte pieces (fully coalesced).
// A step covers 4 edges per slot (4*4*ES edges per work-group); all of its loads
// are issued before the first is consumed, without branches: an edge past the end
// of the row reads the row's last edge instead and is masked out of the sums, so
// a row of up to one step costs one memory round trip after its key indices.
// The key indices of the next step are fetched one step ahead.  The partial
// (max, sum, output) of slots and wavefronts are merged through shuffles and LDS.
// Raw logits of whole steps are parked in prob[e,h] and normalised by a closing
// sweep (4*H bytes per edge); those of the last, partial step stay in registers.
// Needs Dk == Dv, Dv/4 a power of two, H*Dv/4 <= 64.
typedef float float4_v __attribute__((ext_vector_type(4)));

constexpr int DPA_WPQ = 4;     // wavefronts per query row

// Sum over the DV4 adjacent lanes that hold one head's components; every lane of the
// wavefront must be active.
template <int DV4>
__device__ __forceinline__ float head_sum(float s)
{
#pragma unroll
    for (int off = DV4 >> 1; off >= 4; off >>= 1) s += __shfl_xor(s, off, WAVE);
    if (DV4 >= 4) s += dpp_f<DPP_QUAD_2301, 0xF>(0.f, s);
    if (DV4 >= 2) s += dpp_f<DPP_QUAD_1032, 0xF>(0.f, s);
    return s;
}

// Loads and stores at a 32-bit byte offset from a wave-uniform base (scalar base + vector
// offset addressing: no 64-bit address per lane).
__device__ __forceinline__ float4_v ld4(const void *base, uint32_t byte_off)
{
    return *reinterpret_cast<const float4_v *>(static_cast<const char *>(base) + byte_off);
}
// The same for data that is read once (the b_ij stream): marked as streaming so that it does not
// push the key / value rows, which every query row of a crystal reads again, out of the caches.
__device__ __forceinline__ float4_v ld4_stream(const void *base, uint32_t byte_off)
{
    return __builtin_nontemporal_load(reinterpret_cast<const float4_v *>(static_cast<const char *>(base) + byte_off));
}
__device__ __forceinline__ float ld1(const void *base, uint32_t byte_off)
{
    return *reinterpret_cast<const float *>(static_cast<const char *>(base) + byte_off);
}
__device__ __forceinline__ void st1(void *base, uint32_t byte_off, float v)
{
    *reinterpret_cast<float *>(static_cast<char *>(base) + byte_off) = v;
}

// Every byte offset into prob / b_ij / key / value fits 32 bits (checked by the host).
// PREFETCH (long rows): the key indices of the next step are fetched one step ahead and every
// load of a step is in flight together (one memory round trip per step, 80 registers).
// Otherwise (rows of about one step): the indices are read at the top of the step and the
// register budget is that of 8 resident wavefronts per SIMD, which the compiler meets by
// fetching the value rows after the key rows have been used: one more round trip, and all
// rows of a small batch resident at once.
template <int DV4, bool HAS_A, bool HAS_B, bool PREFETCH>
__global__ __launch_bounds__(256, (PREFETCH ? 6 : 7)) void fused_dpa_fwd_stream_kernel(DpaArgs p, int LPE)
{
    __shared__ float part[DPA_WPQ][WAVE][6];
    __shared__ float fin[2][MAXH];
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const uint32_t i = blockIdx.x;
    const uint32_t H = p.H;
    const uint32_t HD4 = LPE;                  // float4 pieces per edge row
    const int ES = WAVE / LPE;                 // edge slots per wavefront
    const int es = lane / LPE;
    const uint32_t piece = lane - es * LPE;    // which float4 of the (H,Dv) row
    const uint32_t h = piece / DV4;
    const bool lead = (piece % DV4) == 0;      // first piece of its head: owns the logit
    const uint32_t e0 = (uint32_t)p.e_start[i], e1 = (uint32_t)p.e_start[i + 1];
    if (p.live_N && (int64_t)i >= live_count(p.live_N, p.N)) return;   // beyond the live atoms (whole work-group)
    if (e0 >= e1) {                            // an atom without edges yields zeros (whole work-group)
        if (threadIdx.x < HD4)
            reinterpret_cast<float4_v *>(p.out)[i * HD4 + threadIdx.x] = float4_v{0.f, 0.f, 0.f, 0.f};
        return;
    }
    const uint32_t e_last = e1 - 1;
    const int64_t *dst = p.edges + p.E;
    const float4_v q4 = ld4(p.que, (i * HD4 + piece) * 16u);

    float m = -1.0e30f, l = 0.f;
    float4_v acc = {0.f, 0.f, 0.f, 0.f};
    float4_v k4[4], v4[4], b4[4];
    float av[4];
    auto fetch = [&](int u, uint32_t e, uint32_t j) {
        // (independent of the key index: first; long rows: a stream that is read once)
        if (HAS_B) b4[u] = PREFETCH ? ld4_stream(p.bij, (e * HD4 + piece) * 16u) : ld4(p.bij, (e * HD4 + piece) * 16u);
        if (HAS_A) av[u] = ld1(p.aij, (e * H + h) * 4u);
        k4[u] = ld4(p.key, (j * HD4 + piece) * 16u);
        v4[u] = ld4(p.val, (j * HD4 + piece) * 16u);
    };
    auto fold = [&](int u, bool valid) -> float {
        float4_v vv = v4[u];
        if (HAS_B) vv += b4[u];
        float s = q4.x * k4[u].x + q4.y * k4[u].y + q4.z * k4[u].z + q4.w * k4[u].w;
        s = head_sum<DV4>(s);
        if (HAS_A) s += av[u];
        const float m_new = valid ? fmaxf(m, s) : m;
        const float sc = exp2_hw((m - m_new) * LOG2E);
        const float pe = valid ? exp2_hw((s - m_new) * LOG2E) : 0.f;
        l = l * sc + pe;
        acc = acc * sc + vv * pe;
        m = m_new;
        return s;
    };
    const uint32_t stride = DPA_WPQ * ES;
    // the main loop takes whole steps of 4 * stride edges (the same number in every lane), the
    // rest of the row (fewer than 4 * stride edges) is the partial step
    uint32_t eb = e0;
    uint32_t e = eb + wave * ES + es;
    float s_tail[4];
    uint32_t jn[4];
    if (PREFETCH) {
#pragma unroll
        for (int u = 0; u < 4; u++) jn[u] = (uint32_t)dst[min(e + u * stride, e_last)];
    }
    for (;;) {
        const bool last = eb + 4 * stride >= e1;                    // uniform
        if (!PREFETCH) {
#pragma unroll
            for (int u = 0; u < 4; u++) jn[u] = (uint32_t)dst[min(e + u * stride, e_last)];
        }
#pragma unroll
        for (int u = 0; u < 4; u++) fetch(u, min(e + u * stride, e_last), jn[u]);
        if (PREFETCH && !last) {
#pragma unroll
            for (int u = 0; u < 4; u++) jn[u] = (uint32_t)dst[min(e + (4 + u) * stride, e_last)];
        }
#pragma unroll
        for (int u = 0; u < 4; u++) s_tail[u] = fold(u, e + u * stride < e1);
        if (last) break;
        if (lead) {
#pragma unroll
            for (int u = 0; u < 4; u++) st1(p.prob, ((e + u * stride) * H + h) * 4u, s_tail[u]);
        }
        eb += 4 * stride;
        e += 4 * stride;
    }
    const uint32_t e_tail = e;                     // first edge of this lane's slot in the last step
    const uint32_t parked = (eb - e0) * H;         // logits parked by the earlier steps
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
    const bool closer = wave == 0 && es == 0;
    if (closer) {
        for (int w = 1; w < DPA_WPQ; w++) {
            const float *src = part[w][piece];
            merge(src[0], src[1], float4_v{src[2], src[3], src[4], src[5]});
        }
        const float inv = l > 0.f ? 1.0f / l : 0.f;
        acc = acc * inv;
        if (lead) {
            fin[0][h] = m;
            fin[1][h] = inv;
        }
    }
    __syncthreads();
    if (closer) reinterpret_cast<float4_v *>(p.out)[i * HD4 + piece] = acc;   // after the barrier: nothing waits for it
    // normalise: the partial step from registers, the parked logits in place (element x of the
    // row's (n,H) block belongs to head x % H)
    if (lead) {
        const float mt = fin[0][h], it = fin[1][h];
#pragma unroll
        for (int u = 0; u < 4; u++)
            if (e_tail + u * stride < e1)
                st1(p.prob, ((e_tail + u * stride) * H + h) * 4u, exp2_hw((s_tail[u] - mt) * LOG2E) * it);
    }
    if (parked > 0) {
        const uint32_t hx = threadIdx.x % H;
        const float mh = fin[0][hx], ih = fin[1][hx];
        float *row = p.prob + (size_t)e0 * H;
        for (uint32_t x = threadIdx.x; x < parked; x += blockDim.x) row[x] = exp2_hw((row[x] - mh) * LOG2E) * ih;
    }
}

// ------------------------------------------------- backward, streaming version
// Same lane layout and load batching as the streaming forward (work-group of 4
// wavefronts per atom, lane = (edge slot, head, 4 components), 4 edges per slot and
// step, loads of a step issued together, edges past the end clamped and masked),
// two kernels, fixed summation order:
//   query side  per query i over its edge row: gb_ij = go_i p_ij (stored),
//               gs_ij = sum_d (v_j + b_ij - o_i) gb_ij (stored as gaij),
//               gq_i = sum_j gs_ij k_j;
//   key side    per key j over the column (i, j) of the crystal's dense block:
//               gv_j = sum_i go_i p_ij, gk_j = sum_i gs_ij q_i.
__device__ __forceinline__ void st4(void *base, uint32_t byte_off, float4_v v)
{
    *reinterpret_cast<float4_v *>(static_cast<char *>(base) + byte_off) = v;
}
// (for data written once and not read again by this launch: the gb_ij stream)
__device__ __forceinline__ void st4_stream(void *base, uint32_t byte_off, float4_v v)
{
    __builtin_nontemporal_store(v, reinterpret_cast<float4_v *>(static_cast<char *>(base) + byte_off));
}

// STREAM (long rows): b_ij is read and gb_ij written with the streaming hint.
template <int DV4, bool HAS_B, bool WANT_GB, bool STREAM>
__global__ __launch_bounds__(256) void fused_dpa_bwd_query_stream_kernel(DpaArgs p, int LPE)
{
    __shared__ float part[DPA_WPQ][WAVE][4];
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const uint32_t i = blockIdx.x;
    const uint32_t H = p.H;
    const uint32_t HD4 = LPE;
    const int ES = WAVE / LPE;
    const int es = lane / LPE;
    const uint32_t piece = lane - es * LPE;
    const uint32_t h = piece / DV4;
    const bool lead = (piece % DV4) == 0;
    const uint32_t e0 = (uint32_t)p.e_start[i], e1 = (uint32_t)p.e_start[i + 1];
    if (e0 >= e1) {                            // an atom without edges: no query gradient (whole work-group)
        if (threadIdx.x < HD4) st4(p.gque, (i * HD4 + threadIdx.x) * 16u, float4_v{0.f, 0.f, 0.f, 0.f});
        return;
    }
    const uint32_t e_last = e1 - 1;
    const int64_t *dst = p.edges + p.E;
    const float4_v go4 = ld4(p.gout, (i * HD4 + piece) * 16u);
    const float4_v o4 = ld4(p.out_in, (i * HD4 + piece) * 16u);
    float4_v gq = {0.f, 0.f, 0.f, 0.f};
    const uint32_t stride = DPA_WPQ * ES;
    uint32_t e = e0 + wave * ES + es;
    for (uint32_t eb = e0; eb < e1; eb += 4 * stride, e += 4 * stride) {
        uint32_t ec[4], j[4];
        float pr[4], gsv[4];
        float4_v k4[4], m4[4], b4[4];
#pragma unroll
        for (int u = 0; u < 4; u++) {
            ec[u] = min(e + u * stride, e_last);
            j[u] = (uint32_t)dst[ec[u]];
        }
#pragma unroll
        for (int u = 0; u < 4; u++) {
            pr[u] = ld1(p.prob_in, (ec[u] * H + h) * 4u);
            if (HAS_B) b4[u] = STREAM ? ld4_stream(p.bij, (ec[u] * HD4 + piece) * 16u) : ld4(p.bij, (ec[u] * HD4 + piece) * 16u);
            m4[u] = ld4(p.val, (j[u] * HD4 + piece) * 16u);
        }
#pragma unroll
        for (int u = 0; u < 4; u++) {
            const bool valid = e + u * stride < e1;
            const float4_v t4 = go4 * pr[u];
            float4_v d4 = m4[u];
            if (HAS_B) d4 += b4[u];
            d4 -= o4;
            float gs = d4.x * t4.x + d4.y * t4.y + d4.z * t4.z + d4.w * t4.w;
            gs = head_sum<DV4>(gs);
            if (valid) {
                if (WANT_GB) {
                    if (STREAM) st4_stream(p.gbij, (ec[u] * HD4 + piece) * 16u, t4);
                    else st4(p.gbij, (ec[u] * HD4 + piece) * 16u, t4);
                }
                if (lead) st1(p.gaij, (ec[u] * H + h) * 4u, gs);
            }
            gsv[u] = valid ? gs : 0.f;
        }
        // the key rows (cache hits: the value rows of the same atoms were just read) come second,
        // into the registers the value and b_ij rows have left
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int u = 0; u < 4; u++) k4[u] = ld4(p.key, (j[u] * HD4 + piece) * 16u);
#pragma unroll
        for (int u = 0; u < 4; u++) gq += k4[u] * gsv[u];
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
        st4(p.gque, (i * HD4 + piece) * 16u, gq);
    }
}

template <int DV4>
__global__ __launch_bounds__(256) void fused_dpa_bwd_key_stream_kernel(DpaArgs p, int LPE)
{
    __shared__ float part[DPA_WPQ][WAVE][8];
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const uint32_t j = blockIdx.x;
    const uint32_t H = p.H;
    const uint32_t HD4 = LPE;
    const int ES = WAVE / LPE;
    const int es = lane / LPE;
    const uint32_t piece = lane - es * LPE;
    const uint32_t h = piece / DV4;
    const int64_t b = p.batch[j];
    const uint32_t ab = (uint32_t)p.atom_start[b];
    const uint32_t n = (uint32_t)p.atom_start[b + 1] - ab;          // >= 1: atom j is one of them
    const uint32_t ebase = (uint32_t)p.edge_start[b] + (j - ab);
    float4_v gv = {0.f, 0.f, 0.f, 0.f}, gk = {0.f, 0.f, 0.f, 0.f};
    const uint32_t stride = DPA_WPQ * ES;
    uint32_t il = wave * ES + es;
    for (uint32_t ib = 0; ib < n; ib += 4 * stride, il += 4 * stride) {
        float pr[4], gs[4];
        float4_v g4[4], q4[4];
#pragma unroll
        for (int u = 0; u < 4; u++) {
            const uint32_t ic = min(il + u * stride, n - 1);
            const uint32_t e = ebase + ic * n;
            pr[u] = ld1(p.prob_in, (e * H + h) * 4u);
            gs[u] = ld1(p.gaij, (e * H + h) * 4u);
            g4[u] = ld4(p.gout, ((ab + ic) * HD4 + piece) * 16u);
            q4[u] = ld4(p.que, ((ab + ic) * HD4 + piece) * 16u);
        }
#pragma unroll
        for (int u = 0; u < 4; u++) {
            const bool valid = il + u * stride < n;
            gv += g4[u] * (valid ? pr[u] : 0.f);
            gk += q4[u] * (valid ? gs[u] : 0.f);
        }
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
        st4(p.gval, (j * HD4 + piece) * 16u, gv);
        st4(p.gkey, (j * HD4 + piece) * 16u, gk);
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

template <int DV4, bool PREFETCH>
void launch_fwd_stream_dv(const DpaArgs &p, int lpe, hipStream_t st)
{
    const dim3 grid((unsigned)p.N), block(DPA_WPQ * WAVE);
    if (p.aij && p.bij) fused_dpa_fwd_stream_kernel<DV4, true, true, PREFETCH><<<grid, block, 0, st>>>(p, lpe);
    else if (p.aij) fused_dpa_fwd_stream_kernel<DV4, true, false, PREFETCH><<<grid, block, 0, st>>>(p, lpe);
    else if (p.bij) fused_dpa_fwd_stream_kernel<DV4, false, true, PREFETCH><<<grid, block, 0, st>>>(p, lpe);
    else fused_dpa_fwd_stream_kernel<DV4, false, false, PREFETCH><<<grid, block, 0, st>>>(p, lpe);
}

void launch_fwd_stream(const DpaArgs &p, int dv4, int lpe, hipStream_t st)
{
    // mean row length beyond two steps of the work-group: the variant that keeps one round trip per step
    const int64_t step_edges = 4 * DPA_WPQ * (WAVE / lpe);
    const bool long_rows = p.E > 2 * step_edges * p.N;
#define CF_DPA_FWD(DV) \
    do { if (long_rows) launch_fwd_stream_dv<DV, true>(p, lpe, st); else launch_fwd_stream_dv<DV, false>(p, lpe, st); } while (0)
    switch (dv4) {
        case 1: CF_DPA_FWD(1); break;
        case 2: CF_DPA_FWD(2); break;
        case 4: CF_DPA_FWD(4); break;
        case 8: CF_DPA_FWD(8); break;
        default: CF_DPA_FWD(16); break;
    }
#undef CF_DPA_FWD
}

template <int DV4, bool STREAM>
void launch_bwd_query_dv(const DpaArgs &p, int lpe, hipStream_t st)
{
    const dim3 grid((unsigned)p.N), block(DPA_WPQ * WAVE);
    if (p.bij && p.gbij) fused_dpa_bwd_query_stream_kernel<DV4, true, true, STREAM><<<grid, block, 0, st>>>(p, lpe);
    else if (p.bij) fused_dpa_bwd_query_stream_kernel<DV4, true, false, STREAM><<<grid, block, 0, st>>>(p, lpe);
    else if (p.gbij) fused_dpa_bwd_query_stream_kernel<DV4, false, true, STREAM><<<grid, block, 0, st>>>(p, lpe);
    else fused_dpa_bwd_query_stream_kernel<DV4, false, false, STREAM><<<grid, block, 0, st>>>(p, lpe);
}

template <int DV4>
void launch_bwd_stream_dv(const DpaArgs &p, int lpe, hipStream_t st)
{
    const dim3 grid((unsigned)p.N), block(DPA_WPQ * WAVE);
    // (the forward's rule for long rows: more than two steps of a work-group on average)
    const int64_t step_edges = 4 * DPA_WPQ * (WAVE / lpe);
    if (p.E > 2 * step_edges * p.N) launch_bwd_query_dv<DV4, true>(p, lpe, st);
    else launch_bwd_query_dv<DV4, false>(p, lpe, st);
    fused_dpa_bwd_key_stream_kernel<DV4><<<grid, block, 0, st>>>(p, lpe);
}

void launch_bwd_stream(const DpaArgs &p, int dv4, int lpe, hipStream_t st)
{
    switch (dv4) {
        case 1: launch_bwd_stream_dv<1>(p, lpe, st); break;
        case 2: launch_bwd_stream_dv<2>(p, lpe, st); break;
        case 4: launch_bwd_stream_dv<4>(p, lpe, st); break;
        case 8: launch_bwd_stream_dv<8>(p, lpe, st); break;
        default: launch_bwd_stream_dv<16>(p, lpe, st); break;
    }
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
    p.live_N = cf::live_atoms(N);
    hipStream_t st = (hipStream_t)stream;
    // streaming kernel when a head's components split into 16-byte pieces that tile a wavefront
    const int64_t dv4 = Dv / 4, lpe = H * dv4;
    const bool pow2 = (dv4 & (dv4 - 1)) == 0 && (H & (H - 1)) == 0;
    const bool fits32 = (E + 1) * H * Dv * 4 < (1ll << 32) && (N + 1) * H * Dv * 4 < (1ll << 32);
    if (Dk == Dv && Dv % 4 == 0 && pow2 && lpe >= 1 && lpe <= 64 && dv4 <= 16 && fits32) {
        launch_fwd_stream(p, (int)dv4, (int)lpe, st);
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
        const bool fits32 = (E + 1) * H * Dv * 4 < (1ll << 32) && (N + 1) * H * Dv * 4 < (1ll << 32);
        if (Dk == Dv && Dv % 4 == 0 && pow2 && lpe >= 1 && lpe <= 64 && dv4 <= 16 && fits32) {
            launch_bwd_stream(p, (int)dv4, (int)lpe, st);
            CF_CHECK_LAUNCH("cf_fused_dpa_bwd: streaming kernels");
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
