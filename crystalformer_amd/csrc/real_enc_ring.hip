// Real-space periodic encoding, forward, with the staged translations of every atom pair kept in
// memory across the blocks of a model (fixed cube of at most 128 translations, shared projection).
//
// What the pair kernel of real_enc_mfma.hip stages per unit -- the translations that reach a bin,
// ordered by the lowest 16-bin tile they reach, with their squared distance, Gaussian argument and
// tile bits, the far ones that can still carry weight, and the smallest squared distance -- depends
// on the geometry and on the bin grid only, not on the Gaussian exponents of a block.  All blocks of
// a forward (and the backward passes) see the same crystals, so the staging is done once
// (ring_stage_kernel, a wavefront per unit, image written to memory) and each block's launch
// (real_enc_fwd_ring_kernel) starts from the stored image: no geometry, no classification, no
// ranking, no lattice or position loads.  Accumulation, far block and projection are those of the
// pair kernel.
//
// Ring image of a unit (RIMG_WORDS 32-bit words): d2[RS], s[RS], bits[RS], header {near count, far
// count, smallest d2, -}.  Near records occupy slots 0 .. near-1 followed by 8 neutral records; far
// records occupy slots RS-1 downwards followed (below) by 4 neutral records.  (Keeping d2 alone and
// recomputing s and the bits in every launch makes the image three times smaller and the staging
// faster, but costs each launch 5% more instructions: 46.4 against 43.8 us on 128 crystals.)
#include "real_enc_pair_fwd.h"

namespace {

using namespace cf;
using namespace cfpair;

constexpr int RC = RIMG_CAP;                // translations of the cube, at most
constexpr int RS = RIMG_SLOTS;              // ring slots

// Gaussian argument s and record bits of a ring slot from its squared distance: 0xFFFF (a real
// translation) plus one bit per 16-bin tile whose window the translation reaches; s = 0 and no
// bits for a neutral slot (d2 = +inf).
template <int NT>
__device__ __forceinline__ int slot_record(const PairArgs &p, float d2, float &s)
{
    if (!(d2 < __builtin_inff())) {
        s = 0.f;
        return 0;
    }
    s = sqrt_hw(d2) * p.s_scale;
    const float xb = s * p.inv_bin_step - 1.0f;          // fractional bin coordinate
    int bits = 0xFFFF;
#pragma unroll
    for (int m = 0; m < NT; m++)
        if (xb >= (float)(16 * m) - p.window && xb <= (float)(16 * m + 15) + p.window) bits |= (0x10000 << m);
    return bits;
}

// ---------------------------------------------------------------- producer
// A wavefront per unit and trip, lane = translation (two chunks of 64); the wavefronts of the grid
// stride over the units, each with the next unit's lattice and offset already requested and the
// pair record of the one after (the two dependent loads are off the critical path).  weak_a2 is
// log2(e) times the weakest (closest to zero) exponent any block can have: a far translation is
// kept when weak_a2 (d2 - d2min) > -40, a superset of what any block's own exponents keep.
struct StageIds { int64_t e_ij, n; };

template <int NT>
__global__ __launch_bounds__(256) void ring_stage_kernel(PairArgs p_, float weak_a2, float *__restrict__ cache)
{
    const PairArgs p = with_live_units(p_);
    const int lane = threadIdx.x & 63;
    const int64_t waves = (int64_t)gridDim.x * (blockDim.x >> 6);
    const int64_t first = __builtin_amdgcn_readfirstlane((int)(blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6)));
    if (first >= p.U) return;
    auto ids_of = [&](int64_t u_) -> StageIds {
        u_ = u_ < p.U ? u_ : p.U - 1;
        return StageIds{p.pairs[u_ * PAIR_FIELDS], p.pairs[u_ * PAIR_FIELDS + 4]};
    };
    auto cell_of = [&](const StageIds &d) -> Cell {
        Cell c_;
        c_.rx = p.rpos[d.e_ij * 3 + 0];
        c_.ry = p.rpos[d.e_ij * 3 + 1];
        c_.rz = p.rpos[d.e_ij * 3 + 2];
#pragma unroll
        for (int x = 0; x < 9; x++) c_.t[x] = p.tvecs[d.n * 9 + x];
        return c_;
    };
    Cell cell = cell_of(ids_of(first));
    StageIds ids_next = ids_of(first + waves);
    for (int64_t u = first; u < p.U; u += waves) {
    const Cell cell_next = cell_of(ids_next);
    ids_next = ids_of(u + 2 * waves);
    BoxDims bx;
    bx.U1 = bx.U2 = bx.U3 = p.lattice_range;
    bx.S3 = bx.S2 = 2 * p.lattice_range + 1;
    bx.plane = bx.S2 * bx.S3;
    bx.T = bx.S2 * bx.plane;
    bx.inv_plane = 1.0f / (float)bx.plane;
    bx.inv_S3 = 1.0f / (float)bx.S3;
    const int T = bx.T;                    // <= RC (checked by the host)
    float d2c[2];
    float best = 1e10f;
#pragma unroll
    for (int ch = 0; ch < 2; ch++) {
        int n1, n2, n3;
        decode(bx, min(ch * WAVE + lane, T - 1), n1, n2, n3);
        d2c[ch] = dist2(cell, (float)n1, (float)n2, (float)n3);
        if (ch * WAVE + lane < T) best = fminf(best, d2c[ch]);
    }
    const float d2min = wave_min(best);
    float *ring_d2 = cache + u * RIMG_WORDS;
    float *ring_s = ring_d2 + RS;
    int *ring_bits = reinterpret_cast<int *>(ring_s + RS);
    int near_cnt = 0, far_cnt = 0;
#pragma unroll
    for (int ch = 0; ch < 2; ch++) {
        const bool valid = ch * WAVE + lane < T;
        const float d2 = d2c[ch];
        float s;
        const int bits = valid ? slot_record<NT>(p, d2, s) : 0;
        const int tiles = bits >> 16;
        const bool is_near = valid && tiles != 0;
        const bool is_far = valid && !is_near && weak_a2 * (d2 - d2min) > -40.0f;
        const unsigned long long far_mask = __ballot(is_far);
        const unsigned long long below = (1ull << lane) - 1ull;
        int pos = -1;
        int near_now;
        if (NT > 1) {
            // near translations ordered by the lowest tile they reach (8-bit counters per class)
            const int key8 = tiles ? 8 * (__builtin_ctz(tiles) >> (NT > 4 ? 1 : 0)) : 0;
            const int onehot = is_near ? (1 << key8) : 0;
            const int incl = wave_inclusive_scan_i(onehot);
            const int totals = __builtin_amdgcn_readlane(incl, 63);
            const int before = (totals << 8) + (totals << 16) + (totals << 24);
            if (is_near) pos = near_cnt + (((before + incl - onehot) >> key8) & 0xFF);
            near_now = (int)(((unsigned)totals * 0x01010101u) >> 24);
        } else {
            const unsigned long long near_mask = __ballot(is_near);
            if (is_near) pos = near_cnt + __popcll(near_mask & below);
            near_now = __popcll(near_mask);
        }
        if (is_far) pos = RS - 1 - (far_cnt + __popcll(far_mask & below));
        if (pos >= 0) {
            ring_d2[pos] = d2;
            ring_s[pos] = s;
            ring_bits[pos] = bits;
        }
        near_cnt += near_now;
        far_cnt += __popcll(far_mask);
    }
    // neutral records: 8 after the near block (last group + look-ahead), 4 below the far block
    if (lane < 12) {
        const int pos = lane < 8 ? near_cnt + lane : RS - far_cnt - 1 - (lane - 8);
        ring_d2[pos] = RIMG_NEUTRAL_D2;
        ring_s[pos] = 0.f;
        ring_bits[pos] = 0;
    }
    if (lane == 0) {
        int *hdr = reinterpret_cast<int *>(ring_d2 + 3 * RS);
        hdr[0] = near_cnt;
        hdr[1] = far_cnt;
        reinterpret_cast<float *>(hdr)[2] = d2min;
        hdr[3] = 0;
    }
    cell = cell_next;
    }
}

// ---------------------------------------------------------------- adaptive boxes: two sets of units
// Which units keep the fixed cube in all their active columns (the range rule of every (atom, head)
// of the unit yields lattice_range on the three axes): those are evaluated from the staged rings, on
// the bits the pair kernel's own shortcut for such units produces; the others go to the pair kernel.
// Three small launches turn the rule into two stably ordered lists of units with their counts on the
// device, so that each of the two kernels walks dense rounds of its own units, however many there
// are of either kind:
//   unit_keeps_kernel    a wavefront per 8 units, lane = (unit, head): the rule for its head of atoms i
//                        and j; a byte per unit and the number of keepers per chunk of PART_CHUNK units;
//   partition_kernel     every chunk places its keepers behind those of the chunks before it and its
//                        others behind all keepers (ranks by ballots, chunks in order: the same lists on
//                        every run); the first work-group leaves {keepers, others} in `counts`.
constexpr int PART_CHUNK = 1024;                  // units per work-group of partition_kernel
constexpr int KEEP_CHUNK = 128;                   // units per work-group of unit_keeps_kernel (8 per wavefront)

__global__ __launch_bounds__(PART_CHUNK) void unit_keeps_kernel(PairArgs p_, unsigned char *__restrict__ keeps,
                                                                int *__restrict__ chunk_keepers)
{
    __shared__ int keepers;
    const PairArgs p = with_live_units(p_);
    const int64_t first = (int64_t)blockIdx.x * KEEP_CHUNK;
    if (first >= p.U) return;
    if (threadIdx.x == 0) keepers = 0;
    __syncthreads();
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int w = lane >> 3, hh = lane & 7;
    const int64_t u = first + 8 * wave + w;
    const bool exists = u < p.U;
    bool keep = true;
    if (exists) {
        const int64_t *d = p.pairs + u * PAIR_FIELDS;
        const int64_t e_ij = d[0], e_ji = d[1], n = d[4];
        if (hh < p.H) {
            const float rvl[3] = {p.rvlen[n * 3 + 0], p.rvlen[n * 3 + 1], p.rvlen[n * 3 + 2]};
#pragma unroll
            for (int side = 0; side < 2; side++) {
                if (side == 1 && e_ji == e_ij) continue;         // a self pair has one direction
                int R1, R2, R3;
                range_rule(p.a_ik[d[2 + side] * p.H + hh], p.cutoff, rvl, p.lattice_range, p.min_range, R1, R2, R3);
                keep = keep && R1 == p.lattice_range && R2 == p.lattice_range && R3 == p.lattice_range;
            }
        }
    }
    const unsigned long long km = __ballot(keep);
    const bool unit_keeps = exists && ((km >> (8 * w)) & 0xFFull) == 0xFFull;
    if (exists && hh == 0) keeps[u] = unit_keeps ? 1 : 0;
    const int mine = __popcll(__ballot(unit_keeps && hh == 0));
    if (lane == 0 && mine) atomicAdd(&keepers, mine);
    __syncthreads();
    if (threadIdx.x == 0) chunk_keepers[blockIdx.x] = keepers;
}

__global__ __launch_bounds__(PART_CHUNK) void partition_kernel(const unsigned char *__restrict__ keeps,
                                                               const int *__restrict__ chunk_keepers, int64_t U_cap,
                                                               const int64_t *live_U, int *__restrict__ order,
                                                               int64_t *__restrict__ counts)
{
    __shared__ int part[PART_CHUNK / WAVE];
    __shared__ int wave_keep[PART_CHUNK / WAVE];
    __shared__ int before_total[2];
    const int64_t U = live_count(live_U, U_cap);
    const int64_t first = (int64_t)blockIdx.x * PART_CHUNK;
    if (blockIdx.x == 0 && U == 0 && threadIdx.x == 0) counts[0] = counts[1] = counts[2] = 0;
    if (first >= U) return;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    // keepers in the chunks before this one, and in all chunks (counted per KEEP_CHUNK units)
    constexpr int SUB = PART_CHUNK / KEEP_CHUNK;
    const int subs = (int)((U + KEEP_CHUNK - 1) / KEEP_CHUNK);
    int before = 0, total = 0;
    for (int g = threadIdx.x; g < subs; g += PART_CHUNK) {
        const int c = chunk_keepers[g];
        total += c;
        if (g < (int)blockIdx.x * SUB) before += c;
    }
    for (int off = 32; off >= 1; off >>= 1) {
        before += __shfl_xor(before, off, WAVE);
        total += __shfl_xor(total, off, WAVE);
    }
    if (lane == 0) {
        part[wave] = before;
        wave_keep[wave] = total;
    }
    __syncthreads();
    if (threadIdx.x == 0) {
        int b = 0, t = 0;
        for (int x = 0; x < PART_CHUNK / WAVE; x++) {
            b += part[x];
            t += wave_keep[x];
        }
        before_total[0] = b;
        before_total[1] = t;
        if (blockIdx.x == 0) {
            counts[0] = t;
            counts[1] = U - t;
            counts[2] = 0;                   // scheduling words of the launch that follows
        }
    }
    __syncthreads();
    const int keep_before = before_total[0], keep_total = before_total[1];
    const int64_t u = first + threadIdx.x;
    const bool valid = u < U;
    const bool keep = valid && keeps[u] != 0;
    const unsigned long long km = __ballot(keep), vm = __ballot(valid);
    const unsigned long long below = (1ull << lane) - 1ull;
    __syncthreads();
    if (lane == 0) wave_keep[wave] = __popcll(km);
    __syncthreads();
    if (valid) {
        int keep_in_chunk_before = 0;
        for (int x = 0; x < wave; x++) keep_in_chunk_before += wave_keep[x];
        const int rank_keep = keep_in_chunk_before + __popcll(km & below);
        const int in_chunk = wave * WAVE + __popcll(vm & below);         // units before this one in the chunk
        const int pos = keep ? keep_before + rank_keep
                             : keep_total + (int)(first - keep_before) + (in_chunk - rank_keep);
        order[pos] = (int)u;
    }
}

// ---------------------------------------------------------------- consumer
// Work-group of 8 wavefronts, one unit per wavefront and round, as in the pair kernel.  The image
// of the next round's unit (its address follows from the round number alone) is requested a round
// ahead into registers and copied to the wavefront's LDS ring at the top of its round.
// LDS: per wave 3 x RS words, exchange buffer 4 NT x XPLANE, 8 x 2 edge ids, 8 x 16 reciprocals.
// With p.order the slots of the rounds hold the units the order lists (adaptive boxes: those that keep
// the cube).
template <int NT, int DT>
__device__ __forceinline__ void real_enc_fwd_ring_body(const PairArgs &p, const float *__restrict__ cache,
                                                       const int block_id, const int grid_size)
{
    extern __shared__ __align__(16) float lds[];
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int q = lane >> 4;
    const int c = lane & 15;
    const int H = p.H, K = p.K, D = p.D;
    const int64_t *__restrict__ g_pairs = p.pairs;
    const float *__restrict__ g_a = p.a_ik;
    float *ring_d2 = lds + wave * (3 * RS);
    float *ring_s = ring_d2 + RS;
    int *ring_bits = reinterpret_cast<int *>(ring_s + RS);
    float *Sbuf = lds + WPB * 3 * RS;                                       // [4 NT][XPLANE]
    int64_t *meta = reinterpret_cast<int64_t *>(Sbuf + 4 * NT * XPLANE);    // [WPB][2]
    float *invbuf = reinterpret_cast<float *>(meta + WPB * 2);              // [WPB][16]

    float ck[NT];
#pragma unroll
    for (int m = 0; m < NT; m++) ck[m] = p.bin_step * (float)(16 * m + c + 1);
    float Wa[DT][4 * NT];
    int wa_hg = -1;

    const int rounds_per_hg = (int)((p.U + WPB - 1) / WPB);
    const int rounds = rounds_per_hg * p.head_groups;
    const int stride = grid_size;
    // unit of this wavefront in round rd_ (0 when the round or the slot does not exist: loads stay valid)
    auto unit_of = [&](int rd_, const RoundPos &rp) -> int64_t {
        const int64_t slot = (int64_t)rp.r * WPB + wave;
        if (!(rd_ < rounds && slot < p.U)) return 0;
        return p.order ? (int64_t)ordered_unit(p.order, (int)slot) : slot;
    };
    auto load_a = [&](const UnitIds &d, const RoundPos &rp) -> float {
        const unsigned h_ = (unsigned)min(rp.hg * 8 + (c & 7), H - 1);
        return g_a[((c < 8) ? (unsigned)d.i : (unsigned)d.j) * (unsigned)H + h_];
    };
    using Image = RingImage;
    auto load_image = [&](int64_t u_) -> Image { return load_ring_image(cache, u_, lane); };

    // rounds of this work-group: block_id, + grid, + 2 grid, ...
    int rd = block_id, rd_next = rd + stride, rd_next2 = rd + 2 * stride;
    RoundPos pos = round_pos(rd, rounds_per_hg, p.head_groups);
    RoundPos pos_next = round_pos(rd_next, rounds_per_hg, p.head_groups);
    int64_t u = unit_of(rd, pos), u_next = unit_of(rd_next, pos_next);
    UnitIds ids = unit_ids(load_unit_ids(g_pairs, u, lane));
    float a_cur = load_a(ids, pos);
    Image img = load_image(u);
    UnitIds ids_next = unit_ids(load_unit_ids(g_pairs, u_next, lane));

    while (rd < rounds) {
        const int hg = pos.hg;
        const bool unit_on = (int64_t)pos.r * WPB + wave < p.U;
        const RoundPos pos_next2 = round_pos(rd_next2, rounds_per_hg, p.head_groups);
        const int64_t u_next2 = unit_of(rd_next2, pos_next2);
        // this round's image into the ring (the previous round's readers of the ring are done:
        // same wavefront, and the epilogue's barriers lie in between)
        const int near_cnt = unit_on ? __builtin_amdgcn_readlane(img.hdr, 0) : 0;
        const int far_cnt = unit_on ? __builtin_amdgcn_readlane(img.hdr, 1) : 0;
        const float d2min = __int_as_float(__builtin_amdgcn_readlane(img.hdr, 2));
        store_ring_image(img, ring_d2, ring_s, ring_bits, lane);
        if (near_cnt + 8 > 2 * WAVE || far_cnt > 0)              // slots 128 .. 143 (wave-uniform, rare)
            copy_ring_tail(cache, u, ring_d2, ring_s, ring_bits, lane);
        if (!unit_on && lane < 8) {          // no unit: an empty near block (neutral records)
            ring_d2[lane] = RIMG_NEUTRAL_D2;
            ring_s[lane] = 0.f;
            ring_bits[lane] = 0;
        }
        // loads for the coming rounds
        const Image img_next = load_image(u_next);
        const float a_next = load_a(ids_next, pos_next);
        const int64_t dv_next2 = load_unit_ids(g_pairs, u_next2, lane);
        if (hg != wa_hg) {
            const int hw = hg * 8 + wave;
            if (hw < H && K == 16 * NT && D == 16 * DT) {
#pragma unroll
                for (int dt = 0; dt < DT; dt++) {
                    const float *wrow = p.W + ((int64_t)hw * D + 16 * dt + c) * K + 4 * q;
#pragma unroll
                    for (int t4 = 0; t4 < NT; t4++) {
                        const float4_t w4 = *reinterpret_cast<const float4_t *>(wrow + 16 * t4);
#pragma unroll
                        for (int r = 0; r < 4; r++) Wa[dt][4 * t4 + r] = w4[r];
                    }
                }
            } else {
                // (taken when the head group changes: its masks and offsets are worked out here,
                // not kept in registers across the rounds)
                int qq = q, cc = c;
                asm volatile("" : "+v"(qq), "+v"(cc));
#pragma unroll
                for (int dt = 0; dt < DT; dt++)
#pragma unroll
                    for (int s = 0; s < 4 * NT; s++) {
                        const int d = 16 * dt + cc, k = proj_bin(s, qq);
                        Wa[dt][s] = (hw < H && d < D && k < K) ? p.W[((int64_t)hw * D + d) * K + k] : 0.f;
                    }
            }
            wa_hg = hg;
        }
        const int64_t e_ij = ids.e_ij, e_ji = ids.e_ji;
        const int h = hg * 8 + (c & 7);
        const bool col_on = unit_on && h < H && (c < 8 || e_ji != e_ij);
        const float a = col_on ? a_cur : -1.0f;
        const float a2 = a * LOG2E;

        float4_t acc[NT];
#pragma unroll
        for (int m = 0; m < NT; m++) acc[m] = float4_t{0.f, 0.f, 0.f, 0.f};
        float sum = 0.f;
        wave_mem_sync();
        // ---- accumulation over the near block: 4 translations per MFMA
        {
            // two groups per trip, each with its own registers for the prefetched records (no
            // copies from "next" to "current"); records beyond the last group are the neutral padding
            const int groups = (near_cnt + 3) >> 2;
            struct Rec { float d2, s; int bits; };
            auto fetch = [&](int g_) -> Rec {
                const int slot = 4 * g_ + q;
                return Rec{ring_d2[slot], ring_s[slot], ring_bits[slot]};
            };
            auto group = [&](const Rec &rec) {
                // (padding records: weight 0 through their d2; columns that are switched off run
                // with a = -1 and finite garbage that is never stored)
                const float w = exp2_hw(a2 * (rec.d2 - d2min));
                sum += w;
                const int reach = group_reach(rec.bits);
#pragma unroll
                for (int m = 0; m < NT; m++) {
                    if (reach & (0x10000 << m)) {                             // wave-uniform
                        float b = ck[m] - rec.s;
                        float gm = exp2_hw(-(b * b));
                        acc[m] = __builtin_amdgcn_mfma_f32_16x16x4f32(gm, w, acc[m], 0, 0, 0);
                    }
                }
            };
            Rec ra = fetch(0);
            for (int g = 0; g < groups; g += 2) {
                const Rec rb = fetch(g + 1);
                group(ra);
                if (g + 1 < groups) {
                    ra = fetch(g + 2);
                    group(rb);
                }
            }
        }
        // ---- the far block only feeds the column sums
        {
            const int groups = (far_cnt + 3) >> 2;
            for (int g = 0; g < groups; g++) {
                const int slot = RS - 4 * (g + 1) + q;
                sum += exp2_hw(a2 * (ring_d2[slot] - d2min));
            }
        }
        wave_mem_sync();
        const UnitIds ids_next2 = unit_ids(dv_next2);
        sum = rows_sum(sum);
        const float inv = __builtin_amdgcn_rcpf(sum);
        // ((edge, head) rows are 32-bit: the launcher refuses E H >= 2^32)
        const unsigned e_col = (c < 8) ? (unsigned)e_ij : (unsigned)e_ji;
        if (col_on && q == 0) p.z[e_col * (unsigned)H + (unsigned)h] = log2_hw(sum) * LN2 + d2min * a;

        // epilogue: park the column sums, project per head (see the pair kernel)
        float *col = Sbuf + xch_base(q, c & 7, wave, c >> 3);
#pragma unroll
        for (int m = 0; m < NT; m++)
#pragma unroll
            for (int r = 0; r < 4; r++) col[(4 * m + r) * XPLANE] = acc[m][r];
        if (q == 0) invbuf[wave * 16 + c] = inv;
        if (lane == 0) {
            meta[2 * wave + 0] = unit_on ? e_ij : -1;
            meta[2 * wave + 1] = (unit_on && e_ji != e_ij) ? e_ji : -1;
        }
        __syncthreads();
        {
            const int hw = hg * 8 + wave;
            const int j = c, unit_j = j & 7, dir_j = j >> 3;
            const float *src = Sbuf + xch_base(q, wave, unit_j, dir_j);
            float4_t out[DT];
#pragma unroll
            for (int dt = 0; dt < DT; dt++) out[dt] = float4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int t4 = 0; t4 < NT; t4++) {
                float sb[4];
#pragma unroll
                for (int r = 0; r < 4; r++) sb[r] = src[(4 * t4 + r) * XPLANE];
#pragma unroll
                for (int r = 0; r < 4; r++)
#pragma unroll
                    for (int dt = 0; dt < DT; dt++)
                        out[dt] = __builtin_amdgcn_mfma_f32_16x16x4f32(Wa[dt][4 * t4 + r], sb[r], out[dt], 0, 0, 0);
            }
            const int64_t e_out = meta[2 * unit_j + dir_j];
            const float inv_j = invbuf[unit_j * 16 + dir_j * 8 + wave];
#pragma unroll
            for (int dt = 0; dt < DT; dt++) out[dt] *= inv_j;
            if (e_out >= 0 && hw < H) {
#pragma unroll
                for (int dt = 0; dt < DT; dt++) {
                    const int dbase = 16 * dt + 4 * q;
                    float *dst = p.v + ((uint64_t)((unsigned)e_out * (unsigned)H + (unsigned)hw) * (unsigned)D +
                                        (unsigned)dbase);
                    if (dbase + 3 < D) {
                        *reinterpret_cast<float4_t *>(dst) = out[dt];
                    } else {
#pragma unroll
                        for (int r = 0; r < 3; r++)
                            if (dbase + r < D) dst[r] = out[dt][r];
                    }
                }
            }
        }
        __syncthreads();
        ids = ids_next;
        a_cur = a_next;
        img = img_next;
        ids_next = ids_next2;
        pos = pos_next;
        pos_next = pos_next2;
        u = u_next;
        u_next = u_next2;
        rd = rd_next;
        rd_next = rd_next2;
        rd_next2 += stride;
    }
}

template <int NT, int DT>
__global__ __launch_bounds__(512, 4) void real_enc_fwd_ring_kernel(PairArgs p_, const float *__restrict__ cache)
{
    const PairArgs p = with_live_units(p_);
    if (p.U == 0) return;          // (an empty list: not even the descriptor of unit 0 may be read)
    real_enc_fwd_ring_body<NT, DT>(p, cache, (int)blockIdx.x, (int)gridDim.x);
}

// Adaptive boxes in one launch: the units that keep the cube (first list of the order) run the ring
// body, the others (second list) the pair kernel's body, at the same time on disjoint sets of
// work-groups.  How the work-groups are split follows the two counts, which only the device knows:
// every work-group reads them and takes the same decision, places in proportion to the work of the two
// lists (a unit of the second list priced at `pair_cost` units of the first), at most one work-group
// per round, at least one per list that is not empty.
template <int NT, int DT>
__global__ __launch_bounds__(512, 4) void real_enc_fwd_two_role_kernel(PairArgs p_ring, PairArgs p_pair,
                                                                       const float *__restrict__ cache,
                                                                       float pair_cost)
{
    PairArgs pr = with_live_units(p_ring), pp = with_live_units(p_pair);
    if (pr.U < pp.U) {
        // Fewer than half of the units keep the cube: the split costs more than the rings save (measured
        // on 256 crystals with r0 = 3 A, 36 % keepers: 515 against 487 us), so the pair body takes all of
        // them -- the order lists every unit, the first list in front of the second.
        pp.order = p_pair.order;
        pp.U += pr.U;
        pr.U = 0;
    }
    const int grid = (int)gridDim.x;
    const int64_t rounds_ring = (pr.U + WPB - 1) / WPB, rounds_pair = (pp.U + WPB - 1) / WPB;
    int pair_blocks = 0;
    if (pp.U > 0) {
        const float wp = (float)pp.U * pair_cost, wr = (float)pr.U;
        pair_blocks = (int)((float)grid * (wp / (wp + wr)) + 0.5f);
        pair_blocks = max(pair_blocks, 1);
        if (pr.U > 0) pair_blocks = min(pair_blocks, grid - 1);
        if ((int64_t)pair_blocks > rounds_pair) pair_blocks = (int)rounds_pair;
    }
    pair_blocks = __builtin_amdgcn_readfirstlane(pair_blocks);
    // (tickets for the pair body's rounds only where a work-group has many of them, as in its own launch)
    if (rounds_pair < 16 * (int64_t)pair_blocks) pp.sched = nullptr;
    if ((int)blockIdx.x < pair_blocks) {
        // (p_pair is the kernel's second argument, behind p_ring in the kernel-argument segment)
        static_assert(sizeof(PairArgs) % 8 == 0, "the second argument follows the first without padding");
        const PairArgsSeg seg = (PairArgsSeg)__builtin_amdgcn_kernarg_segment_ptr() + 1;
        real_enc_fwd_pair_body<NT, false, PROJ_SHARED, DT, false>(pp, seg, (int)blockIdx.x, pair_blocks);
    } else if (pr.U > 0) {
        int ring_blocks = grid - pair_blocks;
        if ((int64_t)ring_blocks > rounds_ring) ring_blocks = (int)rounds_ring;
        const int b = (int)blockIdx.x - pair_blocks;
        if (b < ring_blocks) real_enc_fwd_ring_body<NT, DT>(pr, cache, b, ring_blocks);
    }
}

}  // namespace

namespace cf {

int64_t real_enc_ring_words() { return RIMG_WORDS; }

// Stages every unit's translations into `cache` (U x RIMG_WORDS floats).  Fixed cube of at most 128
// translations, K in 1..128.  CF_ERR_UNSUPPORTED (no error text) otherwise.
int launch_ring_stage(const float *rpos, const float *tvecs, const int64_t *pairs, int64_t U, int64_t K,
                      float bin_step, float s_scale, int lattice_range, float weak_a, float *cache, hipStream_t st)
{
    const int64_t cube = (int64_t)(2 * lattice_range + 1) * (2 * lattice_range + 1) * (2 * lattice_range + 1);
    if (K < 1 || K > 128 || cube > RC) return CF_ERR_UNSUPPORTED;
    if (U == 0) return CF_OK;
    PairArgs p{};
    p.rpos = rpos; p.tvecs = tvecs; p.pairs = pairs; p.U = U; p.K = (int)K;
    p.lattice_range = lattice_range;
    p.bin_step = bin_step; p.s_scale = s_scale; p.inv_bin_step = 1.0f / bin_step;
    p.window = sqrtf(40.0f) / bin_step;
    p.live_U = live_units(U);
    const float weak_a2 = weak_a * LOG2E;
    const int NT = K <= 16 ? 1 : K <= 32 ? 2 : K <= 64 ? 4 : 8;
    int64_t blocks64 = (U + 3) / 4;
    const int64_t cap = persistent_grid_cap(8);
    if (blocks64 > cap) blocks64 = cap;
    const int blocks = (int)blocks64;
    switch (NT) {
        case 1: ring_stage_kernel<1><<<blocks, 256, 0, st>>>(p, weak_a2, cache); break;
        case 2: ring_stage_kernel<2><<<blocks, 256, 0, st>>>(p, weak_a2, cache); break;
        case 4: ring_stage_kernel<4><<<blocks, 256, 0, st>>>(p, weak_a2, cache); break;
        default: ring_stage_kernel<8><<<blocks, 256, 0, st>>>(p, weak_a2, cache); break;
    }
    return CF_OK;
}

// Adaptive boxes from staged rings: the scratch holds {keepers, others, scheduling words} (4 int64), the order of the
// units (U ints, rounded up to a multiple of 2), the keepers per chunk and a byte per unit.
int64_t unit_partition_bytes(int64_t U)
{
    if (U <= 0) return 0;
    const int64_t subs = (U + KEEP_CHUNK - 1) / KEEP_CHUNK;
    return 32 + ((U + 1) / 2) * 8 + ((subs + 1) / 2) * 8 + ((U + 7) / 8) * 8;
}

// The two lists of units (see unit_keeps_kernel).  On return (device side) counts[0] / counts[1] hold
// the numbers of units that keep the cube / do not, order[0 .. counts[0]) the first and
// order[counts[0] .. U) the second kind.  One head group (H <= 8) only.
int launch_unit_partition(const float *a_ik, const float *rvlen, const int64_t *pairs, int64_t U, int64_t N, int64_t H,
                          float cutoff, int lattice_range, int min_range, void *scratch, int64_t **counts_out,
                          int **order_out, hipStream_t st)
{
    if (H > 8 || U < 1 || U >= (1ll << 31)) return CF_ERR_UNSUPPORTED;
    int64_t *counts = (int64_t *)scratch;
    int *order = (int *)(counts + 4);
    int *chunk_keepers = order + ((U + 1) / 2) * 2;
    const int64_t chunks = (U + PART_CHUNK - 1) / PART_CHUNK, subs = (U + KEEP_CHUNK - 1) / KEEP_CHUNK;
    unsigned char *keeps = (unsigned char *)(chunk_keepers + ((subs + 1) / 2) * 2);
    PairArgs p{};
    p.a_ik = a_ik; p.rvlen = rvlen; p.pairs = pairs;
    p.N = N; p.U = U; p.H = (int)H;
    p.head_groups = 1;
    p.cutoff = cutoff; p.lattice_range = lattice_range; p.min_range = min_range;
    p.live_U = live_units(U);
    unit_keeps_kernel<<<(int)subs, PART_CHUNK, 0, st>>>(p, keeps, chunk_keepers);
    partition_kernel<<<(int)chunks, PART_CHUNK, 0, st>>>(keeps, chunk_keepers, U, p.live_U, order, counts);
    *counts_out = counts;
    *order_out = order;
    return CF_OK;
}

// Forward from staged rings (shared projection, D <= 32).  CF_ERR_UNSUPPORTED otherwise.
// With an order only the first *n_units units it lists are evaluated (n_units on the device).
int launch_real_enc_fwd_rings(const float *a_ik, const int64_t *pairs, int64_t U, int64_t N, int64_t H, int64_t E,
                              int64_t K, int64_t D, float bin_step, float s_scale, const float *W,
                              const float *cache, const int *order, const int64_t *n_units,
                              float *z, float *v, hipStream_t st)
{
    if (K < 1 || K > 128 || !W || D < 1 || D > 32) return CF_ERR_UNSUPPORTED;
    if (E * H >= (1ll << 32) || N * H >= (1ll << 32)) return CF_ERR_UNSUPPORTED;      // 32-bit rows in the kernel
    PairArgs p{};
    p.a_ik = a_ik; p.pairs = pairs; p.W = W; p.z = z; p.v = v;
    p.N = N; p.E = E; p.U = U; p.W_num = 1;
    p.H = (int)H; p.K = (int)K; p.D = (int)D;
    p.head_groups = (int)((H + 7) / 8);
    p.bin_step = bin_step; p.s_scale = s_scale; p.inv_bin_step = 1.0f / bin_step;
    p.window = sqrtf(40.0f) / bin_step;
    p.live_U = order ? n_units : live_units(U);
    p.order = order;
    const int NT = K <= 16 ? 1 : K <= 32 ? 2 : K <= 64 ? 4 : 8;
    const int DT = D > 16 ? 2 : 1;
    size_t lds = sizeof(float) * ((size_t)WPB * 3 * RS + (size_t)4 * NT * XPLANE + WPB * 16) +
                 sizeof(int64_t) * WPB * 2 + 8;
    const int64_t rounds = ((U + WPB - 1) / WPB) * p.head_groups;
    if (rounds >= (1ll << 30)) return CF_ERR_UNSUPPORTED;
    int64_t blocks = rounds;
    const int64_t cap = persistent_grid_cap(2);
    if (blocks > cap) blocks = cap;
    if (blocks < 1) return CF_OK;
#define CF_RING(NTV, DTV) real_enc_fwd_ring_kernel<NTV, DTV><<<(int)blocks, WPB * WAVE, lds, st>>>(p, cache)
#define CF_RING_NT(NTV) do { if (DT == 1) CF_RING(NTV, 1); else CF_RING(NTV, 2); } while (0)
    switch (NT) {
        case 1: CF_RING_NT(1); break;
        case 2: CF_RING_NT(2); break;
        case 4: CF_RING_NT(4); break;
        default: CF_RING_NT(8); break;
    }
#undef CF_RING_NT
#undef CF_RING
    return CF_OK;
}

// Adaptive boxes: both lists of launch_unit_partition in one launch (real_enc_fwd_two_role_kernel).
int launch_real_enc_fwd_two_role(const float *a_ik, const float *rpos, const float *tvecs, const int64_t *batch,
                                 const int64_t *edges, const int64_t *pairs, int64_t U, int64_t N, int64_t H,
                                 int64_t E, int64_t K, int64_t D, float bin_step, float s_scale, const float *W,
                                 const float *rvlen, float cutoff, int lattice_range, int min_range,
                                 const float *cache, const int *order, const int64_t *counts, float *z, float *v,
                                 hipStream_t st)
{
    if (K < 1 || K > 128 || !W || D < 1 || D > 32 || cutoff == 0.0f || !order || !counts || H > 8)
        return CF_ERR_UNSUPPORTED;
    if (E * H >= (1ll << 32) || N * H >= (1ll << 32)) return CF_ERR_UNSUPPORTED;      // 32-bit rows in the ring body
    PairArgs pp{};
    pp.a_ik = a_ik; pp.rpos = rpos; pp.tvecs = tvecs; pp.batch = batch; pp.edges = edges; pp.pairs = pairs;
    pp.W = W; pp.rvlen = rvlen; pp.z = z; pp.v = v; pp.sched = nullptr;
    pp.N = N; pp.E = E; pp.U = U; pp.W_num = 1;
    pp.H = (int)H; pp.K = (int)K; pp.D = (int)D;
    pp.head_groups = 1;
    pp.cutoff = cutoff; pp.lattice_range = lattice_range; pp.min_range = min_range;
    pp.bin_step = bin_step; pp.s_scale = s_scale; pp.inv_bin_step = 1.0f / bin_step;
    pp.window = sqrtf(40.0f) / bin_step;
    pp.order = order; pp.order_first = counts; pp.live_U = counts + 1;              // the units that leave the cube
    pp.sched = reinterpret_cast<unsigned int *>(const_cast<int64_t *>(counts) + 2); // (zeroed with the counts)
    PairArgs pr = pp;                                                               // the units that keep it
    pr.rpos = nullptr; pr.tvecs = nullptr; pr.batch = nullptr; pr.edges = nullptr; pr.rvlen = nullptr;
    pr.cutoff = 0.f; pr.order_first = nullptr; pr.live_U = counts; pr.sched = nullptr;
    const int NT = K <= 16 ? 1 : K <= 32 ? 2 : K <= 64 ? 4 : 8;
    const int DT = D > 16 ? 2 : 1;
    const size_t shared_proj = sizeof(float) * ((size_t)4 * NT * XPLANE + WPB * 16) + sizeof(int64_t) * WPB * 2 + 8;
    const size_t lds_ring = sizeof(float) * (size_t)WPB * 3 * RS + shared_proj;
    const size_t lds_pair = sizeof(float) * (size_t)WPB * 3 * (RING_CAP + 16) + shared_proj;
    const size_t lds = lds_ring > lds_pair ? lds_ring : lds_pair;
    const int64_t rounds = (U + WPB - 1) / WPB;
    if (rounds >= (1ll << 30)) return CF_ERR_UNSUPPORTED;
    if (rounds < 1) return CF_OK;
    const int64_t cap = persistent_grid_cap(2);
    const int grid = (int)(rounds < cap ? rounds : cap);
    // a unit that leaves the cube costs about this many units that keep it (its box holds more
    // translations, and they are staged in the launch)
    // (swept on 128 and 256 crystals: 1.5 / 2 / 2.5 / 3 / 4 give 0.506 / 0.461 / 0.431 / 0.420 / 0.414 ms per
    // forward of the default model and 3.45 / 3.17 / 3.20 / 3.19 / 3.45 ms of the seven-block one)
    const float pair_cost = 3.0f;
#define CF_TWO(NTV, DTV) \
    real_enc_fwd_two_role_kernel<NTV, DTV><<<grid, WPB * WAVE, lds, st>>>(pr, pp, cache, pair_cost)
#define CF_TWO_NT(NTV) do { if (DT == 1) CF_TWO(NTV, 1); else CF_TWO(NTV, 2); } while (0)
    switch (NT) {
        case 1: CF_TWO_NT(1); break;
        case 2: CF_TWO_NT(2); break;
        case 4: CF_TWO_NT(4); break;
        default: CF_TWO_NT(8); break;
    }
#undef CF_TWO_NT
#undef CF_TWO
    return CF_OK;
}

}  // namespace cf

namespace {
// Gaussian argument per bin index and per unit of distance, as the other encoding entry points derive them
void bin_scales(int64_t K, double dist_max, double wscale, float &bin_step, float &s_scale)
{
    const float reci_ws_sqrt2 = 1.0f / ((float)wscale * sqrtf(2.0f));
    const float mu0 = (float)dist_max / (float)K;
    bin_step = reci_ws_sqrt2 * sqrtf(cf::LOG2E);
    s_scale = bin_step / mu0;
}
}  // namespace

extern "C" int64_t cf_real_enc_ring_bytes(int64_t U)
{
    return U <= 0 ? 0 : U * RIMG_WORDS * (int64_t)sizeof(float);
}

extern "C" int cf_real_enc_ring_stage(const float *rpos_ij_e, const float *tvecs_n, const int64_t *pairs_u, int64_t U,
                                      int64_t K, double dist_max, double wscale, int lattice_range,
                                      double weakest_exponent, void *rings, void *stream)
{
    CF_REQUIRE(U >= 0, CF_ERR_INVALID_ARGUMENT, "cf_real_enc_ring_stage: negative U");
    if (U == 0) return CF_OK;
    CF_REQUIRE(rpos_ij_e && tvecs_n && pairs_u && rings, CF_ERR_INVALID_ARGUMENT, "cf_real_enc_ring_stage: null pointer");
    CF_REQUIRE(K >= 1 && K <= 128 && dist_max > 0 && wscale > 0, CF_ERR_INVALID_ARGUMENT,
               "cf_real_enc_ring_stage: needs 1 <= K <= 128 and positive dist_max, wscale");
    CF_REQUIRE(weakest_exponent <= 0, CF_ERR_INVALID_ARGUMENT, "cf_real_enc_ring_stage: weakest_exponent must be <= 0");
    CF_REQUIRE(lattice_range >= 0 && (2 * lattice_range + 1) * (2 * lattice_range + 1) * (2 * lattice_range + 1) <= RC,
               CF_ERR_UNSUPPORTED, "cf_real_enc_ring_stage: the fixed cube of lattice_range %d has more than %d translations",
               lattice_range, RC);
    float bin_step, s_scale;
    bin_scales(K, dist_max, wscale, bin_step, s_scale);
    int rc = cf::launch_ring_stage(rpos_ij_e, tvecs_n, pairs_u, U, K, bin_step, s_scale, lattice_range,
                                   (float)weakest_exponent, (float *)rings, (hipStream_t)stream);
    CF_REQUIRE(rc == CF_OK, rc, "cf_real_enc_ring_stage: unsupported shape");
    CF_CHECK_LAUNCH("cf_real_enc_ring_stage");
    return CF_OK;
}

extern "C" int64_t cf_real_enc_flag_bytes(int64_t U, int64_t H)
{
    if (U < 0 || H < 1) return 0;
    return cf::unit_partition_bytes(U);
}

extern "C" int cf_real_enc_fwd_rings(const float *a_ik, const float *rpos_ij_e, const float *tvecs_n,
                                     const int64_t *batch_i, const int64_t *edge_ij_e, const int64_t *pairs_u,
                                     int64_t U, int64_t N, int64_t H, int64_t E, int64_t K, int64_t D,
                                     double dist_max, double wscale, const float *W_k, const float *rvlen_n,
                                     double cutoff_radius, int lattice_range, int minimum_range,
                                     const void *rings, void *flags, int64_t flag_bytes, float *z_ek,
                                     float *v_ekd, void *stream)
{
    CF_REQUIRE(N >= 0 && E >= 0 && U >= 0, CF_ERR_INVALID_ARGUMENT, "cf_real_enc_fwd_rings: negative size");
    CF_REQUIRE(H == 1 || H == 2 || H == 4 || H == 8 || H == 16, CF_ERR_UNSUPPORTED,
               "cf_real_enc_fwd_rings: head count %lld not supported (1,2,4,8,16)", (long long)H);
    CF_REQUIRE(2 * U == E + N, CF_ERR_INVALID_ARGUMENT,
               "cf_real_enc_fwd_rings: a pair list over dense crystal blocks has (E+N)/2 = %lld entries, got %lld",
               (long long)((E + N) / 2), (long long)U);
    if (E == 0) return CF_OK;
    CF_REQUIRE(a_ik && pairs_u && W_k && rings && z_ek && v_ekd, CF_ERR_INVALID_ARGUMENT,
               "cf_real_enc_fwd_rings: null pointer");
    CF_REQUIRE(K >= 1 && K <= 128 && D >= 1 && D <= 32 && dist_max > 0 && wscale > 0, CF_ERR_UNSUPPORTED,
               "cf_real_enc_fwd_rings: needs 1 <= K <= 128, 1 <= D <= 32");
    const int edge = 2 * lattice_range + 1;
    CF_REQUIRE(lattice_range >= 0 && edge * edge * edge <= RC, CF_ERR_UNSUPPORTED,
               "cf_real_enc_fwd_rings: lattice_range %d outside what the rings hold", lattice_range);
    float bin_step, s_scale;
    bin_scales(K, dist_max, wscale, bin_step, s_scale);
    hipStream_t st = (hipStream_t)stream;
    const float cutoff = rvlen_n ? (float)cutoff_radius : 0.0f;
    if (cutoff == 0.0f) {
        int rc = cf::launch_real_enc_fwd_rings(a_ik, pairs_u, U, N, H, E, K, D, bin_step, s_scale, W_k,
                                               (const float *)rings, nullptr, nullptr, z_ek, v_ekd, st);
        CF_REQUIRE(rc == CF_OK, rc, "cf_real_enc_fwd_rings: unsupported shape");
        CF_CHECK_LAUNCH("cf_real_enc_fwd_rings");
        return CF_OK;
    }
    // Adaptive boxes: the units whose columns all keep the cube from the rings, the rest by the
    // pair kernel; both write their own edges of z and v.
    CF_REQUIRE(minimum_range >= 0 && minimum_range <= MAX_RANGE, CF_ERR_INVALID_ARGUMENT,
               "cf_real_enc_fwd_rings: minimum_range %d outside 0..%d", minimum_range, MAX_RANGE);
    CF_REQUIRE(rpos_ij_e && tvecs_n && batch_i && edge_ij_e, CF_ERR_INVALID_ARGUMENT,
               "cf_real_enc_fwd_rings: adaptive boxes need rpos_ij_e, tvecs_n, batch_i and edge_ij_e");
    if (H > 8) {
        // (the two lists are per head group; with more than one, every unit goes to the pair kernel)
        int rc = cf::launch_real_enc_fwd_pairs(a_ik, rpos_ij_e, tvecs_n, batch_i, edge_ij_e, pairs_u, U, N, H, E, K, D,
                                               bin_step, s_scale, W_k, 1, rvlen_n, cutoff, lattice_range, minimum_range,
                                               nullptr, nullptr, nullptr, z_ek, v_ekd, st);
        CF_REQUIRE(rc == CF_OK, rc, "cf_real_enc_fwd_rings: unsupported shape");
        CF_CHECK_LAUNCH("cf_real_enc_fwd_rings (adaptive boxes)");
        return CF_OK;
    }
    CF_REQUIRE(flags && flag_bytes >= cf_real_enc_flag_bytes(U, H), CF_ERR_INVALID_ARGUMENT,
               "cf_real_enc_fwd_rings: adaptive boxes need %lld bytes of flags, %lld given",
               (long long)cf_real_enc_flag_bytes(U, H), (long long)flag_bytes);
    // Two lists of units, then one launch with a role for each: from the rings the units that keep the
    // cube, the pair kernel's body for the others.  Either list may be empty or hold everything; the
    // counts stay on the device.
    int64_t *counts = nullptr;
    int *order = nullptr;
    int rc = cf::launch_unit_partition(a_ik, rvlen_n, pairs_u, U, N, H, cutoff, lattice_range, minimum_range, flags,
                                       &counts, &order, st);
    CF_REQUIRE(rc == CF_OK, rc, "cf_real_enc_fwd_rings: unsupported size");
    rc = cf::launch_real_enc_fwd_two_role(a_ik, rpos_ij_e, tvecs_n, batch_i, edge_ij_e, pairs_u, U, N, H, E, K, D,
                                          bin_step, s_scale, W_k, rvlen_n, cutoff, lattice_range, minimum_range,
                                          (const float *)rings, order, counts, z_ek, v_ekd, st);
    CF_REQUIRE(rc == CF_OK, rc, "cf_real_enc_fwd_rings: unsupported shape");
    CF_CHECK_LAUNCH("cf_real_enc_fwd_rings (adaptive boxes)");
    return CF_OK;
}
