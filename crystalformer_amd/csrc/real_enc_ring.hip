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

// ---------------------------------------------------------------- unit selection
// Adaptive boxes: which units keep the fixed cube in all their active columns (the range rule of
// every (atom, head) of the unit yields lattice_range on the three axes).  Those are evaluated from
// the staged rings, on the bits the pair kernel's own shortcut for such units produces; the others
// go to the pair kernel.  One wavefront per round (8 units) and head group: lane = (unit, head),
// each lane applies the rule to its head of atoms i and j.
__global__ __launch_bounds__(256) void unit_floor_kernel(PairArgs p, unsigned char *__restrict__ unit_flags,
                                                         unsigned char *__restrict__ round_flags)
{
    const int lane = threadIdx.x & 63;
    const int rounds_per_hg = (int)((p.U + WPB - 1) / WPB);
    const int64_t rounds = (int64_t)rounds_per_hg * p.head_groups;
    const int64_t rd = (int64_t)blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
    if (rd >= rounds) return;
    const RoundPos rp = round_pos((int)rd, rounds_per_hg, p.head_groups);
    const int w = lane >> 3, hh = lane & 7;
    const int64_t u = (int64_t)rp.r * WPB + w;
    const bool exists = u < p.U;
    bool keeps = true;
    if (exists) {
        const int64_t *d = p.pairs + u * PAIR_FIELDS;
        const int64_t e_ij = d[0], e_ji = d[1], n = d[4];
        const int h = rp.hg * 8 + hh;
        if (h < p.H) {
            const float rvl[3] = {p.rvlen[n * 3 + 0], p.rvlen[n * 3 + 1], p.rvlen[n * 3 + 2]};
#pragma unroll
            for (int side = 0; side < 2; side++) {
                if (side == 1 && e_ji == e_ij) continue;         // a self pair has one direction
                int R1, R2, R3;
                range_rule(p.a_ik[d[2 + side] * p.H + h], p.cutoff, rvl, p.lattice_range, p.min_range, R1, R2, R3);
                keeps = keeps && R1 == p.lattice_range && R2 == p.lattice_range && R3 == p.lattice_range;
            }
        }
    }
    const unsigned long long km = __ballot(keeps);
    const bool unit_keeps = exists && ((km >> (8 * w)) & 0xFFull) == 0xFFull;
    if (exists && hh == 0) unit_flags[(int64_t)rp.hg * p.U + u] = unit_keeps ? 1 : 0;
    const unsigned long long any_keep = __ballot(unit_keeps), any_other = __ballot(exists && !unit_keeps);
    if (lane == 0) round_flags[rd] = (unsigned char)((any_keep != 0ull ? 1 : 0) | (any_other != 0ull ? 2 : 0));
}

// ---------------------------------------------------------------- consumer
// Work-group of 8 wavefronts, one unit per wavefront and round, as in the pair kernel.  The image
// of the next round's unit (its address follows from the round number alone) is requested a round
// ahead into registers and copied to the wavefront's LDS ring at the top of its round.
// LDS: per wave 3 x RS words, exchange buffer 4 NT x XPLANE, 8 x 2 edge ids, 8 x 16 reciprocals.
// SELECT: only the units picked by p.unit_flags / p.flag_want are evaluated, and only the rounds
// that hold one are walked (p.round_flags).
template <int NT, int DT, bool SELECT>
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
    auto unit_of = [&](int rd_, const RoundPos &rp) -> int64_t {
        const int64_t u_ = (int64_t)rp.r * WPB + wave;
        return (rd_ < rounds && u_ < p.U) ? u_ : 0;
    };
    auto load_a = [&](const UnitIds &d, const RoundPos &rp) -> float {
        const unsigned h_ = (unsigned)min(rp.hg * 8 + (c & 7), H - 1);
        return g_a[((c < 8) ? (unsigned)d.i : (unsigned)d.j) * (unsigned)H + h_];
    };
    using Image = RingImage;
    auto load_image = [&](int64_t u_) -> Image { return load_ring_image(cache, u_, lane); };

    // rounds of this work-group: block_id, + grid, + 2 grid, ...; with SELECT those of them that
    // hold a unit of this launch, known three rounds ahead
    int rd, rd_next, rd_next2;
    if (SELECT) {
        const RoundSeq seq = first_active_rounds(p, block_id, rounds, stride, lane);
        rd = seq.rd[0];
        rd_next = seq.rd[1];
        rd_next2 = seq.rd[2];
    } else {
        rd = block_id;
        rd_next = rd + stride;
        rd_next2 = rd + 2 * stride;
    }
    auto unit_flag = [&](int rd_, const RoundPos &rp) -> int {
        return SELECT ? load_unit_flag(p, unit_of(rd_, rp), rd_ < rounds ? rp.hg : 0) : 0;
    };
    RoundPos pos = round_pos(rd, rounds_per_hg, p.head_groups);
    RoundPos pos_next = round_pos(rd_next, rounds_per_hg, p.head_groups);
    UnitIds ids = unit_ids(load_unit_ids(g_pairs, unit_of(rd, pos), lane));
    float a_cur = load_a(ids, pos);
    Image img = load_image(unit_of(rd, pos));
    int uflag = unit_flag(rd, pos);
    UnitIds ids_next = unit_ids(load_unit_ids(g_pairs, unit_of(rd_next, pos_next), lane));

    while (rd < rounds) {
        const int hg = pos.hg;
        const int64_t u = (int64_t)pos.r * WPB + wave;
        const bool unit_on = u < p.U && (!SELECT || unit_selected(p, uflag));
        const RoundPos pos_next2 = round_pos(rd_next2, rounds_per_hg, p.head_groups);
        // (the round after rd_next2: its candidates' flags are requested here, looked at at the end)
        bool candidate = false;
        if (SELECT) candidate = request_round_candidate(p, rd_next2, rounds, stride, lane);
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
        const Image img_next = load_image(unit_of(rd_next, pos_next));
        const float a_next = load_a(ids_next, pos_next);
        const int uflag_next = unit_flag(rd_next, pos_next);
        const int64_t dv_next2 = load_unit_ids(g_pairs, unit_of(rd_next2, pos_next2), lane);
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
        uflag = uflag_next;
        ids_next = ids_next2;
        pos = pos_next;
        pos_next = pos_next2;
        const int rd_next3 = SELECT ? round_after(p, candidate, rd_next2, rounds, stride, lane)
                                    : rd_next2 + stride;
        rd = rd_next;
        rd_next = rd_next2;
        rd_next2 = rd_next3;
    }
}

template <int NT, int DT, bool SELECT>
__global__ __launch_bounds__(512, 4) void real_enc_fwd_ring_kernel(PairArgs p_, const float *__restrict__ cache)
{
    const PairArgs p = with_live_units(p_);
    if (p.U == 0) return;          // (an empty list: not even the descriptor of unit 0 may be read)
    real_enc_fwd_ring_body<NT, DT, SELECT>(p, cache, (int)blockIdx.x, (int)gridDim.x);
}

// Adaptive boxes in one launch: the first pair_blocks work-groups run the pair kernel's body over the
// rounds that hold an atom pair which does not keep the cube (few, long rounds; a work-group
// without such a round leaves at once and frees its place), the others the ring body over the
// rounds that hold one which does.  Two independent sets of work-groups, each with its own
// numbering; they write different edges.
template <int NT, int DT>
__global__ __launch_bounds__(512, 4) void real_enc_fwd_two_role_kernel(PairArgs p_ring, PairArgs p_pair,
                                                                       const float *__restrict__ cache,
                                                                       int pair_blocks)
{
    if ((int)blockIdx.x < pair_blocks) {
        // (p_pair is the kernel's second argument, behind p_ring in the kernel-argument segment)
        static_assert(sizeof(PairArgs) % 8 == 0, "the second argument follows the first without padding");
        const PairArgsSeg seg = (PairArgsSeg)__builtin_amdgcn_kernarg_segment_ptr() + 1;
        real_enc_fwd_pair_body<NT, false, PROJ_SHARED, DT, false>(p_pair, seg, (int)blockIdx.x, pair_blocks);
    } else {
        real_enc_fwd_ring_body<NT, DT, true>(p_ring, cache, (int)blockIdx.x - pair_blocks,
                                             (int)gridDim.x - pair_blocks);
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

// Flags for the two launches of the adaptive rule (see unit_floor_kernel): unit_flags holds
// head_groups x U bytes, round_flags one byte per round.
int64_t real_enc_round_count(int64_t U, int64_t H) { return ((U + WPB - 1) / WPB) * ((H + 7) / 8); }

int launch_unit_floor(const float *a_ik, const float *rvlen, const int64_t *pairs, int64_t U, int64_t N, int64_t H,
                      float cutoff, int lattice_range, int min_range, unsigned char *unit_flags,
                      unsigned char *round_flags, hipStream_t st)
{
    PairArgs p{};
    p.a_ik = a_ik; p.rvlen = rvlen; p.pairs = pairs;
    p.N = N; p.U = U; p.H = (int)H;
    p.head_groups = (int)((H + 7) / 8);
    p.cutoff = cutoff; p.lattice_range = lattice_range; p.min_range = min_range;
    const int64_t rounds = real_enc_round_count(U, H);
    if (rounds >= (1ll << 30)) return CF_ERR_UNSUPPORTED;
    if (rounds < 1) return CF_OK;
    unit_floor_kernel<<<(int)((rounds + 3) / 4), 256, 0, st>>>(p, unit_flags, round_flags);
    return CF_OK;
}

// Adaptive boxes, one launch for both kinds of atom pairs (real_enc_fwd_two_role_kernel).
int launch_real_enc_fwd_two_role(const float *a_ik, const float *rpos, const float *tvecs, const int64_t *batch,
                                 const int64_t *edges, const int64_t *pairs, int64_t U, int64_t N, int64_t H,
                                 int64_t E, int64_t K, int64_t D, float bin_step, float s_scale, const float *W,
                                 const float *rvlen, float cutoff, int lattice_range, int min_range,
                                 const float *cache, const unsigned char *unit_flags,
                                 const unsigned char *round_flags, float *z, float *v, hipStream_t st)
{
    if (K < 1 || K > 128 || !W || D < 1 || D > 32 || cutoff == 0.0f || !unit_flags || !round_flags)
        return CF_ERR_UNSUPPORTED;
    if (E * H >= (1ll << 32) || N * H >= (1ll << 32)) return CF_ERR_UNSUPPORTED;      // 32-bit rows in the ring body
    PairArgs pp{};
    pp.a_ik = a_ik; pp.rpos = rpos; pp.tvecs = tvecs; pp.batch = batch; pp.edges = edges; pp.pairs = pairs;
    pp.W = W; pp.rvlen = rvlen; pp.z = z; pp.v = v; pp.sched = nullptr;
    pp.N = N; pp.E = E; pp.U = U; pp.W_num = 1;
    pp.H = (int)H; pp.K = (int)K; pp.D = (int)D;
    pp.head_groups = (int)((H + 7) / 8);
    pp.cutoff = cutoff; pp.lattice_range = lattice_range; pp.min_range = min_range;
    pp.bin_step = bin_step; pp.s_scale = s_scale; pp.inv_bin_step = 1.0f / bin_step;
    pp.window = sqrtf(40.0f) / bin_step;
    pp.unit_flags = unit_flags; pp.round_flags = round_flags; pp.flag_want = 0;       // pairs that leave the cube
    PairArgs pr = pp;                                                                   // pairs that keep it
    pr.rpos = nullptr; pr.tvecs = nullptr; pr.batch = nullptr; pr.edges = nullptr; pr.rvlen = nullptr;
    pr.cutoff = 0.f; pr.flag_want = 1;
    const int NT = K <= 16 ? 1 : K <= 32 ? 2 : K <= 64 ? 4 : 8;
    const int DT = D > 16 ? 2 : 1;
    const size_t shared_proj = sizeof(float) * ((size_t)4 * NT * XPLANE + WPB * 16) + sizeof(int64_t) * WPB * 2 + 8;
    const size_t lds_ring = sizeof(float) * (size_t)WPB * 3 * RS + shared_proj;
    const size_t lds_pair = sizeof(float) * (size_t)WPB * 3 * (RING_CAP + 16) + shared_proj;
    const size_t lds = lds_ring > lds_pair ? lds_ring : lds_pair;
    const int64_t rounds = ((U + WPB - 1) / WPB) * pp.head_groups;
    if (rounds >= (1ll << 30)) return CF_ERR_UNSUPPORTED;
    if (rounds < 1) return CF_OK;
    const int64_t cap = persistent_grid_cap(2);
    const int64_t ring_blocks = rounds < cap ? rounds : cap;
    int64_t pair_blocks = cap / 8 < 1 ? 1 : cap / 8;       // few long rounds: an eighth of the places, freed at once where idle
    if (pair_blocks > rounds) pair_blocks = rounds;
    const int grid = (int)(ring_blocks + pair_blocks);
#define CF_TWO(NTV, DTV) \
    real_enc_fwd_two_role_kernel<NTV, DTV><<<grid, WPB * WAVE, lds, st>>>(pr, pp, cache, (int)pair_blocks)
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

// Forward from staged rings (shared projection, D <= 32).  CF_ERR_UNSUPPORTED otherwise.
// With unit flags only the units that keep the cube are evaluated.
int launch_real_enc_fwd_rings(const float *a_ik, const int64_t *pairs, int64_t U, int64_t N, int64_t H, int64_t E,
                              int64_t K, int64_t D, float bin_step, float s_scale, const float *W,
                              const float *cache, const unsigned char *unit_flags, const unsigned char *round_flags,
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
    p.unit_flags = unit_flags; p.round_flags = round_flags; p.flag_want = 1;      // units that keep the cube
    const bool select = unit_flags != nullptr;
    p.live_U = live_units(U);
    if (p.live_U && select) return CF_ERR_UNSUPPORTED;       // (the flags are laid out for a known U)
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
#define CF_RING(NTV, DTV)                                                                               \
    do {                                                                                                \
        if (select) real_enc_fwd_ring_kernel<NTV, DTV, true><<<(int)blocks, WPB * WAVE, lds, st>>>(p, cache);   \
        else real_enc_fwd_ring_kernel<NTV, DTV, false><<<(int)blocks, WPB * WAVE, lds, st>>>(p, cache);         \
    } while (0)
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

extern "C" int64_t cf_real_enc_ring_bytes(int64_t U) { return (U < 0 ? 0 : U) * RIMG_WORDS * (int64_t)sizeof(float); }

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
    return ((H + 7) / 8) * U + cf::real_enc_round_count(U, H);
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
    CF_REQUIRE(!cf::live_units(U), CF_ERR_UNSUPPORTED,
               "cf_real_enc_fwd_rings: adaptive boxes from the rings need sizes known on the host "
               "(a size header is set): use cf_real_enc_fwd");
    CF_REQUIRE(minimum_range >= 0 && minimum_range <= MAX_RANGE, CF_ERR_INVALID_ARGUMENT,
               "cf_real_enc_fwd_rings: minimum_range %d outside 0..%d", minimum_range, MAX_RANGE);
    CF_REQUIRE(rpos_ij_e && tvecs_n && batch_i && edge_ij_e, CF_ERR_INVALID_ARGUMENT,
               "cf_real_enc_fwd_rings: adaptive boxes need rpos_ij_e, tvecs_n, batch_i and edge_ij_e");
    CF_REQUIRE(flags && flag_bytes >= cf_real_enc_flag_bytes(U, H), CF_ERR_INVALID_ARGUMENT,
               "cf_real_enc_fwd_rings: adaptive boxes need %lld bytes of flags, %lld given",
               (long long)cf_real_enc_flag_bytes(U, H), (long long)flag_bytes);
    unsigned char *unit_flags = (unsigned char *)flags;
    unsigned char *round_flags = unit_flags + ((H + 7) / 8) * U;
    int rc = cf::launch_unit_floor(a_ik, rvlen_n, pairs_u, U, N, H, cutoff, lattice_range, minimum_range, unit_flags,
                                   round_flags, st);
    CF_REQUIRE(rc == CF_OK, rc, "cf_real_enc_fwd_rings: unsupported size");
    // One launch for both kinds of atom pairs.  (Tried before: the two kernels one after the other,
    // 60.4 us per block at 128 crystals, the pair kernel's part being one long round of a few
    // work-groups; and that launch on a second stream between two events beside the ring launch, where
    // fork and join cost more than the overlap won, 62.5 us and 0.31 against 0.26 ms per step with
    // four forwards in flight.)
    rc = cf::launch_real_enc_fwd_two_role(a_ik, rpos_ij_e, tvecs_n, batch_i, edge_ij_e, pairs_u, U, N, H, E, K, D,
                                          bin_step, s_scale, W_k, rvlen_n, cutoff, lattice_range, minimum_range,
                                          (const float *)rings, unit_flags, round_flags, z_ek, v_ekd, st);
    CF_REQUIRE(rc == CF_OK, rc, "cf_real_enc_fwd_rings: unsupported shape");
    CF_CHECK_LAUNCH("cf_real_enc_fwd_rings (adaptive boxes)");
    return CF_OK;
}
