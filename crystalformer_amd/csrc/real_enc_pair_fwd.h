// Real-space periodic encoding, forward, matrix-core version for gfx950: the body of the pair
// kernel, shared by the kernel of real_enc_mfma.hip and the two-role kernel of real_enc_ring.hip.
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
// A work-group is 8 wavefronts; in every round each wavefront owns one unit.
// Lane roles inside a wavefront (q = lane / 16, c = lane % 16):
//   staging      lane = translation (64 at a time): decode, d^2, sqrt, in-box
//                bits of the 16 columns and "which 16-bin tiles can this distance
//                reach" bits -> per-wave LDS ring.  Translations out of reach of
//                every bin are packed at the back of the ring so that whole
//                groups of 4 skip the Gaussians;
//   accumulation for each group of 4 translations, lane (q, c) reads translation
//                q of the group, forms column c's weight exp(a_c (d^2 - d^2min_c))
//                (B operand) and, for the tiles the group can reach, the Gaussians
//                of bins 16m + c (A operands);
//   projection   v = W_h S: the 8 wavefronts park their normalised S in LDS; then
//                wavefront w multiplies head w's D x K matrix (held in registers
//                as MFMA A operands for the whole kernel) with the 16 columns of
//                that head (8 units x 2 directions) and stores 16-byte rows of v.
//
// Adaptive boxes (UNIFORM = false): the 16 columns of a unit have half-widths of their own
// (models/kernels/real_enc_fwd.cu:58-85), worked out one axis per lane.  Three kinds of unit,
// told apart with one ballot each: all columns have the cube [-lattice_range, lattice_range]^3
// (the cube's shortcuts: translations decoded once per kernel, no column masks); all columns
// have the same box (no per-column tables, lookups, minima or masks); otherwise per-axis
// tables of column sets and a 16-bit column mask per translation.
#pragma once

#include <type_traits>

#include "real_enc_pair.h"

namespace cfpair {

constexpr int RING_CAP = 192;            // translations staged per pass (256 is 3 % slower with boxes of ~100, 1 % faster with ~1000)
constexpr int RING_CAP_SMALL = 128;      // the same for a fixed cube that fits (see SHORT_RING in the kernel)
constexpr int RING_SLOTS = RING_CAP + 16; // + neutral padding (last groups, look-ahead) between the two blocks


// Projection modes
constexpr int PROJ_NONE = 0;             // v = normalised Gaussian averages (E,H,K)
constexpr int PROJ_SHARED = 1;           // one W per head: batched on the matrix cores
constexpr int PROJ_INDEXED = 2;          // W per edge or per atom: read from global memory


// LDS per work-group: per wave three ring arrays of ring capacity + 16 words (d^2, distance
// argument, flag bits); for PROJ_SHARED also the exchange buffer of 4 NT planes of XPLANE floats
// (layout in real_enc_pair.h), WPB x 2 edge ids and WPB x 16 reciprocal column totals.
// block_id / grid_size: this work-group's position among the work-groups that share the rounds.
template <int NT, bool UNIFORM, int PROJ, int DT, bool SHORT_RING>
__device__ __forceinline__ void real_enc_fwd_pair_body(const PairArgs &p, const PairArgsSeg seg, const int block_id,
                                                       const int grid_size)
{
    extern __shared__ __align__(16) float lds[];
    constexpr int SPLANE = XPLANE;      // exchange buffer of the shared-projection epilogue
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);   // wave-uniform by construction
    const int q = lane >> 4;
    const int c = lane & 15;
    const int H = p.H, K = p.K, D = p.D;
    // (p: the arguments as the compiler holds them; seg: the same in the kernel-argument segment, for
    // the pointers that are fetched when they are needed, see real_enc_pair.h)
    // SHORT_RING (a fixed cube of at most 128 translations, the default cube has 125): the ring
    // holds 128 translations per pass, no more than the cube needs.  Fewer distances cached in
    // registers across the staging passes and less LDS per work-group than with a ring of 256:
    // 56.0 against 57.8 us at 56 440 edges, and more room for the kernels of other streams.
    static_assert(!SHORT_RING || UNIFORM, "the short ring is for the fixed cube");
    constexpr int RCAP = SHORT_RING ? RING_CAP_SMALL : RING_CAP;
    constexpr int RSLOTS = RCAP + 16;
    float *ring_d2 = lds + wave * (3 * RSLOTS);
    float *ring_s = ring_d2 + RSLOTS;
    int *ring_bits = reinterpret_cast<int *>(ring_s + RSLOTS);
    float *Sbuf = lds + WPB * 3 * RSLOTS;                            // [4 NT][SPLANE]
    int64_t *meta = reinterpret_cast<int64_t *>(Sbuf + 4 * NT * SPLANE);   // [WPB][2]
    float *invbuf = reinterpret_cast<float *>(meta + WPB * 2);             // [WPB][16]

    // Gaussian argument of bin 16m + c at distance 0
    float ck[NT];
#pragma unroll
    for (int m = 0; m < NT; m++) ck[m] = p.bin_step * (float)(16 * m + c + 1);

    // projection operands of this wave's head, reloaded when the head group changes
    float Wa[PROJ == PROJ_SHARED ? DT : 1][PROJ == PROJ_SHARED ? 4 * NT : 1];
    int wa_hg = -1;

    const int rounds_per_hg = (int)((p.U + WPB - 1) / WPB);
    const int rounds = rounds_per_hg * p.head_groups;
    // unit of round rd_ for this wave (0 when the round or the unit does not exist: loads stay valid)
    auto unit_of = [&](int rd_, const RoundPos &rp) -> int64_t {
        const int64_t slot = (int64_t)rp.r * WPB + wave;
        if (!(rd_ < rounds && slot < p.U)) return 0;
        return p.order ? (int64_t)ordered_unit(p.order, (int)slot) : slot;
    };
    // exponent of column c of a unit in the head group of a round
    auto load_a = [&](const float *g_a, const UnitIds &d, const RoundPos &rp) -> float {
        const int h_ = min(rp.hg * 8 + (c & 7), H - 1);
        return g_a[((c < 8) ? d.i : d.j) * H + h_];
    };
    // Rounds: the first three of a work-group are dealt by position (blockIdx, + grid, + 2 grid);
    // after that either the fixed stride goes on or, with scheduling words, every further round
    // is a ticket drawn from a counter shared by all work-groups, so that they run dry together
    // whatever their units cost.  A unit's result does not depend on who computes it.
    __shared__ int tick[2];
    unsigned int *__restrict__ sched = p.sched;
    const int stride = grid_size;
    int rd_first = block_id, rd_next = block_id + stride, rd_next2 = block_id + 2 * stride;
    RoundPos pos = round_pos(rd_first, rounds_per_hg, p.head_groups);
    RoundPos pos_next = round_pos(rd_next, rounds_per_hg, p.head_groups);
    // fill the descriptor pipeline: current round complete, next round's ids known
    UnitIds ids = unit_ids(load_unit_ids(p.pairs, unit_of(rd_first, pos), lane));
    float a_cur;
    UnitGeom geo;
    UnitIds ids_next;
    {
        const float gv0 = load_unit_geom(ids, lane, p.rpos, p.tvecs, UNIFORM ? nullptr : p.rvlen);
        a_cur = load_a(p.a_ik, ids, pos);
        const int64_t dv1 = load_unit_ids(p.pairs, unit_of(rd_next, pos_next), lane);
        geo = unit_geom(gv0, !UNIFORM);
        ids_next = unit_ids(dv1);
    }
    // Fixed cube: the translation a lane evaluates in chunk ch is the same in every round; the
    // first two chunks (128 translations, the default cube has 125) are decoded once.
    // The adaptive rule yields that very cube for every unit whose 16 columns all stay at the
    // floor of lattice_range (most units when the floor is on and the Gaussians are narrow), so
    // the adaptive kernel keeps the decoded cube as well and takes the cube's shortcuts for them.
    constexpr int NPRE = 2;
    float npre[NPRE][3];
    {
        BoxDims b0;
        b0.U1 = b0.U2 = b0.U3 = p.lattice_range;
        b0.S3 = b0.S2 = 2 * p.lattice_range + 1;
        b0.plane = b0.S2 * b0.S3;
        b0.T = b0.S2 * b0.plane;
        b0.inv_plane = 1.0f / (float)b0.plane;
        b0.inv_S3 = 1.0f / (float)b0.S3;
#pragma unroll
        for (int ch = 0; ch < NPRE; ch++) {
            int n1, n2, n3;
            decode(b0, min(ch * WAVE + lane, b0.T - 1), n1, n2, n3);
            npre[ch][0] = (float)n1;
            npre[ch][1] = (float)n2;
            npre[ch][2] = (float)n3;
        }
    }
    int it = 0;
    for (int rd = rd_first; rd < rounds; it++) {
        const int hg = pos.hg;
        const bool unit_on = (int64_t)pos.r * WPB + wave < p.U;
        const RoundPos pos_next2 = round_pos(rd_next2, rounds_per_hg, p.head_groups);
        // (adaptive boxes: the addresses of the once-a-round loads are formed here, not kept in
        // registers across the rounds)
        int lane_r = lane;
        if (!UNIFORM) asm volatile("" : "+v"(lane_r));
        // ticket for the round after rd_next2 (once past the end, no more draws): requested here,
        // looked at only before the epilogue, like the loads below
        unsigned int ticket_old = 0;
        const bool draw = sched && wave == 0 && rd_next2 < rounds;
        if (draw && lane == 0) ticket_old = atomicAdd(sched, 1u);
        // loads for the coming rounds, consumed just before this round's epilogue
        const PairArgsSeg in = reread(seg);
        const float *__restrict__ g_rvlen = UNIFORM ? nullptr : seg_pointer(&in->rvlen);
        const float gv_next = load_unit_geom(ids_next, lane_r, seg_pointer(&in->rpos), seg_pointer(&in->tvecs), g_rvlen);
        const float a_next = load_a(in->a_ik, ids_next, pos_next);
        const int64_t dv_next2 = load_unit_ids(in->pairs, unit_of(rd_next2, pos_next2), lane_r);
        if (PROJ == PROJ_SHARED && hg != wa_hg) {
            const int hw = hg * 8 + wave;
            const float *__restrict__ g_W = reread(seg)->W;
            if (hw < H && K == 16 * NT && D == 16 * DT) {
                // full tiles: one base address per lane, 16-byte loads at fixed offsets
                // (proj_bin(s, q) = 16 (s / 4) + 4 q + s % 4)
                int qw = q, cw = c;
                if (!UNIFORM) asm volatile("" : "+v"(qw), "+v"(cw));
#pragma unroll
                for (int dt = 0; dt < DT; dt++) {
                    const float *wrow = g_W + ((int64_t)hw * D + 16 * dt + cw) * K + 4 * qw;
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
                        Wa[dt][s] = (hw < H && d < D && k < K) ? g_W[((int64_t)hw * D + d) * K + k] : 0.f;
                    }
            }
            wa_hg = hg;
        }
        const int64_t e_ij = ids.e_ij, e_ji = ids.e_ji, i = ids.i, j = ids.j;
        Cell cell;
        cell.rx = geo.rx;
        cell.ry = geo.ry;
        cell.rz = geo.rz;
#pragma unroll
        for (int x = 0; x < 9; x++) cell.t[x] = geo.t[x];

        // column c: head (hg*8 + c%8) of atom i (c < 8) or atom j (c >= 8)
        const int h = hg * 8 + (c & 7);
        const bool col_on = unit_on && h < H && (c < 8 || e_ji != e_ij);
        const int64_t atom = (c < 8) ? i : j;
        const float a = col_on ? a_cur : -1.0f;
        const float a2 = a * LOG2E;

        // translation box: union over the 16 columns; per-column boxes when they differ
        BoxDims bx;
        bx.U1 = bx.U2 = bx.U3 = p.lattice_range;
        // (lane (q, c) works out axis q of column c; the row maxima are the union box)
        int Rq = 0, Uq = 0;
        if (!UNIFORM) {
            Rq = column_axis_range(a, p.cutoff, geo.rvl, p.lattice_range, p.min_range, q, col_on);
            Uq = row16_max_i(Rq);
            bx.U1 = __builtin_amdgcn_readlane(Uq, 0);
            bx.U2 = __builtin_amdgcn_readlane(Uq, 16);
            bx.U3 = __builtin_amdgcn_readlane(Uq, 32);
        }
        bx.S3 = 2 * bx.U3 + 1;
        bx.S2 = 2 * bx.U2 + 1;
        bx.plane = bx.S2 * bx.S3;
        bx.T = (2 * bx.U1 + 1) * bx.plane;
        bx.inv_plane = __builtin_amdgcn_rcpf((float)bx.plane);
        bx.inv_S3 = __builtin_amdgcn_rcpf((float)bx.S3);
        const int T = bx.T;
        // all active columns of this unit have the box [-lattice_range, lattice_range]^3 (wave-uniform)
        // ... or at least all the same box, the union (wave-uniform as well): then every translation of
        // the box counts for every column and the per-column tables, lookups and minima are not needed
        bool cube = UNIFORM, same_box = UNIFORM;
        if (!UNIFORM) {
            const int lr = p.lattice_range;
            const bool other = col_on && q < 3 && Rq != Uq;
            same_box = __ballot(other) == 0ull;
            cube = same_box && bx.U1 == lr && bx.U2 == lr && bx.U3 == lr && NPRE * WAVE >= T;
        }

        ColumnBoxes cbox{0, 0, 0};
        if (!UNIFORM && !same_box) cbox = column_boxes_rows(Rq, bx, lane);
        // geometry of one translation: d^2 and the in-box bits of the 16 columns
        auto geometry = [&](int idx, bool valid, float &d2, int &colbits) {
            int n1, n2, n3;
            decode(bx, valid ? idx : 0, n1, n2, n3);
            d2 = dist2(cell, (float)n1, (float)n2, (float)n3);
            if (UNIFORM) {
                colbits = valid ? 0xFFFF : 0;
            } else {
                colbits = 0xFFFF;
                if (!same_box) colbits = column_bits(cbox, n1, n2, n3);     // all lanes take part in the lookup
                if (!valid) colbits = 0;
            }
        };
        // First pass over the box: the nearest image inside at least one column's box.  Boxes of up
        // to RCAP translations are evaluated once and kept in registers.
        float best = 1e10f;
        int best_idx = 0;
        auto track_min = [&](float d2, int colbits, int idx) {
            if (colbits != 0 && d2 < best) {
                best = d2;
                best_idx = idx;
            }
        };
        // (adaptive boxes: only the cube's distances are kept; other boxes are evaluated again by the
        // staging passes, their minimum coming from the cube where it can, see below)
        constexpr int NCACHE = UNIFORM ? RCAP / WAVE : NPRE;
        float d2c[NCACHE];
        const bool cached = UNIFORM ? T <= RCAP : cube;
        // chunks of 64 translations in the box; kept opaque so that the chunk guards below stay
        // real (wave-uniform) branches instead of being folded into lane predicates
        const int nchunk = __builtin_amdgcn_readfirstlane((T + WAVE - 1) / WAVE);
        // Boxes too large to keep: where the box of every active column holds the pre-decoded cube,
        // the smallest d^2 over the cube stands in for the minimum over the box and the first pass
        // is left out.  It is an upper bound of every column's own minimum, so the weights
        // exp(a (d^2 - d^2ref)) of closer images exceed 1 (bounded by 2^100, see the test) and the
        // 2^-40 drop below stays on the safe side; z = log(sum) + a d^2ref holds for any d^2ref.
        bool quick_min = false;
        if (!UNIFORM && !cached) {
            const int lr = p.lattice_range;
            const int side = 2 * lr + 1;
            const bool short_col = col_on && q < 3 && Rq < lr;
            if (NPRE * WAVE >= side * side * side && __ballot(short_col) == 0ull) {
                float m = 1e10f;
#pragma unroll
                for (int ch = 0; ch < NPRE; ch++)        // (lanes past the cube repeat its last translation)
                    m = fminf(m, dist2(cell, npre[ch][0], npre[ch][1], npre[ch][2]));
                m = wave_min(m);
                const float a2_strong = row16_max(col_on ? -a2 : 0.f);
                quick_min = __builtin_amdgcn_readfirstlane((int)(a2_strong * m <= 100.0f)) != 0;
                if (quick_min) best = m;
            }
        }
        if (cached) {
#pragma unroll
            for (int ch = 0; ch < NCACHE; ch++) {
                d2c[ch] = 0.f;
                if (ch < nchunk) {
                    int cb;
                    if (cube && ch < NPRE) {
                        d2c[ch] = dist2(cell, npre[ch < NPRE ? ch : 0][0], npre[ch < NPRE ? ch : 0][1],
                                        npre[ch < NPRE ? ch : 0][2]);
                        cb = ch * WAVE + lane < T ? 0xFFFF : 0;
                    } else {
                        geometry(ch * WAVE + lane, ch * WAVE + lane < T, d2c[ch], cb);
                    }
                    track_min(d2c[ch], cb, ch * WAVE + lane);
                }
            }
        } else if (!quick_min) {
            for (int c0 = 0; c0 < T; c0 += WAVE) {
                float d2;
                int cb;
                geometry(c0 + lane, c0 + lane < T, d2, cb);
                track_min(d2, cb, c0 + lane);
            }
        }
        // Per-column minimum of d^2 over the column's own box: the overall minimum wherever the
        // nearest image lies inside the column's box (nearly always); otherwise a pass that
        // tracks the 16 columns separately.
        float d2min = wave_min(best);
        if (!UNIFORM && !same_box && !quick_min) {
            const unsigned long long holders = __ballot(best == d2min);
            const int src = __builtin_amdgcn_readfirstlane(__ffsll((long long)holders) - 1);
            const int idx_star = __builtin_amdgcn_readlane(best_idx, src);
            int n1, n2, n3;
            decode(bx, idx_star, n1, n2, n3);
            const int inside = __builtin_amdgcn_readfirstlane(column_bits(cbox, n1, n2, n3));
            const bool own_min = col_on && !((inside >> c) & 1);
            if (__ballot(own_min) != 0ull) {
                float mloc[16];
#pragma unroll
                for (int x = 0; x < 16; x++) mloc[x] = 1e10f;
                for (int c0 = 0; c0 < T; c0 += WAVE) {
                    float d2;
                    int cb;
                    geometry(c0 + lane, c0 + lane < T, d2, cb);
#pragma unroll
                    for (int x = 0; x < 16; x++)
                        if ((cb >> x) & 1) mloc[x] = fminf(mloc[x], d2);
                }
#pragma unroll
                for (int x = 0; x < 16; x++) {
                    const float mx = wave_min(mloc[x]);
                    if (c == x) d2min = mx;
                }
            }
        }
        // A translation out of reach of every bin whose weight is below 2^-40 of the leading
        // term in EVERY column cannot change an fp32 sum and is dropped.  For all columns
        // a2_c (d2 - d2min_c) <= a2_weak (d2 - d2min_far) with the weakest decay and the
        // largest per-column minimum.
        // (every row of 16 lanes holds the 16 columns, so a reduction over a row is complete)
        const float a2_weak = row16_max(col_on ? a2 : -3.0e38f);
        const float d2min_far = UNIFORM ? d2min : row16_max(col_on ? d2min : 0.f);

        float4_t acc[NT];
#pragma unroll
        for (int m = 0; m < NT; m++) acc[m] = float4_t{0.f, 0.f, 0.f, 0.f};
        float sum = 0.f;
        for (int s0 = 0; s0 < T; s0 += RCAP) {
            const int cnt = min(RCAP, T - s0);
            // ---- staging, lane = translation.  "Near" translations (some bin within reach)
            // are packed upwards from slot 0, the remaining live ones downwards from the top
            // of the ring, so that the second kind never enters the Gaussian loop.
            int near_cnt = 0, far_cnt = 0;
            auto stage = [&](float d2, int colbits, bool valid) {
                asm volatile("" : "+v"(d2));      // keeps this chunk's arithmetic behind its guard
                const float s = sqrt_hw(d2) * p.s_scale;
                const float xb = s * p.inv_bin_step - 1.0f;          // fractional bin coordinate
                int bits = colbits;
                if (valid) {
#pragma unroll
                    for (int m = 0; m < NT; m++)
                        if (xb >= (float)(16 * m) - p.window && xb <= (float)(16 * m + 15) + p.window)
                            bits |= (0x10000 << m);
                }
                const int tiles = bits >> 16;
                const bool is_near = valid && tiles != 0;
                const bool is_far = valid && !is_near && colbits != 0 && a2_weak * (d2 - d2min_far) > -40.0f;
                const unsigned long long far_mask = __ballot(is_far);
                const unsigned long long below = (1ull << lane) - 1ull;
                int pos = -1;
                int near_now;
                if (NT > 1) {
                    // The near translations of this chunk go in ordered by the lowest tile they
                    // reach, so that the four translations of a group reach ~1.9 tiles between
                    // them instead of ~2.5 in box order (each tile costs an exponential and an
                    // MFMA).  One packed prefix sum ranks all classes at once: 8-bit counters per
                    // class (at most 64 per chunk), class = lowest tile (pairs of tiles for 8).
                    const int key8 = tiles ? 8 * (__builtin_ctz(tiles) >> (NT > 4 ? 1 : 0)) : 0;
                    const int onehot = is_near ? (1 << key8) : 0;
                    const int incl = wave_inclusive_scan_i(onehot);
                    const int totals = __builtin_amdgcn_readlane(incl, 63);
                    const int before = (totals << 8) + (totals << 16) + (totals << 24);   // classes below, packed
                    if (is_near) pos = near_cnt + (((before + incl - onehot) >> key8) & 0xFF);
                    near_now = (int)(((unsigned)totals * 0x01010101u) >> 24);
                } else {
                    const unsigned long long near_mask = __ballot(is_near);
                    if (is_near) pos = near_cnt + __popcll(near_mask & below);
                    near_now = __popcll(near_mask);
                }
                if (is_far) pos = RSLOTS - 1 - (far_cnt + __popcll(far_mask & below));
                if (pos >= 0) {
                    ring_d2[pos] = d2;
                    ring_s[pos] = s;
                    ring_bits[pos] = bits;
                }
                near_cnt += near_now;
                far_cnt += __popcll(far_mask);
            };
            if (cached) {
#pragma unroll
                for (int ch = 0; ch < NCACHE; ch++)
                    if (ch < nchunk) stage(d2c[ch], ch * WAVE + lane < T ? 0xFFFF : 0, ch * WAVE + lane < T);
            } else {
                for (int c0 = 0; c0 < cnt; c0 += WAVE) {
                    float d2;
                    int cb;
                    geometry(s0 + c0 + lane, c0 + lane < cnt, d2, cb);
                    stage(d2, cb, c0 + lane < cnt);
                }
            }
            // neutral records: 8 after the near block (last group + look-ahead), 4 below the far block
            if (lane < 12) {
                const int pos = lane < 8 ? near_cnt + lane : RSLOTS - far_cnt - 1 - (lane - 8);
                ring_d2[pos] = __builtin_inff();
                ring_s[pos] = 0.f;
                ring_bits[pos] = 0;
            }
            wave_mem_sync();
            // the tiles any of a group's four records reaches, kept in each record (see
            // with_group_reach): the four records of a group sit in four adjacent lanes here
            for (int s4 = 0; s4 < near_cnt; s4 += WAVE) {
                const bool held = s4 + lane < near_cnt + 8;          // (slots up to near_cnt + 7 hold records)
                const int marked = with_group_reach(held ? ring_bits[s4 + lane] : 0);
                if (held) ring_bits[s4 + lane] = marked;
            }
            wave_mem_sync();
            // ---- accumulation over the near block: 4 translations per MFMA, two groups per trip,
            // each with its own registers for the prefetched records (records beyond the last
            // group are the neutral padding)
            {
                const int groups = (near_cnt + 3) >> 2;
                struct Rec { float d2, s; int bits; };
                auto fetch = [&](int g_) -> Rec {
                    const int slot = 4 * g_ + q;
                    return Rec{ring_d2[slot], ring_s[slot], ring_bits[slot]};
                };
                // PLAIN: every staged translation counts for every column (fixed cube, or adaptive
                // boxes that came out the same for all columns)
                auto group = [&](const Rec &rec, auto plain) {
                    constexpr bool PLAIN = decltype(plain)::value;
                    float w = exp2_hw(a2 * (rec.d2 - d2min));
                    // (fixed cube: every staged translation is inside every column's box, and the
                    // padding records carry d2 = +inf, i.e. weight 0)
                    w = (col_on && (PLAIN || ((rec.bits >> c) & 1))) ? w : 0.f;
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
                if (UNIFORM || same_box) {
                    for (int g = 0; g < groups; g += 2) {
                        const Rec rb = fetch(g + 1);
                        group(ra, std::true_type{});
                        if (g + 1 < groups) {
                            ra = fetch(g + 2);
                            group(rb, std::true_type{});
                        }
                    }
                } else {
                    for (int g = 0; g < groups; g += 2) {
                        const Rec rb = fetch(g + 1);
                        group(ra, std::false_type{});
                        if (g + 1 < groups) {
                            ra = fetch(g + 2);
                            group(rb, std::false_type{});
                        }
                    }
                }
            }
            // ---- the far block only feeds the column sums
            {
                const int groups = (far_cnt + 3) >> 2;
                for (int g = 0; g < groups; g++) {
                    const int slot = RSLOTS - 4 * (g + 1) + q;
                    const float d2t = ring_d2[slot];
                    const int bits = ring_bits[slot];
                    float w = exp2_hw(a2 * (d2t - d2min));
                    sum += (col_on && (same_box || ((bits >> c) & 1))) ? w : 0.f;
                }
            }
            wave_mem_sync();
        }
        // the loads issued at the top of the round have landed: make them uniform before the
        // stores of the epilogue so that nothing younger is waited for
        const UnitGeom geo_next = unit_geom(gv_next, !UNIFORM);
        const UnitIds ids_next2 = unit_ids(dv_next2);
        if (sched && wave == 0) {
            // read by all wavefronts at the end of the iteration, behind the barriers of the epilogue
            const int t = draw ? 3 * stride + (int)__builtin_amdgcn_readfirstlane(ticket_old) : rd_next2;
            if (lane == 0) tick[it & 1] = t;
        }
        // column totals: the 4 lanes sharing c hold partial sums
        sum = rows_sum(sum);
        const float inv = __builtin_amdgcn_rcpf(sum);      // 1 ulp, one instruction
        const int64_t e_col = (c < 8) ? e_ij : e_ji;
        const PairArgsSeg outp = reread(seg);
        float *__restrict__ g_z = outp->z;
        float *__restrict__ g_v = outp->v;
        if (col_on && q == 0) g_z[e_col * H + h] = log2_hw(sum) * LN2 + d2min * a;

        // epilogue: lane (q,c) holds S[bin = 16m + 4q + r][column c] in acc[m][r]
        if (PROJ == PROJ_NONE) {
            if (col_on) {
#pragma unroll
                for (int m = 0; m < NT; m++) {
                    int k0 = 16 * m + 4 * q;
                    float *dst = g_v + (e_col * H + h) * K + k0;
#pragma unroll
                    for (int r = 0; r < 4; r++)
                        if (k0 + r < K) dst[r] = acc[m][r] * inv;
                }
            }
        } else if (PROJ == PROJ_SHARED) {
            // park the column sums (inactive columns hold zeros: their weights are masked) and the
            // reciprocal of the column totals, then project per head
            float *col = Sbuf + xch_base(q, c & 7, wave, c >> 3);
#pragma unroll
            for (int m = 0; m < NT; m++)
#pragma unroll
                for (int r = 0; r < 4; r++) col[(4 * m + r) * SPLANE] = acc[m][r];
            if (q == 0) invbuf[wave * 16 + c] = inv;
            if (lane == 0) {
                meta[2 * wave + 0] = unit_on ? e_ij : -1;
                meta[2 * wave + 1] = (unit_on && e_ji != e_ij) ? e_ji : -1;
            }
            __syncthreads();
            {
                // this wave: head hw; column j of the product = direction j/8 of unit j%8
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
                    for (int r = 0; r < 4; r++) sb[r] = src[(4 * t4 + r) * SPLANE];
#pragma unroll
                    for (int r = 0; r < 4; r++)
#pragma unroll
                        for (int dt = 0; dt < DT; dt++)
                            out[dt] = __builtin_amdgcn_mfma_f32_16x16x4f32(Wa[dt][4 * t4 + r], sb[r], out[dt], 0, 0, 0);
                }
                // lane (q, j) holds components 16dt + 4q + r of column j, still to be normalised
                const int64_t e_out = meta[2 * unit_j + dir_j];
                const float inv_j = invbuf[unit_j * 16 + dir_j * 8 + wave];
#pragma unroll
                for (int dt = 0; dt < DT; dt++) out[dt] *= inv_j;
                if (e_out >= 0 && hw < H) {
#pragma unroll
                    for (int dt = 0; dt < DT; dt++) {
                        const int dbase = 16 * dt + 4 * q;
                        float *dst = g_v + (e_out * H + hw) * D + dbase;
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
        } else {
            int64_t w_ind = 0;
            if (p.W_num == p.E) w_ind = e_col;
            else if (p.W_num == p.N) w_ind = atom;
            const float *Wg = reread(seg)->W + (w_ind * H + (col_on ? h : 0)) * (int64_t)D * K;
            for (int d0 = 0; d0 < D; d0 += 16) {
                float o0 = 0.f, o1 = 0.f, o2 = 0.f, o3 = 0.f;   // this lane's 4 output components
#pragma unroll
                for (int dd = 0; dd < 16; dd++) {
                    float o = 0.f;
                    if (col_on && d0 + dd < D) {
#pragma unroll
                        for (int m = 0; m < NT; m++) {
                            const int k0 = 16 * m + 4 * q;
#pragma unroll
                            for (int r = 0; r < 4; r++)
                                if (k0 + r < K) o = fmaf(Wg[(int64_t)(d0 + dd) * K + k0 + r], acc[m][r], o);
                        }
                    }
                    o = rows_sum(o);
                    // lane q keeps components 4q .. 4q+3
                    if ((dd >> 2) == q) {
                        if ((dd & 3) == 0) o0 = o;
                        else if ((dd & 3) == 1) o1 = o;
                        else if ((dd & 3) == 2) o2 = o;
                        else o3 = o;
                    }
                }
                if (col_on) {
                    const int dbase = d0 + 4 * q;
                    float *dst = g_v + (e_col * H + h) * D + dbase;
                    if (dbase + 0 < D) dst[0] = o0 * inv;
                    if (dbase + 1 < D) dst[1] = o1 * inv;
                    if (dbase + 2 < D) dst[2] = o2 * inv;
                    if (dbase + 3 < D) dst[3] = o3 * inv;
                }
            }
        }
        ids = ids_next;
        geo = geo_next;
        a_cur = a_next;
        ids_next = ids_next2;
        pos = pos_next;
        pos_next = pos_next2;
        int rd_next3 = rd_next2 + stride;
        if (sched) {
            if (PROJ != PROJ_SHARED) __syncthreads();     // (the shared projection has its own barriers)
            rd_next3 = tick[it & 1];
        }
        rd = rd_next;
        rd_next = rd_next2;
        rd_next2 = rd_next3;
    }
    if (sched && threadIdx.x == 0) {
        // the last work-group to run dry leaves the words as it found them
        if (atomicAdd(sched + 1, 1u) == grid_size - 1) {
            sched[0] = 0;
            sched[1] = 0;
        }
    }
}

}  // namespace cfpair
