// Real-space periodic encoding, backward, matrix-core version for gfx950
// (shared projection W of shape (H,D,K), the default model path).
//
// Per directed edge and head, with p_t = exp(a d2_t - z):
//     PX = sum_t p_t d2_t,  S_k = sum_t p_t g_k(t),  Q_k = sum_t p_t d2_t g_k(t)
//     ga_edge = gz PX + gv.(W Q) - PX gv.(W S)          (gradient wrt the exponent a)
//             = gz PX + gv.(W (Q - PX S))
//     gW     += gv (x) S                                 (gradient wrt the projection)
// Same decomposition as the forward kernel: a unit is an unordered atom pair, its
// Gaussians are evaluated once per translation for 2 x 16 weight columns
// (8 heads of i and of j, each with p and p*d2), S and Q accumulate on
// v_mfma_f32_16x16x4_f32.  A work-group is 8 wavefronts; per round every
// wavefront owns one unit, then the 8 wavefronts exchange Q' = Q - PX S (and S,
// when the weight gradient is wanted) through LDS and wavefront w does head w
// for all 8 units: W Q' (the forward's projection), its dot product with gv,
// and the rank-16 update of that head's D x K block of gW, which is kept for the
// whole kernel (in registers from staged rings, otherwise in LDS slots of its
// own) and written once per work-group; a second kernel adds the
// per-work-group blocks in a fixed order.  No atomics.
#include <type_traits>
#include "real_enc_pair.h"

namespace {

using namespace cf;
using namespace cfpair;

constexpr int BRING_CAP = RIMG_CAP;         // translations staged per pass
constexpr int BRING_SLOTS = RIMG_SLOTS;

// RINGS: the staged translations of every unit come from memory (p.rings, written once per
// geometry by the staging kernel of real_enc_ring.hip; fixed cube only) instead of being worked
// out here: no lattice or offset loads, no decoding, distances, classification or ranking.
template <int NT, bool UNIFORM, bool RINGS>
__global__ __launch_bounds__(512, 4) void real_enc_bwd_pair_kernel(PairArgs p)
{
    static_assert(UNIFORM || !RINGS, "staged rings hold the fixed cube");
    extern __shared__ __align__(16) float lds[];
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int q = lane >> 4;
    const int c = lane & 15;
    const int H = p.H, K = p.K, D = p.D;
    const int64_t *__restrict__ g_pairs = p.pairs;
    const float *__restrict__ g_rpos = p.rpos;
    const float *__restrict__ g_tvecs = p.tvecs;
    const float *__restrict__ g_a = p.a_ik;
    const float *__restrict__ g_rvlen = p.rvlen;
    const float *__restrict__ g_z = p.z_in;
    const float *__restrict__ g_gz = p.gz;
    const float *__restrict__ g_gv = p.gv;
    float *ring_d2 = lds + wave * (3 * BRING_SLOTS);
    float *ring_s = ring_d2 + BRING_SLOTS;
    int *ring_bits = reinterpret_cast<int *>(ring_s + BRING_SLOTS);
    float *Sbuf = lds + WPB * 3 * BRING_SLOTS;                          // exchange buffer, 4 NT planes (real_enc_pair.h)
    float *PXbuf = Sbuf + 4 * NT * XPLANE;                              // [8 units][16 cols]

    float ck[NT];
#pragma unroll
    for (int m = 0; m < NT; m++) ck[m] = p.bin_step * (float)(16 * m + c + 1);

    // this wave's head: the projection operands are fetched per round just before they are used.
    // The running block of gW: staging for itself, the kernel has no registers to spare and keeps it
    // in LDS between rounds (one 16-byte slot per lane and tile, touched by its own lane only); from
    // staged rings it stays in registers, and the LDS it would take holds a second exchange buffer
    // (S next to Q': one exchange and two barriers per round instead of two and four).
    float4_t *gw_slot = reinterpret_cast<float4_t *>(PXbuf + WPB * 16) + (wave * NT) * WAVE + lane;
    float *Sbuf2 = PXbuf + WPB * 16;                                    // (RINGS only; same place)
    float4_t gWreg[NT];
#pragma unroll
    for (int t = 0; t < NT; t++) gWreg[t] = float4_t{0.f, 0.f, 0.f, 0.f};
    int wa_hg = -1;

    const int rounds_per_hg = (int)((p.U + WPB - 1) / WPB);
    const int rounds = rounds_per_hg * p.head_groups;
    auto unit_of = [&](int rd_, const RoundPos &rp) -> int64_t {
        const int64_t u_ = (int64_t)rp.r * WPB + wave;
        return (rd_ < rounds && u_ < p.U) ? u_ : 0;
    };
    // exponent and forward output of column c of a unit in the head group of a round
    // (atom and edge rows times H fit 32 bits: checked by the launcher)
    auto load_a = [&](const UnitIds &d, const RoundPos &rp) -> float {
        const unsigned h_ = (unsigned)min(rp.hg * 8 + (c & 7), H - 1);
        return g_a[((c < 8) ? (unsigned)d.i : (unsigned)d.j) * (unsigned)H + h_];
    };
    auto load_z = [&](const UnitIds &d, const RoundPos &rp) -> float {
        const unsigned h_ = (unsigned)min(rp.hg * 8 + (c & 7), H - 1);
        return g_z[((c < 8) ? (unsigned)d.e_ij : (unsigned)d.e_ji) * (unsigned)H + h_];
    };
    // edge of product column c of round rd_: direction c/8 of the unit of wave c%8
    // (-1: no such unit, or the reverse of a self edge)
    // (32-bit: the launcher refuses edge counts of 2^31 and more)
    auto load_col_edge = [&](int rd_, const RoundPos &rp) -> int {
        const unsigned u_ = (unsigned)rp.r * WPB + (unsigned)(c & 7);       // (rounds < 2^30)
        if (rd_ >= rounds || (int64_t)u_ >= p.U) return -1;
        const int64_t *d_ = g_pairs + (uint64_t)u_ * PAIR_FIELDS;
        const int e0 = (int)d_[0], e1 = (int)d_[1];
        return (c < 8) ? e0 : (e1 != e0 ? e1 : -1);
    };
    auto flush_gW = [&](int hg_) {
        // lane (q, j) holds gW[d = 4q + r][bin = 16t + j] of head hg_*8 + wave
        const int hw = hg_ * 8 + wave;
        if (p.gW_part && hw < H) {
            // (the flush sits inside the round loop for the change of head group; its 16 offsets and
            // masks are worked out here each time, not kept in registers across the rounds)
            int qq = q, cc = c;
            asm volatile("" : "+v"(qq), "+v"(cc));
            float *dst = p.gW_part + ((int64_t)blockIdx.x * H + hw) * D * K;
#pragma unroll
            for (int t = 0; t < NT; t++)
#pragma unroll
                for (int r = 0; r < 4; r++) {
                    const int d = 4 * qq + r, k = 16 * t + cc;
                    if (d < D && k < K) dst[(unsigned)(d * K + k)] = RINGS ? gWreg[t][r] : gw_slot[t * WAVE][r];
                }
        }
    };
    // The cube [-lattice_range, lattice_range]^3 (every unit of the fixed rule, most units of the adaptive
    // one) is decoded once: for the lane's translation of each of the first two chunks of 64, n + 8 per
    // axis in 4 bits, all in one register (unpacking costs a fifth of decoding again).
    int npre = 0;
    const int cube_T = (2 * p.lattice_range + 1) * (2 * p.lattice_range + 1) * (2 * p.lattice_range + 1);
    const bool cube_packed = !RINGS && p.lattice_range <= 7 && cube_T <= 2 * WAVE;
    if (cube_packed) {
        BoxDims b0;
        b0.U1 = b0.U2 = b0.U3 = p.lattice_range;
        b0.S3 = b0.S2 = 2 * p.lattice_range + 1;
        b0.plane = b0.S2 * b0.S3;
        b0.T = cube_T;
        b0.inv_plane = 1.0f / (float)b0.plane;
        b0.inv_S3 = 1.0f / (float)b0.S3;
#pragma unroll
        for (int ch = 0; ch < 2; ch++) {
            int n1, n2, n3;
            decode(b0, min(ch * WAVE + lane, b0.T - 1), n1, n2, n3);
            npre |= ((n1 + 8) | ((n2 + 8) << 4) | ((n3 + 8) << 8)) << (12 * ch);
        }
    }
    const int stride = gridDim.x;
    RoundPos pos = round_pos(blockIdx.x, rounds_per_hg, p.head_groups);
    RoundPos pos_next = round_pos(blockIdx.x + stride, rounds_per_hg, p.head_groups);
    UnitIds ids = unit_ids(load_unit_ids(g_pairs, unit_of(blockIdx.x, pos), lane));
    float a_cur, z_cur;
    UnitGeom geo{};
    RingImage img{};
    UnitIds ids_next;
    int col_edge = load_col_edge(blockIdx.x, pos);
    {
        float gv0 = 0.f;
        if (RINGS) img = load_ring_image(p.rings, unit_of(blockIdx.x, pos), lane);
        else gv0 = load_unit_geom(ids, lane, g_rpos, g_tvecs, UNIFORM ? nullptr : g_rvlen);
        a_cur = load_a(ids, pos);
        z_cur = load_z(ids, pos);
        const int64_t dv1 = load_unit_ids(g_pairs, unit_of(blockIdx.x + stride, pos_next), lane);
        if (!RINGS) geo = unit_geom(gv0, !UNIFORM);
        ids_next = unit_ids(dv1);
    }
    for (int rd = blockIdx.x; rd < rounds; rd += stride) {
        const int hg = pos.hg;
        const int64_t u = (int64_t)pos.r * WPB + wave;
        const bool unit_on = u < p.U;
        const RoundPos pos_next2 = round_pos(rd + 2 * stride, rounds_per_hg, p.head_groups);
        int near_cnt = 0, far_cnt = 0;
        if (RINGS) {
            // this round's image into the ring (its previous readers are done: same wavefront,
            // and the exchange's barriers lie in between), then the next round's image requested
            near_cnt = unit_on ? __builtin_amdgcn_readlane(img.hdr, 0) : 0;
            far_cnt = unit_on ? __builtin_amdgcn_readlane(img.hdr, 1) : 0;
            store_ring_image(img, ring_d2, ring_s, ring_bits, lane);
            if (near_cnt + 8 > 2 * WAVE || far_cnt > 0)          // slots 128 .. 143 (wave-uniform, rare)
                copy_ring_tail(p.rings, u, ring_d2, ring_s, ring_bits, lane);
            if (!unit_on && lane < 8) {                          // no unit: an empty near block
                ring_d2[lane] = RIMG_NEUTRAL_D2;
                ring_s[lane] = 0.f;
                ring_bits[lane] = 0;
            }
            img = load_ring_image(p.rings, unit_of(rd + stride, pos_next), lane);
        }
        // loads for the coming rounds, consumed just before this round's exchange
        float gv_next = 0.f;
        // (adaptive boxes: the lane parts of the once-a-round addresses are formed in the round, not
        // kept in registers across the rounds)
        int lane_r = lane, q_r = q, c_r = c;
        if (!UNIFORM) asm volatile("" : "+v"(lane_r), "+v"(q_r), "+v"(c_r));
        if (!RINGS) gv_next = load_unit_geom(ids_next, lane_r, g_rpos, g_tvecs, UNIFORM ? nullptr : g_rvlen);
        const float a_next = load_a(ids_next, pos_next);
        const float z_next = load_z(ids_next, pos_next);
        const int col_edge_next = load_col_edge(rd + stride, pos_next);
        if (hg != wa_hg) {
            if (wa_hg >= 0) flush_gW(wa_hg);
#pragma unroll
            for (int t = 0; t < NT; t++) {
                if (RINGS) gWreg[t] = float4_t{0.f, 0.f, 0.f, 0.f};
                else gw_slot[t * WAVE] = float4_t{0.f, 0.f, 0.f, 0.f};
            }
            wa_hg = hg;
        }
        const int64_t e_ij = ids.e_ij, e_ji = ids.e_ji;
        Cell cell;
        cell.rx = geo.rx;
        cell.ry = geo.ry;
        cell.rz = geo.rz;
#pragma unroll
        for (int x = 0; x < 9; x++) cell.t[x] = geo.t[x];

        const int h = hg * 8 + (c & 7);
        const bool col_on = unit_on && h < H && (c < 8 || e_ji != e_ij);
        const float a = col_on ? a_cur : -1.0f;
        const float a2 = a * LOG2E;
        const float z2 = col_on ? z_cur * LOG2E : 0.f;

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
        // all active columns have the cube [-lattice_range, lattice_range]^3 (wave-uniform): under
        // the adaptive rule with its floor switched on that is most units, and they skip the
        // per-column box tables and lookups
        // ... and so do units whose active columns all have the same box, whatever it is: every
        // translation of the union box then counts for every column
        bool cube = UNIFORM, same_box = UNIFORM;
        if (!UNIFORM) {
            const int lr = p.lattice_range;
            const bool other = col_on && q < 3 && Rq != Uq;
            same_box = __ballot(other) == 0ull;
            cube = same_box && bx.U1 == lr && bx.U2 == lr && bx.U3 == lr;
        }
        ColumnBoxes cbox{0, 0, 0};
        if (!same_box) cbox = column_boxes_rows(Rq, bx, lane);

        // p_t <= 2^-40 in every column when a2_weak d2 - z2_floor <= -40
        // (every row of 16 lanes holds the 16 columns, so a reduction over a row is complete)
        const float a2_weak = row16_max(col_on ? a2 : -3.0e38f);
        const float z2_floor = row16_min(col_on ? z2 : 3.0e38f);

        float4_t accS[NT], accQ[NT];
#pragma unroll
        for (int m = 0; m < NT; m++) accS[m] = accQ[m] = float4_t{0.f, 0.f, 0.f, 0.f};
        float px = 0.f;
        for (int s0 = 0; s0 < (RINGS ? 1 : T); s0 += BRING_CAP) {
            const int cnt = RINGS ? 0 : min(BRING_CAP, T - s0);
            if (!RINGS) near_cnt = far_cnt = 0;
            for (int c0 = 0; c0 < cnt; c0 += WAVE) {
                const bool valid = c0 + lane < cnt;
                int n1, n2, n3;
                if (cube && cube_packed) {                   // (wave-uniform; the cube is a single pass: s0 == 0)
                    const unsigned f = (unsigned)npre >> (c0 == 0 ? 0 : 12);
                    n1 = (int)(f & 15u) - 8;
                    n2 = (int)((f >> 4) & 15u) - 8;
                    n3 = (int)((f >> 8) & 15u) - 8;
                } else {
                    decode(bx, valid ? s0 + c0 + lane : 0, n1, n2, n3);
                }
                const float d2 = dist2(cell, (float)n1, (float)n2, (float)n3);
                int bits = 0;
                if (same_box) {
                    bits = valid ? 0xFFFF : 0;
                } else {
                    bits = column_bits(cbox, n1, n2, n3);     // all lanes take part in the lookup
                    if (!valid) bits = 0;
                }
                const int colbits = bits;
                const float s = sqrt_hw(d2) * p.s_scale;
                const float xb = s * p.inv_bin_step - 1.0f;
                if (valid) {
#pragma unroll
                    for (int m = 0; m < NT; m++)
                        if (xb >= (float)(16 * m) - p.window && xb <= (float)(16 * m + 15) + p.window)
                            bits |= (0x10000 << m);
                }
                const int tiles = bits >> 16;
                const bool is_near = valid && tiles != 0;
                const bool is_far = valid && !is_near && colbits != 0 && a2_weak * d2 - z2_floor > -40.0f;
                const unsigned long long far_mask = __ballot(is_far);
                const unsigned long long below = (1ull << lane) - 1ull;
                int pos = -1;
                int near_now;
                if (NT > 1) {
                    // near translations of the chunk ordered by the lowest tile they reach (see the
                    // forward kernel): fewer tiles per group of four, two MFMAs saved per tile here
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
                if (is_far) pos = BRING_SLOTS - 1 - (far_cnt + __popcll(far_mask & below));
                if (pos >= 0) {
                    ring_d2[pos] = d2;
                    ring_s[pos] = s;
                    ring_bits[pos] = bits;
                }
                near_cnt += near_now;
                far_cnt += __popcll(far_mask);
            }
            if (!RINGS && lane < 12) {
                const int pos = lane < 8 ? near_cnt + lane : BRING_SLOTS - far_cnt - 1 - (lane - 8);
                ring_d2[pos] = RIMG_NEUTRAL_D2;          // (finite: weight 0 and 0 * d2 = 0, as in an image)
                ring_s[pos] = 0.f;
                ring_bits[pos] = 0;
            }
            wave_mem_sync();
            if (!RINGS) {
                // the tiles any of a group's four records reaches, kept in each record (an image
                // gets them on its way into the ring): a group's records sit in adjacent lanes here
                for (int s4 = 0; s4 < near_cnt; s4 += WAVE) {
                    const bool held = s4 + lane < near_cnt + 8;      // (slots up to near_cnt + 7 hold records)
                    const int marked = with_group_reach(held ? ring_bits[s4 + lane] : 0);
                    if (held) ring_bits[s4 + lane] = marked;
                }
                wave_mem_sync();
            }
            {
                // two groups per trip, each with its own registers for the prefetched records;
                // records beyond the last group are the neutral padding
                const int groups = (near_cnt + 3) >> 2;
                struct Rec { float d2, s; int bits; };
                auto fetch = [&](int g_) -> Rec {
                    const int slot = 4 * g_ + q;
                    return Rec{ring_d2[slot], ring_s[slot], ring_bits[slot]};
                };
                // PLAIN (staged rings; boxes that are the same for all columns): every record is in every
                // column's box, the padding has a large finite d2, i.e. weight 0 and 0 * d2 = 0, and columns
                // that are switched off run with a = -1 and finite garbage that is never stored: nothing
                // to mask.
                auto group = [&](const Rec &rec, auto plain) {
                    constexpr bool PLAIN = decltype(plain)::value;
                    const bool on = PLAIN || (col_on && ((rec.bits >> c) & 1));
                    const float w = on ? exp2_hw(a2 * rec.d2 - z2) : 0.f;
                    const float wd = on ? w * rec.d2 : 0.f;
                    px += wd;
                    // tiles within reach of any of the group's 4 translations (one record per q)
                    const int reach = group_reach(rec.bits);
#pragma unroll
                    for (int m = 0; m < NT; m++) {
                        if (reach & (0x10000 << m)) {
                            float b = ck[m] - rec.s;
                            float gm = exp2_hw(-(b * b));
                            accS[m] = __builtin_amdgcn_mfma_f32_16x16x4f32(gm, w, accS[m], 0, 0, 0);
                            accQ[m] = __builtin_amdgcn_mfma_f32_16x16x4f32(gm, wd, accQ[m], 0, 0, 0);
                        }
                    }
                };
                Rec ra = fetch(0);
                if (RINGS || same_box) {
                    for (int g = 0; g < groups; g += 2) {
                        const Rec rb = fetch(g + 1);
                        group(ra, std::true_type{});
                        if (g + 1 < groups) {
                            ra = fetch(g + 2);
                            group(rb, std::true_type{});
                        }
                    }
                } else {
                    // (columns with boxes of their own: no registers to spare for the second record set)
                    for (int g = 0; g < groups; g++) {
                        const Rec rb = fetch(g + 1);
                        group(ra, std::false_type{});
                        ra = rb;
                    }
                }
            }
            {
                const int groups = (far_cnt + 3) >> 2;
                for (int g = 0; g < groups; g++) {
                    const int slot = BRING_SLOTS - 4 * (g + 1) + q;
                    const float d2t = ring_d2[slot];
                    const int bits = ring_bits[slot];
                    if (RINGS || same_box || (col_on && ((bits >> c) & 1))) px += exp2_hw(a2 * d2t - z2) * d2t;
                }
            }
            wave_mem_sync();
        }
        // the loads issued at the top of the round have landed; the descriptor of the round after
        // next is requested here and looked at after the exchange (it would otherwise occupy two
        // registers through the whole accumulation)
        UnitGeom geo_next{};
        if (!RINGS) geo_next = unit_geom(gv_next, !UNIFORM);
        const int64_t dv_next2 = load_unit_ids(g_pairs, unit_of(rd + 2 * stride, pos_next2), lane_r);
        px = rows_sum(px);

        // ---- exchange: column (dir, head) of unit `wave` -> row ((head*2 + dir)*8 + wave)
        if (q == 0) PXbuf[wave * 16 + c_r] = px;
        const int hw = hg * 8 + wave;
        const int jcol = c, unit_j = jcol & 7, dir_j = jcol >> 3;    // product column j = dir*8 + unit
        const float *src = Sbuf + xch_base(q, wave, unit_j, dir_j);
        // projection operands of this wave's head (W stays in cache across rounds)
        float Wa[4 * NT];
        if (hw < H && K == 16 * NT && D == 16) {
            // full tiles: one base address per lane, 16-byte loads at fixed offsets
            // (proj_bin(s, q) = 16 (s / 4) + 4 q + s % 4)
            // (wave-uniform base + 32-bit lane offset: no 64-bit address per lane kept across rounds)
            const float *wbase = p.W + (int64_t)hw * D * K;
            const unsigned woff = (unsigned)(c_r * K + 4 * q_r);
#pragma unroll
            for (int t4 = 0; t4 < NT; t4++) {
                const float4_t w4 = *reinterpret_cast<const float4_t *>(wbase + (woff + 16u * t4));
#pragma unroll
                for (int r = 0; r < 4; r++) Wa[4 * t4 + r] = w4[r];
            }
        } else {
            // (partial tiles: masks and offsets worked out here, not kept in registers across the rounds)
            int qq = q, cc = c;
            asm volatile("" : "+v"(qq), "+v"(cc));
#pragma unroll
            for (int s = 0; s < 4 * NT; s++) {
                const int d = cc, k = proj_bin(s, qq);
                Wa[s] = (hw < H && d < D && k < K) ? p.W[((int64_t)hw * D + d) * K + k] : 0.f;
            }
        }
        // gradient operands of this wave's head for the 16 product columns, requested before
        // the exchange so that they arrive while the columns are parked
        // (edge, head) rows are 32-bit: the launcher refuses E H >= 2^32
        const int e_out = col_edge;
        const unsigned row_out = (unsigned)col_edge * (unsigned)H + (unsigned)hw;
        float4_t gv4 = {0.f, 0.f, 0.f, 0.f};
        float gz_out = 0.f;
        float gvk[4] = {0.f, 0.f, 0.f, 0.f};
        if (hw < H) {
            if (e_out >= 0 && g_gz && q == 0) gz_out = g_gz[row_out];
            if (e_out >= 0 && g_gv) {
                const float *gp = g_gv + ((uint64_t)row_out * (unsigned)D + (unsigned)(4 * q_r));
                if (4 * q + 3 < D) {
                    gv4 = *reinterpret_cast<const float4_t *>(gp);
                } else {
#pragma unroll
                    for (int r = 0; r < 3; r++)
                        if (4 * q + r < D) gv4[r] = gp[r];
                }
            }
        }
        // With PX in hand the two projected sums collapse into one: gv.(W Q) - PX gv.(W S) =
        // gv.(W Q'), Q' = Q - PX S, formed here on the unit's own columns (px is complete in
        // every lane of a column).  One projection instead of two, and S crosses the exchange
        // only for the weight gradient.
#pragma unroll
        for (int m = 0; m < NT; m++)
#pragma unroll
            for (int r = 0; r < 4; r++) accQ[m][r] = fmaf(-px, accS[m][r], accQ[m][r]);
        if constexpr (RINGS) {
            // ---- one exchange: Q' and (for the weight gradient) S parked side by side
            const bool want_gW = p.gW_part != nullptr && g_gv != nullptr;
            {
                const int at = xch_base(q, c & 7, wave, c >> 3);
#pragma unroll
                for (int m = 0; m < NT; m++)
#pragma unroll
                    for (int r = 0; r < 4; r++) {
                        // (inactive columns hold zeros: their weights are masked in the loop)
                        Sbuf[at + (4 * m + r) * XPLANE] = accQ[m][r];
                        if (want_gW) Sbuf2[at + (4 * m + r) * XPLANE] = accS[m][r];
                    }
            }
            __syncthreads();
            {
                float4_t out = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int t4 = 0; t4 < NT; t4++) {
                    float sb[4];
#pragma unroll
                    for (int r = 0; r < 4; r++) sb[r] = src[(4 * t4 + r) * XPLANE];
#pragma unroll
                    for (int r = 0; r < 4; r++)
                        out = __builtin_amdgcn_mfma_f32_16x16x4f32(Wa[4 * t4 + r], sb[r], out, 0, 0, 0);
                }
                // lane (q, j): components d = 4q + r of W Q' for column j; dot with gv
                float dot = out[0] * gv4[0] + out[1] * gv4[1] + out[2] * gv4[2] + out[3] * gv4[3];
                dot = rows_sum(dot);
                if (q == 0 && e_out >= 0 && hw < H) {
                    const float PX = PXbuf[(c_r & 7) * 16 + (c_r >> 3) * 8 + wave];      // (unit_j, dir_j)
                    p.ga_edge[row_out] = fmaf(PX, gz_out, dot);
                }
            }
            if (want_gW) {
                // This head's gradient rows once more, transposed: lane (q, j) holds gv[column j][4q .. 4q + 3],
                // the update wants gv[column 4 s4 + q][c].  Through the wavefront's own ring, whose records
                // have been used (16 rows of 17 floats): no second fetch from memory.
                float *T = ring_d2;
#pragma unroll
                for (int r = 0; r < 4; r++) T[c * 17 + 4 * q + r] = gv4[r];
                wave_mem_sync();
                // gW_h[d][bin] += sum over the 16 columns of gv[col][d] * S[bin][col]
                // A[i = d][k = col], B[k = col][j = bin]; column 4*s4 + kk
#pragma unroll
                for (int s4 = 0; s4 < 4; s4++) {
                    const int colk = 4 * s4 + q;                    // this lane's reduction index
                    const float av = T[colk * 17 + c];
                    // bin 16 t + c of column colk: plane 4 t + c % 4, q index c / 4
                    const float *srck = Sbuf2 + (c & 3) * XPLANE + xch_base(c >> 2, wave, colk & 7, colk >> 3);
#pragma unroll
                    for (int t = 0; t < NT; t++)
                        gWreg[t] = __builtin_amdgcn_mfma_f32_16x16x4f32(av, srck[4 * t * XPLANE], gWreg[t], 0, 0, 0);
                }
            }
            __syncthreads();
        } else {
        const int passes = p.gW_part ? 2 : 1;
            for (int pass = 0; pass < passes; pass++) {
                // pass 0 exchanges Q' (projection, dot with gv, ga), pass 1 exchanges S (gW update):
                // Q' first, so that its accumulators are dead before the gW block comes in from LDS
                {
                    float *col = Sbuf + xch_base(q, c & 7, wave, c >> 3);
    #pragma unroll
                    for (int m = 0; m < NT; m++)
    #pragma unroll
                        for (int r = 0; r < 4; r++) {
                            // (inactive columns hold zeros: their weights are masked in the loop)
                            col[(4 * m + r) * XPLANE] = pass == 0 ? accQ[m][r] : accS[m][r];
                        }
                }
                __syncthreads();
                if (pass == 0) {
                    float4_t out = {0.f, 0.f, 0.f, 0.f};
    #pragma unroll
                    for (int t4 = 0; t4 < NT; t4++) {
                        float sb[4];
    #pragma unroll
                        for (int r = 0; r < 4; r++) sb[r] = src[(4 * t4 + r) * XPLANE];
    #pragma unroll
                        for (int r = 0; r < 4; r++)
                            out = __builtin_amdgcn_mfma_f32_16x16x4f32(Wa[4 * t4 + r], sb[r], out, 0, 0, 0);
                    }
                    // lane (q, j): components d = 4q + r of W Q' for column j; dot with gv
                    float dot = out[0] * gv4[0] + out[1] * gv4[1] + out[2] * gv4[2] + out[3] * gv4[3];
                    dot = rows_sum(dot);
                    if (q == 0 && e_out >= 0 && hw < H) {
                        const float PX = PXbuf[(c_r & 7) * 16 + (c_r >> 3) * 8 + wave];      // (unit_j, dir_j)
                        p.ga_edge[row_out] = fmaf(PX, gz_out, dot);
                    }
                    // operands of the gW update of the next pass, requested now so that they arrive
                    // while S is being exchanged
                    if (hw < H && p.gW_part && g_gv) {
    #pragma unroll
                        for (int s4 = 0; s4 < 4; s4++) {
                            const int e_k = __builtin_amdgcn_ds_bpermute((4 * s4 + q) << 2, col_edge);   // column 4*s4 + q
                            const unsigned row_k = (unsigned)e_k * (unsigned)H + (unsigned)hw;
                            if (e_k >= 0 && c < D) gvk[s4] = g_gv[(uint64_t)row_k * (unsigned)D + (unsigned)c_r];
                        }
                    }
                } else {
                    // gW_h[d][bin] += sum over the 16 columns of gv[col][d] * S[bin][col]
                    // A[i = d][k = col], B[k = col][j = bin]; column 4*s4 + kk
                    float4_t gWacc[NT];
    #pragma unroll
                    for (int t = 0; t < NT; t++) gWacc[t] = gw_slot[t * WAVE];
    #pragma unroll
                    for (int s4 = 0; s4 < 4; s4++) {
                        const int colk = 4 * s4 + q;                    // this lane's reduction index
                        const float av = gvk[s4];
                        // bin 16 t + c of column colk: plane 4 t + c % 4, q index c / 4
                        const float *srck = Sbuf + (c & 3) * XPLANE + xch_base(c >> 2, wave, colk & 7, colk >> 3);
    #pragma unroll
                        for (int t = 0; t < NT; t++)
                            gWacc[t] = __builtin_amdgcn_mfma_f32_16x16x4f32(av, srck[4 * t * XPLANE], gWacc[t], 0, 0, 0);
                    }
    #pragma unroll
                    for (int t = 0; t < NT; t++) gw_slot[t * WAVE] = gWacc[t];
                }
                __syncthreads();
            }
        }
        ids = ids_next;
        geo = geo_next;
        a_cur = a_next;
        z_cur = z_next;
        ids_next = unit_ids(dv_next2);
        col_edge = col_edge_next;
        pos = pos_next;
        pos_next = pos_next2;
    }
    if (wa_hg >= 0) flush_gW(wa_hg);
}

// The two reductions behind the pair kernel in one launch (they are independent, and a launch
// costs more than either): work-groups below gw_groups fold the per-work-group partial weight
// gradients, the others fold the per-edge exponent gradients into per-atom ones.
//
// gW[x] = sum over work-groups of part[b][x], fixed order.  A work-group of 256 threads takes
// 32 consecutive elements; 8 groups of threads each sum every 8th block (two running sums),
// and the 8 partial results are added in order through LDS.
//
// ga[i,h] = sum over the edge row of atom i of ga_edge[e,h]: one thread per (i,h), eight
// running sums over the row in order.
__global__ __launch_bounds__(256) void bwd_reductions_kernel(const float *part, int blocks, int64_t HDK, float *gW,
                                                             int gw_groups, const float *ga_edge,
                                                             const int64_t *e_start, int64_t N, int H, float *ga)
{
    __shared__ float red[8][32];
    if ((int)blockIdx.x >= gw_groups) {
        const int64_t tid = (int64_t)(blockIdx.x - gw_groups) * 256 + threadIdx.x;
        if (tid >= N * H) return;
        const int64_t i = tid / H;
        const int h = (int)(tid - i * H);
        const int64_t e0 = e_start[i], e1 = e_start[i + 1];
        float acc[8] = {0, 0, 0, 0, 0, 0, 0, 0};
        int64_t e = e0;
        for (; e + 8 <= e1; e += 8)
#pragma unroll
            for (int u = 0; u < 8; u++) acc[u] += ga_edge[(e + u) * H + h];
        for (int u = 0; e < e1; e++, u++) acc[u] += ga_edge[e * H + h];
        ga[tid] = ((acc[0] + acc[1]) + (acc[2] + acc[3])) + ((acc[4] + acc[5]) + (acc[6] + acc[7]));
        return;
    }
    const int ex = threadIdx.x & 31, pt = threadIdx.x >> 5;
    const int64_t x = (int64_t)blockIdx.x * 32 + ex;
    float acc0 = 0.f, acc1 = 0.f;
    if (x < HDK) {
        int b = pt;
        // 8 loads in flight per thread; the two running sums take alternate blocks
        for (; b + 56 < blocks; b += 64) {
            float v[8];
#pragma unroll
            for (int u = 0; u < 8; u++) v[u] = part[(int64_t)(b + 8 * u) * HDK + x];
#pragma unroll
            for (int u = 0; u < 8; u += 2) {
                acc0 += v[u];
                acc1 += v[u + 1];
            }
        }
        for (; b + 8 < blocks; b += 16) {
            acc0 += part[(int64_t)b * HDK + x];
            acc1 += part[(int64_t)(b + 8) * HDK + x];
        }
        if (b < blocks) acc0 += part[(int64_t)b * HDK + x];
    }
    red[pt][ex] = acc0 + acc1;
    __syncthreads();
    if (pt == 0 && x < HDK) {
        float total = red[0][ex];
#pragma unroll
        for (int g = 1; g < 8; g++) total += red[g][ex];
        gW[x] = total;
    }
}

}  // namespace

namespace cf {

int real_enc_bwd_pairs_blocks(int64_t U, int64_t H)
{
    const int64_t rounds = ((U + WPB - 1) / WPB) * ((H + 7) / 8);
    int64_t blocks = rounds;
    const int64_t cap = (int64_t)device_cu_count() * 2;
    if (blocks > cap) blocks = cap;
    return (int)(blocks < 1 ? 1 : blocks);
}

// Returns CF_ERR_UNSUPPORTED (no error text) for shapes this kernel does not cover.
int launch_real_enc_bwd_pairs(const float *a_ik, const float *rpos, const float *tvecs, const int64_t *batch,
                              const int64_t *edges, const int64_t *pairs, int64_t U, const float *z,
                              const float *gz, const float *gv, int64_t N, int64_t H, int64_t E, int64_t K,
                              int64_t D, float bin_step, float s_scale, const float *W, const float *rvlen,
                              float cutoff, int lattice_range, int min_range, float *ga_edge,
                              float *gW_part, float *gW, const int64_t *e_start, float *ga_ik,
                              const float *rings, hipStream_t st)
{
    if (K < 1 || K > 64 || !W || D < 1 || D > 16) return CF_ERR_UNSUPPORTED;
    PairArgs p{};
    p.a_ik = a_ik; p.rpos = rpos; p.tvecs = tvecs; p.batch = batch; p.edges = edges; p.pairs = pairs;
    p.W = W; p.rvlen = rvlen; p.z_in = z; p.gz = gz; p.gv = gv; p.ga_edge = ga_edge; p.gW_part = gW_part;
    p.N = N; p.E = E; p.U = U; p.W_num = 1;
    p.H = (int)H; p.K = (int)K; p.D = (int)D;
    p.head_groups = (int)((H + 7) / 8);
    p.cutoff = cutoff; p.lattice_range = lattice_range; p.min_range = min_range;
    p.bin_step = bin_step; p.s_scale = s_scale;
    p.inv_bin_step = 1.0f / bin_step;
    p.window = sqrtf(40.0f) / bin_step;
    const int NT = K <= 16 ? 1 : K <= 32 ? 2 : 4;
    const bool uniform = cutoff == 0.0f;
    const int side = 2 * lattice_range + 1;
    if (rings && (!uniform || side * side * side > RIMG_CAP)) rings = nullptr;     // not what rings are staged for
    p.rings = rings;
    // rings, exchange buffer, PX, and either the gW slots or (from staged rings) a second exchange buffer
    const size_t gw_words = (size_t)WPB * NT * WAVE * 4, xch_words = (size_t)4 * NT * XPLANE;
    const size_t lds = sizeof(float) * ((size_t)WPB * 3 * BRING_SLOTS + xch_words + WPB * 16 +
                                        (rings ? xch_words : gw_words)) + 16;
    if (((U + WPB - 1) / WPB) * ((H + 7) / 8) >= (1ll << 30)) return CF_ERR_UNSUPPORTED;   // 32-bit round positions
    if (E >= (1ll << 31) || E * H >= (1ll << 32) || N * H >= (1ll << 32)) return CF_ERR_UNSUPPORTED;   // 32-bit ids, rows
    const int blocks = real_enc_bwd_pairs_blocks(U, H);
#define CF_BPAIR(NTV)                                                                              \
    do {                                                                                           \
        if (rings) real_enc_bwd_pair_kernel<NTV, true, true><<<blocks, WPB * WAVE, lds, st>>>(p);          \
        else if (uniform) real_enc_bwd_pair_kernel<NTV, true, false><<<blocks, WPB * WAVE, lds, st>>>(p);  \
        else real_enc_bwd_pair_kernel<NTV, false, false><<<blocks, WPB * WAVE, lds, st>>>(p);              \
    } while (0)
    switch (NT) {
        case 1: CF_BPAIR(1); break;
        case 2: CF_BPAIR(2); break;
        default: CF_BPAIR(4); break;
    }
#undef CF_BPAIR
    {
        const int64_t HDK = (gW_part && gW) ? H * D * K : 0;
        const int gw_groups = (int)((HDK + 31) / 32);
        const int64_t ga_groups = (N * H + 255) / 256;
        bwd_reductions_kernel<<<(int)(gw_groups + ga_groups), 256, 0, st>>>(gW_part, blocks, HDK, gW, gw_groups, ga_edge,
                                                                            e_start, N, (int)H, ga_ik);
    }
    return CF_OK;
}

}  // namespace cf
