// Shared pieces of the pair-evaluated periodic-encoding kernels (forward and
// backward): argument block, translation geometry, box decoding.
#pragma once

#include "cf_common.h"

namespace cfpair {

using namespace cf;

typedef float float4_t __attribute__((ext_vector_type(4)));

struct PairArgs {
    const float *a_ik;
    const float *rpos;
    const float *tvecs;
    const int64_t *batch;
    const int64_t *edges;
    const int64_t *pairs;   // (U,5): edge (i->j) with i <= j, its reverse, atoms i and j, crystal
    const float *W;
    const float *rvlen;
    float *z;
    float *v;
    unsigned int *sched;    // forward only, nullable: {next ticket, finished work-groups}, both 0 at launch
    // backward only
    const float *z_in;      // (E,H) forward output
    const float *gz;        // (E,H), nullable
    const float *gv;        // (E,H,D), nullable
    float *ga_edge;         // (E,H) per-edge contributions to ga
    float *gW_part;         // (grid, H, D, K) per-work-group partial sums of gW, nullable
    int64_t N, E, U;
    int64_t W_num;
    int H, K, D;
    int head_groups;        // ceil(H / 8)
    float cutoff;
    int lattice_range, min_range;
    float bin_step, s_scale;
    float inv_bin_step;     // distance argument -> fractional bin coordinate
    float window;           // bins beyond which a Gaussian is below 2^-40 and is not evaluated
    const float *rings;     // staged translations of every unit (RIMG_WORDS each), nullable
    // Order of the units, nullable: slot -> unit (8 r + w is the slot of wavefront w in round r; without
    // an order slot and unit are the same).  Adaptive boxes from staged rings split the units in two
    // stably ordered sets this way -- those whose columns all keep the cube, then the others -- and
    // give each set to its own launch: order_first (device, nullable) is the slot in `order` where
    // this launch's units begin, live_U how many there are.
    const int *order;
    const int64_t *order_first;
    // Live unit count on the device, nullable (forward and staging kernels): U is then the capacity
    // of the unit list -- what the grid and the buffers are sized for -- and the kernel walks the
    // first *live_U units only.
    const int64_t *live_U;
};

#if defined(__HIPCC__)
// The arguments a kernel body works with: U replaced by the live count when there is one.
__device__ __forceinline__ PairArgs with_live_units(const PairArgs &p)
{
    PairArgs q = p;
    q.U = live_count(p.live_U, p.U);
    if (p.order && p.order_first) q.order = p.order + live_count(p.order_first, p.U);
    return q;
}
#endif

// The arguments where the launch put them, in the kernel-argument segment.  A pointer that a
// kernel uses once a round is read from there when it is needed (a scalar load that hits the
// constant cache) instead of occupying two scalar registers through the whole kernel: the pair
// kernels need more scalar registers than there are, and every value the compiler parks in a
// vector register's lanes costs a vector instruction to get back.
typedef const PairArgs __attribute__((address_space(4))) *PairArgsSeg;

// (the reads through the returned pointer stay behind this point and are not kept across rounds)
__device__ __forceinline__ PairArgsSeg reread(PairArgsSeg seg)
{
    int off = 0;
    asm volatile("" : "+s"(off));
    return reinterpret_cast<PairArgsSeg>(reinterpret_cast<const char __attribute__((address_space(4))) *>(seg) + off);
}

// A pointer field of the segment, read as a 64-bit word (hipcc of ROCm 7.2 stops with an internal
// error on a lane-dependent choice between pointers that were loaded as pointers from there).
template <typename T>
__device__ __forceinline__ T *seg_pointer(T *const __attribute__((address_space(4))) *field)
{
    typedef const unsigned long long __attribute__((address_space(4))) *Word;
    return reinterpret_cast<T *>(*reinterpret_cast<Word>(field));
}

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

// Box geometry of one unit (wave-uniform).
struct BoxDims {
    int U1, U2, U3, S2, S3, plane, T;
    float inv_plane, inv_S3;
};

// idx -> (n1,n2,n3), first index slowest; float reciprocals with one correction
// step instead of integer division (idx < 2^21).
__device__ __forceinline__ void decode(const BoxDims &bx, int idx, int &n1, int &n2, int &n3)
{
    int q1 = (int)(((float)idx + 0.5f) * bx.inv_plane);
    int rem = idx - q1 * bx.plane;
    if (rem < 0) { q1--; rem += bx.plane; }
    if (rem >= bx.plane) { q1++; rem -= bx.plane; }
    int q2 = (int)(((float)rem + 0.5f) * bx.inv_S3);
    int r3 = rem - q2 * bx.S3;
    if (r3 < 0) { q2--; r3 += bx.S3; }
    if (r3 >= bx.S3) { q2++; r3 -= bx.S3; }
    n1 = q1 - bx.U1;
    n2 = q2 - bx.U2;
    n3 = r3 - bx.U3;
}

__device__ __forceinline__ int wave_max_int(int v) { return wave_max_i(v); }

// ---- per-column boxes --------------------------------------------------------
// Under the adaptive rule the 16 columns of a unit have their own half-widths
// (R1,R2,R3 in lanes 0..15).  Lane r of the tables holds, for |n| = r + 1 along one
// axis, the set of columns whose box reaches that far; |n| = 0 is inside every box.
struct ColumnBoxes { int m1, m2, m3; };

__device__ __forceinline__ int axis_table(int R, int U, int lane)
{
    int m = 0;
    for (int r = 1; r <= U; r++) {       // U is wave-uniform
        const int mask = (int)(__ballot(R >= r) & 0xFFFFull);
        m = (lane == r - 1) ? mask : m;
    }
    return m;
}

__device__ __forceinline__ ColumnBoxes column_boxes(int R1, int R2, int R3, const BoxDims &bx, int lane)
{
    ColumnBoxes cb;
    cb.m1 = axis_table(R1, bx.U1, lane);
    cb.m2 = axis_table(R2, bx.U2, lane);
    cb.m3 = axis_table(R3, bx.U3, lane);
    return cb;
}

// The same tables from half-widths laid out one axis per row of 16 lanes (lane 16 q + c: axis q of
// column c; 0 in row 3): one ballot per |n| serves the three axes.
__device__ __forceinline__ ColumnBoxes column_boxes_rows(int Rq, const BoxDims &bx, int lane)
{
    ColumnBoxes cb{0, 0, 0};
    const int top = max(bx.U1, max(bx.U2, bx.U3));       // wave-uniform
    for (int r = 1; r <= top; r++) {
        const unsigned long long m = __ballot(Rq >= r);
        const bool mine = lane == r - 1;
        cb.m1 = mine ? (int)(m & 0xFFFFull) : cb.m1;
        cb.m2 = mine ? (int)((m >> 16) & 0xFFFFull) : cb.m2;
        cb.m3 = mine ? (int)((m >> 32) & 0xFFFFull) : cb.m3;
    }
    return cb;
}

// Half-width of column c along axis q for the lanes of row q < 3 (0 in row 3 and for columns that
// are off): cf::range_rule, one axis per lane instead of three.
__device__ __forceinline__ int column_axis_range(float a, float cutoff, const float *rvl, int lattice_range,
                                                 int minimum_range, int q, bool col_on)
{
    int R = lattice_range;
    if (cutoff != 0.0f) {
        const float rv = q == 0 ? rvl[0] : (q == 1 ? rvl[1] : rvl[2]);
        const bool counts = col_on && q < 3;
        if (cutoff < 0.0f) {
            // First with the one-ulp reciprocal and square root: the quotient that is rounded up
            // comes out within 1e-6 of the exact rule's (relative), so unless it lies within 1e-4
            // of a whole number (or is not finite, not below 1e6) both give the same half-width.
            const float cut = __builtin_amdgcn_sqrtf(-0.5f * __builtin_amdgcn_rcpf(a)) * (-cutoff);
            const float qf = (cut + 0.01f) * rv * (float)(1.0 / (2.0 * (double)PI_F));
            const bool clear = fabsf(qf - rintf(qf)) > 1.0e-4f * fmaxf(fabsf(qf), 1.0f) && fabsf(qf) < 1.0e6f;
            if (__ballot(counts && !clear) == 0ull) {             // (wave-uniform; nearly always)
                const float up = ceilf(qf);
                const int r = up <= 0.f ? 0 : (up > (float)MAX_RANGE ? MAX_RANGE : (int)up);
                return counts ? max(r, minimum_range) : 0;
            }
            cutoff = sqrtf(-0.5f / a) * (-cutoff);
        }
        R = range_axis(cutoff, rv, minimum_range);
    }
    return (col_on && q < 3) ? R : 0;
}

// columns whose box contains translation (n1,n2,n3); |n| <= 64 on every axis
__device__ __forceinline__ int column_bits(const ColumnBoxes &cb, int n1, int n2, int n3)
{
    const int a1 = abs(n1), a2 = abs(n2), a3 = abs(n3);
    int b1 = __shfl(cb.m1, max(a1 - 1, 0), WAVE);
    int b2 = __shfl(cb.m2, max(a2 - 1, 0), WAVE);
    int b3 = __shfl(cb.m3, max(a3 - 1, 0), WAVE);
    b1 = a1 == 0 ? 0xFFFF : b1;
    b2 = a2 == 0 ? 0xFFFF : b2;
    b3 = a3 == 0 ? 0xFFFF : b3;
    return b1 & b2 & b3;
}

constexpr int WPB = 8;                   // wavefronts per work-group = units per round
constexpr int PAIR_FIELDS = 5;           // words per unit descriptor: e_ij, e_ji, i, j, crystal

// Exchange buffer of the shared-projection epilogues (forward and backward): the column sums a
// wavefront holds for its unit are parked in LDS and read back by the wavefront that owns a head.
// Element (bin = 16 m + 4 q + r, unit, column = 8 dir + head) lives at
//     (4 m + r) * XPLANE + dir * 256 + unit * 32 + ((8 q + head) ^ unit).
// A writer (one unit; lanes over q, dir, head), a reader (one head; lanes over q, dir, unit) and
// the reader of the weight-gradient update (one head; lanes over 16 consecutive bins and 4
// consecutive columns) all spread over the 32 banks with two lanes per bank, the least 64
// lanes can do; a plain [column][bin] array puts four lanes on a bank on both sides, and the LDS
// port is shared by the 16 wavefronts of a CU.
constexpr int XPLANE = 516;
__device__ __forceinline__ int xch_base(int q, int head, int unit, int dir)
{
    return dir * 256 + unit * 32 + ((8 * q + head) ^ unit);
}

// Position of a round: head group and round index inside it.  32-bit; the launchers
// refuse work with 2^30 rounds or more.  One head group (H <= 8) needs no division.
struct RoundPos { int hg, r; };

__device__ __forceinline__ RoundPos round_pos(int rd, int rounds_per_hg, int head_groups)
{
    RoundPos x;
    if (head_groups == 1) {
        x.hg = 0;
        x.r = rd;
    } else {
        x.hg = rd / rounds_per_hg;
        x.r = rd - x.hg * rounds_per_hg;
    }
    return x;
}

// order[slot] as a scalar load (slot is wave-uniform; the order was written by an earlier launch)
__device__ __forceinline__ int ordered_unit(const int *order, int slot)
{
    typedef const int __attribute__((address_space(4))) *ConstInt;
    return ((ConstInt)order)[slot];
}

// ---- unit descriptors --------------------------------------------------------
// Everything a round needs about its unit is fetched with per-lane vector loads
// one or two rounds ahead and turned into wave-uniform values with readlane just
// before the epilogue of the round in flight: the dependent chain
// descriptor -> (p_j - p_i, lattice, exponents) never sits in front of compute,
// and the waits land where the loads are a whole round old.
struct UnitIds { int64_t e_ij, e_ji, i, j, n; };
struct UnitGeom { float rx, ry, rz, t[9], rvl[3]; };

__device__ __forceinline__ int64_t readlane_i64(int64_t v, int l)
{
    const int lo = __builtin_amdgcn_readlane((int)(v & 0xffffffffll), l);
    const int hi = __builtin_amdgcn_readlane((int)(v >> 32), l);
    return ((int64_t)hi << 32) | (int64_t)(unsigned int)lo;
}

// pins a wave-uniform value in a scalar register at this point of the program
__device__ __forceinline__ float pin_uniform(float v)
{
    int x = __float_as_int(v);
    asm volatile("" : "+s"(x));
    return __int_as_float(x);
}
__device__ __forceinline__ int64_t pin_uniform(int64_t v)
{
    asm volatile("" : "+s"(v));
    return v;
}

// lanes 0..4 receive the five descriptor words of unit u
__device__ __forceinline__ int64_t load_unit_ids(const int64_t *__restrict__ pairs, int64_t u, int lane)
{
    return pairs[u * PAIR_FIELDS + min(lane, PAIR_FIELDS - 1)];
}

__device__ __forceinline__ UnitIds unit_ids(int64_t dv)
{
    UnitIds d;
    d.e_ij = pin_uniform(readlane_i64(dv, 0));
    d.e_ji = pin_uniform(readlane_i64(dv, 1));
    d.i = pin_uniform(readlane_i64(dv, 2));
    d.j = pin_uniform(readlane_i64(dv, 3));
    d.n = pin_uniform(readlane_i64(dv, 4));
    return d;
}

// lanes 0..2: p_j - p_i of the edge, 3..11: lattice rows, 12..14: reciprocal lengths
__device__ __forceinline__ float load_unit_geom(const UnitIds &d, int lane, const float *__restrict__ rpos,
                                                const float *__restrict__ tvecs,
                                                const float *__restrict__ rvlen)
{
    const int l = min(lane, rvlen ? 14 : 11);
    const float *src = l < 3 ? rpos + d.e_ij * 3 + l
                     : l < 12 ? tvecs + d.n * 9 + (l - 3)
                              : rvlen + d.n * 3 + (l - 12);
    return *src;
}

__device__ __forceinline__ UnitGeom unit_geom(float gv, bool with_rvlen)
{
    UnitGeom g;
    g.rx = pin_uniform(readlane_f(gv, 0));
    g.ry = pin_uniform(readlane_f(gv, 1));
    g.rz = pin_uniform(readlane_f(gv, 2));
#pragma unroll
    for (int x = 0; x < 9; x++) g.t[x] = pin_uniform(readlane_f(gv, 3 + x));
#pragma unroll
    for (int x = 0; x < 3; x++) g.rvl[x] = with_rvlen ? pin_uniform(readlane_f(gv, 12 + x)) : 0.f;
    return g;
}

// Bin handled by reduction step s (0..4*NT-1) and sub-lane kk (0..3) of the projection:
// chosen so that a lane's 4 consecutive steps read 4 consecutive bins.
__device__ __forceinline__ int proj_bin(int s, int kk) { return 16 * (s >> 2) + 4 * kk + (s & 3); }

// ---- staged rings in memory ---------------------------------------------------
// Image of a unit's staged translations (fixed cube of at most RIMG_CAP translations), RIMG_WORDS
// 32-bit words: d2[RIMG_SLOTS], s[RIMG_SLOTS], bits[RIMG_SLOTS], header {near count, far count,
// smallest d2, -}.  Near records occupy slots 0 .. near-1 followed by 8 neutral records
// (d2 = RIMG_NEUTRAL_D2, no bits); far records occupy slots RIMG_SLOTS-1 downwards followed (below) by 4
// neutral records.
constexpr int RIMG_CAP = 128;
constexpr int RIMG_SLOTS = RIMG_CAP + 16;
constexpr int RIMG_WORDS = 3 * RIMG_SLOTS + 4;

// d2 of a neutral record of an image: large and finite, so that a weight exp(a d2) is 0 for every
// exponent and 0 * d2 is 0 too (no masking of the padding in the loops that run from an image)
constexpr float RIMG_NEUTRAL_D2 = 1e30f;

// slots lane and 64 + lane of the three arrays, and the header word min(lane, 3)
struct RingImage { float d2[2], s[2]; int bits[2]; int hdr; };

__device__ __forceinline__ RingImage load_ring_image(const float *__restrict__ rings, int64_t u, int lane)
{
    const float *base = rings + u * RIMG_WORDS;
    RingImage im;
#pragma unroll
    for (int k = 0; k < 2; k++) {
        im.d2[k] = base[k * WAVE + lane];
        im.s[k] = base[RIMG_SLOTS + k * WAVE + lane];
        im.bits[k] = __float_as_int(base[2 * RIMG_SLOTS + k * WAVE + lane]);
    }
    im.hdr = __float_as_int(base[3 * RIMG_SLOTS + min(lane, 3)]);
    return im;
}

// The accumulation takes four consecutive slots at a time and needs the tiles any of the four
// reaches as one wave-uniform value.  The four records sit in four adjacent lanes here (a quad), so
// the union is formed on the way into LDS (two quad swaps) and kept in bits 24..31 of each record:
// the loop then reads it from any lane instead of collecting four records' bits.
__device__ __forceinline__ int with_group_reach(int bits)
{
    int t = (bits >> 16) & 0xFF;
    t |= dpp_i<DPP_QUAD_1032, 0xF>(t, t);
    t |= dpp_i<DPP_QUAD_2301, 0xF>(t, t);
    return bits | (t << 24);
}
// tiles within reach of the group of a record read back from the ring (wave-uniform, tile m at bit 16 + m)
__device__ __forceinline__ int group_reach(int bits) { return __builtin_amdgcn_readfirstlane(bits) >> 8; }

__device__ __forceinline__ void store_ring_image(const RingImage &im, float *ring_d2, float *ring_s, int *ring_bits,
                                                 int lane)
{
#pragma unroll
    for (int k = 0; k < 2; k++) {
        ring_d2[k * WAVE + lane] = im.d2[k];
        ring_s[k * WAVE + lane] = im.s[k];
        ring_bits[k * WAVE + lane] = with_group_reach(im.bits[k]);
    }
}

// slots 2*WAVE .. RIMG_SLOTS-1: the end of a full near block and the far block
__device__ __forceinline__ void copy_ring_tail(const float *__restrict__ rings, int64_t u, float *ring_d2,
                                               float *ring_s, int *ring_bits, int lane)
{
    if (lane < RIMG_SLOTS - 2 * WAVE) {
        const float *base = rings + u * RIMG_WORDS;
        ring_d2[2 * WAVE + lane] = base[2 * WAVE + lane];
        ring_s[2 * WAVE + lane] = base[RIMG_SLOTS + 2 * WAVE + lane];
        ring_bits[2 * WAVE + lane] = with_group_reach(__float_as_int(base[2 * RIMG_SLOTS + 2 * WAVE + lane]));
    }
}

}  // namespace cfpair
