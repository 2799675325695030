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
#include "real_enc_pair_fwd.h"

namespace {

using namespace cf;
using namespace cfpair;

template <int NT, bool UNIFORM, int PROJ, int DT, bool SHORT_RING>
__global__ __launch_bounds__(512, 4) void real_enc_fwd_pair_kernel(PairArgs p_)
{
    const PairArgs p = with_live_units(p_);
    if (p.U == 0) return;          // (an empty list: not even the descriptor of unit 0 may be read)
    // (p_ is the kernel's first argument: it lies at the start of the kernel-argument segment)
    const cfpair::PairArgsSeg seg = (cfpair::PairArgsSeg)__builtin_amdgcn_kernarg_segment_ptr();
    real_enc_fwd_pair_body<NT, UNIFORM, PROJ, DT, SHORT_RING>(p, seg, (int)blockIdx.x, (int)gridDim.x);
}

// Unit descriptors: the (i <= j) edges of every crystal's dense block, their reverses,
// the two atoms and the crystal.
__global__ void edge_pairs_kernel(const int64_t *atom_start, const int64_t *edge_start,
                                  const int64_t *unit_start, int64_t B, int64_t E, const int64_t *live_E,
                                  int64_t *pairs)
{
    int64_t e = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (e >= live_count(live_E, E)) return;
    const EdgeEnds r = edge_ends(atom_start, edge_start, B, e);
    const int64_t u = unit_of_edge(r, unit_start[r.crystal]);
    if (u < 0) return;                    // (i > j: the reverse edge owns the unit)
    int64_t *d = pairs + PAIR_FIELDS * u;
    d[0] = e;
    d[1] = reverse_edge(r);
    d[2] = r.i;
    d[3] = r.j;
    d[4] = r.crystal;
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
                              int min_range, unsigned int *sched, const int *order, const int64_t *counts,
                              float *z, float *v, hipStream_t st)
{
    if (K < 0 || K > 128) return CF_ERR_UNSUPPORTED;
    if (W && (D < 1 || D > 64)) return CF_ERR_UNSUPPORTED;
    PairArgs p{};
    p.a_ik = a_ik; p.rpos = rpos; p.tvecs = tvecs; p.batch = batch; p.edges = edges; p.pairs = pairs;
    p.W = W; p.rvlen = rvlen; p.z = z; p.v = v; p.sched = sched;
    p.N = N; p.E = E; p.U = U; p.W_num = W_num;
    p.H = (int)H; p.K = (int)K; p.D = (int)D;
    p.head_groups = (int)((H + 7) / 8);
    p.cutoff = cutoff; p.lattice_range = lattice_range; p.min_range = min_range;
    p.bin_step = bin_step; p.s_scale = s_scale;
    p.inv_bin_step = 1.0f / bin_step;
    p.window = sqrtf(40.0f) / bin_step;                 // exp2(-(bin_step*x)^2) < 2^-40 beyond it
    if (K == 0) {
        // bias only: no bins, so no translation is ever "near"; all of them feed the column sums
        p.bin_step = p.s_scale = p.inv_bin_step = 0.f;
        p.window = -1.0e30f;
    }
    const int NT = K <= 16 ? 1 : K <= 32 ? 2 : K <= 64 ? 4 : 8;
    const bool uniform = cutoff == 0.0f;
    int mode = PROJ_NONE;
    if (W) mode = (W_num == 1) ? PROJ_SHARED : PROJ_INDEXED;
    if (mode == PROJ_SHARED && D > 32) return CF_ERR_UNSUPPORTED;
    const int DT = (mode == PROJ_SHARED && D > 16) ? 2 : 1;
    // a fixed cube that fits one pass of the short ring
    const int64_t cube = (int64_t)(2 * lattice_range + 1) * (2 * lattice_range + 1) * (2 * lattice_range + 1);
    const bool short_ring = uniform && cube <= RING_CAP_SMALL;
    size_t lds = sizeof(float) * (size_t)WPB * 3 * ((short_ring ? RING_CAP_SMALL : RING_CAP) + 16);
    if (mode == PROJ_SHARED)
        lds += sizeof(float) * (size_t)4 * NT * XPLANE + sizeof(int64_t) * WPB * 2 + sizeof(float) * WPB * 16 + 8;
    const int64_t rounds = ((U + WPB - 1) / WPB) * p.head_groups;
    if (rounds >= (1ll << 30)) return CF_ERR_UNSUPPORTED;   // round positions are 32-bit in the kernel
    int64_t blocks = rounds;
    int64_t cap = persistent_grid_cap(2);              // 16 waves per CU, times the launch share
    if (blocks > cap) blocks = cap;
    if (blocks < 1) return CF_OK;
    // A ticket is drawn three rounds before it is executed (descriptor, then geometry, each
    // fetched a round ahead), so with few rounds per work-group the draw is as good as fixed
    // and the fixed stride, which costs nothing, does better (measured: 64.5 against 70 us at
    // 7 rounds per work-group; 1.66 against 1.81 ms at 217).
    if (rounds < 16 * blocks) p.sched = nullptr;
    p.live_U = live_units(U);
    if (order) {
        // the second of two lists of units (the first runs from the staged rings): counts[1] units
        // from slot counts[0] on; how many rounds that makes is not known here, so no tickets
        p.order = order;
        p.order_first = counts;
        p.live_U = counts + 1;
        p.sched = nullptr;
    }
#define CF_PAIR(NTV, UNI, PRJ, DTV, SR) \
    real_enc_fwd_pair_kernel<NTV, UNI, PRJ, DTV, SR><<<(int)blocks, WPB * WAVE, lds, st>>>(p)
#define CF_PAIR_MODE(NTV, UNI, SR)                                            \
    do {                                                                      \
        if (mode == PROJ_NONE) CF_PAIR(NTV, UNI, PROJ_NONE, 1, SR);           \
        else if (mode == PROJ_INDEXED) CF_PAIR(NTV, UNI, PROJ_INDEXED, 1, SR); \
        else if (DT == 1) CF_PAIR(NTV, UNI, PROJ_SHARED, 1, SR);              \
        else CF_PAIR(NTV, UNI, PROJ_SHARED, 2, SR);                           \
    } while (0)
#define CF_PAIR_NT(NTV)                                     \
    do {                                                    \
        if (short_ring) CF_PAIR_MODE(NTV, true, true);      \
        else if (uniform) CF_PAIR_MODE(NTV, true, false);   \
        else CF_PAIR_MODE(NTV, false, false);               \
    } while (0)
    switch (NT) {
        case 1: CF_PAIR_NT(1); break;
        case 2: CF_PAIR_NT(2); break;
        case 4: CF_PAIR_NT(4); break;
        default: CF_PAIR_NT(8); break;
    }
#undef CF_PAIR_NT
#undef CF_PAIR_MODE
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
                                                                              unit_start_n, B, E, cf::live_edges(E),
                                                                              pairs_u);
    CF_CHECK_LAUNCH("cf_edge_pairs");
    return CF_OK;
}
