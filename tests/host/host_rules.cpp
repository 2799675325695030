// Host build of the integer / range arithmetic the device kernels use (csrc/cf_index_rules.h), behind a
// C interface for the CPU tests: the same source the kernels compile, run by the host compiler so that
// it can be checked value by value against the CPU oracle and run under AddressSanitizer / UBSan.
// Test infrastructure: nothing in the product loads this.
#define CF_HOST_BUILD 1
#include "../../crystalformer_amd/csrc/cf_index_rules.h"

extern "C" {

int host_max_range(void) { return cf::MAX_RANGE; }

// R_out (N,H,3): cf::range_rule per (atom, head), as translation_ranges_kernel applies it
void host_translation_ranges(const float *a_ik, const float *rvlen_n, const int64_t *batch_i, int64_t N, int64_t H,
                             double cutoff_radius, int lattice_range, int minimum_range, int32_t *R_out)
{
    static const float zero3[3] = {0.f, 0.f, 0.f};
    for (int64_t i = 0; i < N; i++)
        for (int64_t h = 0; h < H; h++) {
            const float *rvl = rvlen_n ? rvlen_n + batch_i[i] * 3 : zero3;
            int R1, R2, R3;
            cf::range_rule(a_ik[i * H + h], rvlen_n ? (float)cutoff_radius : 0.0f, rvl, lattice_range,
                           minimum_range, R1, R2, R3);
            int32_t *o = R_out + (i * H + h) * 3;
            o[0] = R1; o[1] = R2; o[2] = R3;
        }
}

// What cf_batch_layout's kernels write, item by item, with the same functions: prefix sums
// (B+1 each), e_start (N+1), edges (2,E), pairs (U,5), batch (N).  Returns 0, or -1 when the sizes
// do not add up to N and E.
int host_batch_layout(const int64_t *sizes, int64_t B, int64_t N, int64_t E, int64_t *atom_start,
                      int64_t *edge_start, int64_t *unit_start, int64_t *e_start, int64_t *edges, int64_t *pairs,
                      int64_t *batch)
{
    atom_start[0] = edge_start[0] = unit_start[0] = 0;
    for (int64_t b = 0; b < B; b++) {
        const int64_t n = sizes[b];
        atom_start[b + 1] = atom_start[b] + n;
        edge_start[b + 1] = edge_start[b] + n * n;
        unit_start[b + 1] = unit_start[b] + n * (n + 1) / 2;
    }
    if (atom_start[B] != N || edge_start[B] != E) return -1;
    for (int64_t i = 0; i < N; i++) {
        int64_t crystal;
        e_start[i] = cf::row_start(atom_start, edge_start, B, i, &crystal);
        batch[i] = crystal;
    }
    e_start[N] = edge_start[B];
    for (int64_t e = 0; e < E; e++) {
        const cf::EdgeEnds r = cf::edge_ends(atom_start, edge_start, B, e);
        edges[e] = r.i;
        edges[E + e] = r.j;
        const int64_t u = cf::unit_of_edge(r, unit_start[r.crystal]);
        if (u < 0) continue;
        int64_t *d = pairs + 5 * u;
        d[0] = e;
        d[1] = cf::reverse_edge(r);
        d[2] = r.i;
        d[3] = r.j;
        d[4] = r.crystal;
    }
    return 0;
}

}  // extern "C"
