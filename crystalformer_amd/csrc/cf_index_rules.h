// Integer and range arithmetic shared by the device kernels and by a host build: the translation
// half-width rule and the index arithmetic of the dense per-crystal edge blocks.  Everything here is
// a pure function of its arguments, so that the same source can be compiled by a host compiler with
// sanitizers and checked value by value against the CPU oracle (the device build marks the
// functions __device__; a host build that defines CF_HOST_BUILD gets plain inline functions).
#pragma once

#include <math.h>
#include <stdint.h>

#if defined(CF_HOST_BUILD)
#define CF_HD static inline
#else
#define CF_HD __device__ __forceinline__
#endif

namespace cf {

// The reference kernels divide by 2.0 * CUDART_PI_F (the float constant widened
// to double); the translation half-widths are only bit-exact with that value.
constexpr float PI_F = 3.141592654f;
constexpr int MAX_RANGE = 64;

// Translation half-width along one axis: ceil((cutoff+0.01f)*rvl / (2*pi)),
// float product, double quotient.  The double division only runs where it can
// matter: a float quotient is within 1.3e-7 relative of the exact one, so its
// ceiling is already the answer unless it lies that close to an integer.
// Always within [max(0, minimum_range), max(MAX_RANGE, minimum_range)]: a quotient that is
// negative gives 0, one beyond MAX_RANGE (or +inf) gives MAX_RANGE, and NaN (an exponent a >= 0
// under the sigma rule, a NaN input) gives MAX_RANGE as well, so that every loop over a box
// terminates whatever the inputs hold.
CF_HD int range_axis(float cutoff, float rvl, int minimum_range)
{
    const float num = (cutoff + 0.01f) * rvl;
    const float qf = num * (float)(1.0 / (2.0 * (double)PI_F));
    int r;
    if (fabsf(qf - rintf(qf)) > 1.0e-6f * fabsf(qf) && fabsf(qf) < 1.0e6f) {
        const float c = ceilf(qf);
        r = c <= 0.f ? 0 : (c > (float)MAX_RANGE ? MAX_RANGE : (int)c);
    } else {
        const double q = ceil((double)num / (2.0 * (double)PI_F));
        r = (q >= 0.0 && q <= (double)MAX_RANGE) ? (int)q : (q > (double)MAX_RANGE ? MAX_RANGE : 0);
        if (q != q) r = MAX_RANGE;  // NaN exponent: bounded loop, result is NaN anyway
    }
    return r > minimum_range ? r : minimum_range;
}

// Half-widths for one (atom, head).  cutoff == 0 selects the fixed cube.
CF_HD void range_rule(float a, float cutoff, const float *rvl, int lattice_range, int minimum_range,
                      int &R1, int &R2, int &R3)
{
    R1 = R2 = R3 = lattice_range;
    if (cutoff != 0.0f) {
        if (cutoff < 0.0f) cutoff = sqrtf(-0.5f / a) * (-cutoff);
        R1 = range_axis(cutoff, rvl[0], minimum_range);
        R2 = range_axis(cutoff, rvl[1], minimum_range);
        R3 = range_axis(cutoff, rvl[2], minimum_range);
    }
}

// ---- dense per-crystal edge blocks ---------------------------------------------------------------
// start[] is a leading-zero cumulative sum over B >= 1 crystals (of n, or of n^2); the crystal that
// holds item x, start[lo] <= x < start[lo + 1], by bisection.  Crystals without items (equal
// consecutive entries) are skipped.  x must lie in [0, start[B]).
CF_HD int64_t locate_crystal(const int64_t *start, int64_t B, int64_t x)
{
    int64_t lo = 0, hi = B;   // invariant: start[lo] <= x < start[hi]
    while (hi - lo > 1) {
        const int64_t mid = (lo + hi) >> 1;
        if (start[mid] <= x) lo = mid; else hi = mid;
    }
    return lo;
}

// Edge e of the batch: crystal b, atoms (i, j) = a0 + divmod(e - e0, n) (i-major)
struct EdgeEnds { int64_t crystal, i, j, a0, n, e0; };
CF_HD EdgeEnds edge_ends(const int64_t *atom_start, const int64_t *edge_start, int64_t B, int64_t e)
{
    EdgeEnds r;
    r.crystal = locate_crystal(edge_start, B, e);
    r.a0 = atom_start[r.crystal];
    r.n = atom_start[r.crystal + 1] - r.a0;
    r.e0 = edge_start[r.crystal];
    const int64_t local = e - r.e0;
    const int64_t il = local / r.n;
    r.i = r.a0 + il;
    r.j = r.a0 + (local - il * r.n);
    return r;
}

// Unit (unordered atom pair) that owns edge (i <= j) of a crystal: row il of the upper triangle starts
// after il n - il (il - 1) / 2 units.  Returns -1 for an edge with i > j (its reverse owns the unit).
CF_HD int64_t unit_of_edge(const EdgeEnds &r, int64_t unit_start_of_crystal)
{
    const int64_t il = r.i - r.a0, jl = r.j - r.a0;
    if (il > jl) return -1;
    return unit_start_of_crystal + il * r.n - (il * (il - 1)) / 2 + (jl - il);
}

// the reverse edge (j -> i) of the same block
CF_HD int64_t reverse_edge(const EdgeEnds &r) { return r.e0 + (r.j - r.a0) * r.n + (r.i - r.a0); }

// First edge of atom i's row: edge_start[b] + (i - a0) n_b
CF_HD int64_t row_start(const int64_t *atom_start, const int64_t *edge_start, int64_t B, int64_t i, int64_t *crystal)
{
    const int64_t lo = locate_crystal(atom_start, B, i);
    const int64_t a0 = atom_start[lo];
    if (crystal) *crystal = lo;
    return edge_start[lo] + (i - a0) * (atom_start[lo + 1] - a0);
}

}  // namespace cf
