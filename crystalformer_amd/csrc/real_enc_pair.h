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
    const int64_t *pairs;   // (U,2): edge (i->j) with i <= j and its reverse
    const float *W;
    const float *rvlen;
    float *z;
    float *v;
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
};

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

__device__ __forceinline__ int wave_max_int(int v)
{
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v = max(v, __shfl_xor(v, off, WAVE));
    return v;
}

constexpr int WPB = 8;                   // wavefronts per work-group = units per round

// Bin handled by reduction step s (0..4*NT-1) and sub-lane kk (0..3) of the projection:
// chosen so that a lane's 4 consecutive steps read 4 consecutive bins.
__device__ __forceinline__ int proj_bin(int s, int kk) { return 16 * (s >> 2) + 4 * kk + (s & 3); }

}  // namespace cfpair
