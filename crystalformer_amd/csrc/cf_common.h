// Shared helpers for the gfx950 kernels: error reporting for the C ABI,
// wave64 reductions and the hardware transcendental wrappers.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>

#include "../../include/crystalformer_hip.h"
#include "cf_index_rules.h"

namespace cf {

constexpr int WAVE = 64;
constexpr float LOG2E = 1.4426950408889634f;
constexpr float LN2 = 0.6931471805599453f;

// ---- error reporting -------------------------------------------------------
void set_error(const char *fmt, ...);
int hip_failed(hipError_t err, const char *what);
int device_cu_count();
// Work-groups a persistent kernel may launch at `per_cu` per CU, scaled by the calling
// thread's launch share (cf_set_launch_share).
int persistent_grid_cap(int per_cu);
// Live sizes on the device (cf_set_size_header).  Each returns the header word that holds the
// live count when the calling thread has a header set and the argument is the capacity that
// word goes with (atoms, edges, atom pairs), else NULL: the size argument is then the size.
const int64_t *live_atoms(int64_t N);
const int64_t *live_edges(int64_t E);
const int64_t *live_units(int64_t U);
int64_t *size_header_for_layout(int64_t N, int64_t E);

// real_enc_mfma.hip
// order / counts (nullable, adaptive boxes from staged rings): the launch takes the units
// order[counts[0] .. counts[0] + counts[1]) (both counts on the device)
int launch_real_enc_fwd_pairs(const float *a_ik, const float *rpos, const float *tvecs, const int64_t *batch,
                              const int64_t *edges, const int64_t *pairs, int64_t U, int64_t N, int64_t H,
                              int64_t E, int64_t K, int64_t D, float bin_step, float s_scale, const float *W,
                              int64_t W_num, const float *rvlen, float cutoff, int lattice_range,
                              int min_range, unsigned int *sched, const int *order, const int64_t *counts,
                              float *z, float *v, hipStream_t st);

// real_enc_mfma_bwd.hip
int real_enc_bwd_pairs_blocks(int64_t U, int64_t H);
int launch_real_enc_bwd_pairs(const float *a_ik, const float *rpos, const float *tvecs, const int64_t *batch,
                              const int64_t *edges, const int64_t *pairs, int64_t U, const float *z,
                              const float *gz, const float *gv, int64_t N, int64_t H, int64_t E, int64_t K,
                              int64_t D, float bin_step, float s_scale, const float *W, const float *rvlen,
                              float cutoff, int lattice_range, int min_range, float *ga_edge,
                              float *gW_part, float *gW, const int64_t *e_start, float *ga_ik,
                              const float *rings, hipStream_t st);

// real_enc_ring.hip
int launch_ring_stage(const float *rpos, const float *tvecs, const int64_t *pairs, int64_t U, int64_t K,
                      float bin_step, float s_scale, int lattice_range, float weak_a, float *cache, hipStream_t st);
int launch_real_enc_fwd_rings(const float *a_ik, const int64_t *pairs, int64_t U, int64_t N, int64_t H, int64_t E,
                              int64_t K, int64_t D, float bin_step, float s_scale, const float *W,
                              const float *cache, const int *order, const int64_t *n_units,
                              float *z, float *v, hipStream_t st);
int64_t unit_partition_bytes(int64_t U);
int launch_unit_partition(const float *a_ik, const float *rvlen, const int64_t *pairs, int64_t U, int64_t N, int64_t H,
                          float cutoff, int lattice_range, int min_range, void *scratch, int64_t **counts_out,
                          int **order_out, hipStream_t st);

#define CF_REQUIRE(cond, code, ...)            \
    do {                                       \
        if (!(cond)) {                         \
            cf::set_error(__VA_ARGS__);        \
            return (code);                     \
        }                                      \
    } while (0)

#define CF_CHECK_LAUNCH(what)                                        \
    do {                                                             \
        hipError_t _e = hipGetLastError();                           \
        if (_e != hipSuccess) return cf::hip_failed(_e, (what));     \
    } while (0)

// ---- device helpers --------------------------------------------------------
#if defined(__HIPCC__)

// The live count behind a size argument: *live (clamped to the capacity, so that no value the
// header can hold sends a kernel outside its buffers) when a header word is given, else the
// argument itself.  Wave-uniform.
__device__ __forceinline__ int64_t live_count(const int64_t *live, int64_t capacity)
{
    if (!live) return capacity;
    const int64_t n = *live;
    const int64_t c = n < 0 ? 0 : (n > capacity ? capacity : n);
    const int lo = __builtin_amdgcn_readfirstlane((int)(c & 0xFFFFFFFFll));
    const int hi = __builtin_amdgcn_readfirstlane((int)(c >> 32));
    return ((int64_t)hi << 32) | (unsigned int)lo;
}

__device__ __forceinline__ float exp2_hw(float x) { return __builtin_amdgcn_exp2f(x); }
__device__ __forceinline__ float log2_hw(float x) { return __builtin_amdgcn_logf(x); }
__device__ __forceinline__ float sqrt_hw(float x) { return __builtin_amdgcn_sqrtf(x); }

__device__ __forceinline__ float readlane_f(float v, int lane)
{
    return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), lane));
}

// ---- wave64 reductions on the DPP data path (no LDS round trips) --------------
// Four steps inside each row of 16 lanes (quad swaps, rotations by 4 and 8), then
// row 0 -> 1 and 2 -> 3 (row_bcast:15) and rows 0..1 -> 2..3 (row_bcast:31): lane 63
// holds the result, which is returned wave-uniform.
template <int CTRL, int ROW_MASK>
__device__ __forceinline__ int dpp_i(int old, int v)
{
    return __builtin_amdgcn_update_dpp(old, v, CTRL, ROW_MASK, 0xF, false);
}
template <int CTRL, int ROW_MASK>
__device__ __forceinline__ float dpp_f(float old, float v)
{
    return __int_as_float(dpp_i<CTRL, ROW_MASK>(__float_as_int(old), __float_as_int(v)));
}
constexpr int DPP_QUAD_1032 = 0xB1, DPP_QUAD_2301 = 0x4E, DPP_ROW_ROR4 = 0x124, DPP_ROW_ROR8 = 0x128,
              DPP_ROW_BCAST15 = 0x142, DPP_ROW_BCAST31 = 0x143;

__device__ __forceinline__ float wave_sum(float v)
{
    v += dpp_f<DPP_QUAD_1032, 0xF>(0.f, v);
    v += dpp_f<DPP_QUAD_2301, 0xF>(0.f, v);
    v += dpp_f<DPP_ROW_ROR4, 0xF>(0.f, v);
    v += dpp_f<DPP_ROW_ROR8, 0xF>(0.f, v);
    v += dpp_f<DPP_ROW_BCAST15, 0xA>(0.f, v);
    v += dpp_f<DPP_ROW_BCAST31, 0xC>(0.f, v);
    return readlane_f(v, 63);
}

__device__ __forceinline__ float wave_min(float v)
{
    v = fminf(v, dpp_f<DPP_QUAD_1032, 0xF>(v, v));
    v = fminf(v, dpp_f<DPP_QUAD_2301, 0xF>(v, v));
    v = fminf(v, dpp_f<DPP_ROW_ROR4, 0xF>(v, v));
    v = fminf(v, dpp_f<DPP_ROW_ROR8, 0xF>(v, v));
    v = fminf(v, dpp_f<DPP_ROW_BCAST15, 0xA>(v, v));
    v = fminf(v, dpp_f<DPP_ROW_BCAST31, 0xC>(v, v));
    return readlane_f(v, 63);
}

__device__ __forceinline__ float wave_max(float v)
{
    v = fmaxf(v, dpp_f<DPP_QUAD_1032, 0xF>(v, v));
    v = fmaxf(v, dpp_f<DPP_QUAD_2301, 0xF>(v, v));
    v = fmaxf(v, dpp_f<DPP_ROW_ROR4, 0xF>(v, v));
    v = fmaxf(v, dpp_f<DPP_ROW_ROR8, 0xF>(v, v));
    v = fmaxf(v, dpp_f<DPP_ROW_BCAST15, 0xA>(v, v));
    v = fmaxf(v, dpp_f<DPP_ROW_BCAST31, 0xC>(v, v));
    return readlane_f(v, 63);
}

// Maximum over each row of 16 lanes, left in every lane of the row.
__device__ __forceinline__ float row16_max(float v)
{
    v = fmaxf(v, dpp_f<DPP_QUAD_1032, 0xF>(v, v));
    v = fmaxf(v, dpp_f<DPP_QUAD_2301, 0xF>(v, v));
    v = fmaxf(v, dpp_f<DPP_ROW_ROR4, 0xF>(v, v));
    v = fmaxf(v, dpp_f<DPP_ROW_ROR8, 0xF>(v, v));
    return v;
}

__device__ __forceinline__ float row16_min(float v)
{
    v = fminf(v, dpp_f<DPP_QUAD_1032, 0xF>(v, v));
    v = fminf(v, dpp_f<DPP_QUAD_2301, 0xF>(v, v));
    v = fminf(v, dpp_f<DPP_ROW_ROR4, 0xF>(v, v));
    v = fminf(v, dpp_f<DPP_ROW_ROR8, 0xF>(v, v));
    return v;
}

__device__ __forceinline__ int row16_max_i(int v)
{
    v = max(v, dpp_i<DPP_QUAD_1032, 0xF>(v, v));
    v = max(v, dpp_i<DPP_QUAD_2301, 0xF>(v, v));
    v = max(v, dpp_i<DPP_ROW_ROR4, 0xF>(v, v));
    v = max(v, dpp_i<DPP_ROW_ROR8, 0xF>(v, v));
    return v;
}

__device__ __forceinline__ int wave_max_i(int v)
{
    v = max(v, dpp_i<DPP_QUAD_1032, 0xF>(v, v));
    v = max(v, dpp_i<DPP_QUAD_2301, 0xF>(v, v));
    v = max(v, dpp_i<DPP_ROW_ROR4, 0xF>(v, v));
    v = max(v, dpp_i<DPP_ROW_ROR8, 0xF>(v, v));
    v = max(v, dpp_i<DPP_ROW_BCAST15, 0xA>(v, v));
    v = max(v, dpp_i<DPP_ROW_BCAST31, 0xC>(v, v));
    return __builtin_amdgcn_readlane(v, 63);
}

// Sum over the four rows of 16 lanes (lanes c, c + 16, c + 32, c + 48), left in every lane: two
// lane-swap instructions of gfx950 (odd rows of one copy against even rows of the other, then the
// upper half against the lower half) instead of two trips through the LDS permute path.
typedef unsigned int uint2_cf __attribute__((ext_vector_type(2)));
__device__ __forceinline__ float rows_sum(float v)
{
    unsigned int x = (unsigned int)__float_as_int(v);
    uint2_cf r = __builtin_amdgcn_permlane16_swap(x, x, false, false);
    v = __int_as_float((int)r[0]) + __int_as_float((int)r[1]);
    x = (unsigned int)__float_as_int(v);
    r = __builtin_amdgcn_permlane32_swap(x, x, false, false);
    return __int_as_float((int)r[0]) + __int_as_float((int)r[1]);
}

// Inclusive prefix sum over the 64 lanes (Hillis-Steele inside each row of 16 lanes on
// row shifts, then the row totals carried across with the two broadcasts), 6 instructions.
constexpr int DPP_ROW_SHR1 = 0x111, DPP_ROW_SHR2 = 0x112, DPP_ROW_SHR4 = 0x114, DPP_ROW_SHR8 = 0x118;
__device__ __forceinline__ int wave_inclusive_scan_i(int v)
{
    v += dpp_i<DPP_ROW_SHR1, 0xF>(0, v);
    v += dpp_i<DPP_ROW_SHR2, 0xF>(0, v);
    v += dpp_i<DPP_ROW_SHR4, 0xF>(0, v);
    v += dpp_i<DPP_ROW_SHR8, 0xF>(0, v);
    v += dpp_i<DPP_ROW_BCAST15, 0xA>(0, v);
    v += dpp_i<DPP_ROW_BCAST31, 0xC>(0, v);
    return v;
}

// Orders this wave's earlier LDS/global writes before its later reads.
__device__ __forceinline__ void wave_mem_sync()
{
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
}

#endif  // __HIPCC__

}  // namespace cf
