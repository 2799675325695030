// Row-block linear layers for gfx950: Y = act(X W^T + b) (+ R) for the small dense
// layers around the attention (a few thousand rows, 128..512 columns), where a
// library GEMM plus separate bias / activation / residual launches are all latency.
// fp32 on v_mfma_f32_16x16x4_f32, operands straight from global memory (the weights
// stay in L2), bias, ReLU and the residual in the epilogue, and up to three weight
// matrices of equal shape served by one launch (query / key / value projections).
#include "cf_common.h"

namespace {

using namespace cf;

typedef float float4_t __attribute__((ext_vector_type(4)));

struct LinArgs {
    const float *x;            // (N, K)
    const float *w[3];         // each (C, K), row-major: out = x w^T
    const float *bias;         // (nw * C) or null
    const float *res;          // (N, C) or null (nw == 1)
    float *y[3];               // each (N, C)
    int64_t N;
    int K, C, nw, relu;
};

constexpr int LIN_ROWS = 16;   // rows per work-group
constexpr int LIN_COLS = 32;   // columns per work-group (two 16 x 16 accumulator tiles)
constexpr int LIN_WAVES = 4;   // wavefronts per work-group, splitting the reduction dimension

// A work-group owns 16 rows x 32 columns; its 4 wavefronts take the 16-wide k-steps
// round robin (few dependent loads per wavefront: these layers are latency, not
// throughput) and wavefront 0 adds the partial tiles from LDS and runs the epilogue.
// Lane (q, c) = (lane / 16, lane % 16) loads 16 bytes of row c of X and of rows c, c + 16
// of W at k = 16 s + 4 q: four MFMA steps per load, step r reducing over
// k = 16 s + 4 q' + r (q' = 0..3) in both operands.
__global__ __launch_bounds__(64 * LIN_WAVES) void linear_rows_kernel(LinArgs p)
{
    __shared__ float part[LIN_WAVES - 1][8][WAVE];
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int q = lane >> 4, c = lane & 15;
    const int64_t row0 = (int64_t)blockIdx.x * LIN_ROWS;
    const int col0 = blockIdx.y * LIN_COLS;                         // column over all weights
    const int total_cols = p.nw * p.C;
    const int64_t arow = min(row0 + c, p.N - 1);
    const float *xa = p.x + arow * p.K + 4 * q;
    const float *wb[2];
#pragma unroll
    for (int t = 0; t < 2; t++) {
        const int col = min(col0 + 16 * t + c, total_cols - 1);
        const int wi = col / p.C;
        wb[t] = p.w[wi] + (int64_t)(col - wi * p.C) * p.K + 4 * q;
    }
    float4_t acc[2] = {float4_t{0.f, 0.f, 0.f, 0.f}, float4_t{0.f, 0.f, 0.f, 0.f}};
    auto step = [&](const float4_t &a, const float4_t &b0, const float4_t &b1) {
#pragma unroll
        for (int r = 0; r < 4; r++) {
            acc[0] = __builtin_amdgcn_mfma_f32_16x16x4f32(a[r], b0[r], acc[0], 0, 0, 0);
            acc[1] = __builtin_amdgcn_mfma_f32_16x16x4f32(a[r], b1[r], acc[1], 0, 0, 0);
        }
    };
    const int stride = 16 * LIN_WAVES;
    int k0 = 16 * wave;
    for (; k0 + 3 * stride < p.K; k0 += 4 * stride) {     // 12 loads in flight, then 32 MFMAs
        float4_t a[4], b0[4], b1[4];
#pragma unroll
        for (int u = 0; u < 4; u++) {
            a[u] = *reinterpret_cast<const float4_t *>(xa + k0 + stride * u);
            b0[u] = *reinterpret_cast<const float4_t *>(wb[0] + k0 + stride * u);
            b1[u] = *reinterpret_cast<const float4_t *>(wb[1] + k0 + stride * u);
        }
#pragma unroll
        for (int u = 0; u < 4; u++) step(a[u], b0[u], b1[u]);
    }
    for (; k0 < p.K; k0 += stride)
        step(*reinterpret_cast<const float4_t *>(xa + k0), *reinterpret_cast<const float4_t *>(wb[0] + k0),
             *reinterpret_cast<const float4_t *>(wb[1] + k0));
    if (wave > 0) {
#pragma unroll
        for (int t = 0; t < 2; t++)
#pragma unroll
            for (int r = 0; r < 4; r++) part[wave - 1][4 * t + r][lane] = acc[t][r];
    }
    __syncthreads();
    if (wave > 0) return;
#pragma unroll
    for (int w = 0; w < LIN_WAVES - 1; w++)
#pragma unroll
        for (int t = 0; t < 2; t++)
#pragma unroll
            for (int r = 0; r < 4; r++) acc[t][r] += part[w][4 * t + r][lane];
    // lane (q, c) holds rows row0 + 4 q + r, column col0 + 16 t + c
#pragma unroll
    for (int t = 0; t < 2; t++) {
        const int col = col0 + 16 * t + c;
        if (col >= total_cols) continue;
        const int wi = col / p.C;
        const int lc = col - wi * p.C;
        const float bv = p.bias ? p.bias[col] : 0.f;
        float *y = p.y[wi];
#pragma unroll
        for (int r = 0; r < 4; r++) {
            const int64_t row = row0 + 4 * q + r;
            if (row >= p.N) continue;
            float v = acc[t][r] + bv;
            if (p.res) v += p.res[row * p.C + lc];
            if (p.relu) v = fmaxf(v, 0.f);
            y[row * p.C + lc] = v;
        }
    }
}

}  // namespace

extern "C" int cf_linear_rows(const float *x, int64_t N, int64_t K, const float *w0, const float *w1,
                              const float *w2, int n_weights, int64_t C, const float *bias,
                              const float *residual, int relu, float *y0, float *y1, float *y2, void *stream)
{
    CF_REQUIRE(N >= 0 && K >= 1 && C >= 1 && n_weights >= 1 && n_weights <= 3, CF_ERR_INVALID_ARGUMENT,
               "cf_linear_rows: bad sizes N=%lld K=%lld C=%lld weights=%d", (long long)N, (long long)K,
               (long long)C, n_weights);
    if (N == 0) return CF_OK;
    CF_REQUIRE(K % 16 == 0 && K <= (1 << 20) && C <= (1 << 20), CF_ERR_UNSUPPORTED,
               "cf_linear_rows: the input width must be a multiple of 16 (got %lld)", (long long)K);
    CF_REQUIRE(!residual || n_weights == 1, CF_ERR_INVALID_ARGUMENT,
               "cf_linear_rows: a residual needs a single weight matrix");
    const float *w[3] = {w0, w1, w2};
    float *y[3] = {y0, y1, y2};
    CF_REQUIRE(x, CF_ERR_INVALID_ARGUMENT, "cf_linear_rows: x is NULL");
    LinArgs p{};
    p.x = x;
    for (int i = 0; i < 3; i++) {
        if (i < n_weights)
            CF_REQUIRE(w[i] && y[i], CF_ERR_INVALID_ARGUMENT, "cf_linear_rows: weight or output %d is NULL", i);
        p.w[i] = i < n_weights ? w[i] : w[0];
        p.y[i] = i < n_weights ? y[i] : y[0];
    }
    p.bias = bias; p.res = residual;
    p.N = N; p.K = (int)K; p.C = (int)C; p.nw = n_weights; p.relu = relu;
    const int64_t gx = (N + LIN_ROWS - 1) / LIN_ROWS;
    const int64_t gy = ((int64_t)n_weights * C + LIN_COLS - 1) / LIN_COLS;
    CF_REQUIRE(gx < (1ll << 31) && gy < 65536, CF_ERR_UNSUPPORTED, "cf_linear_rows: too large");
    linear_rows_kernel<<<dim3((unsigned)gx, (unsigned)gy), 64 * LIN_WAVES, 0, (hipStream_t)stream>>>(p);
    CF_CHECK_LAUNCH("cf_linear_rows");
    return CF_OK;
}
