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
    const int64_t *live_N;     // nullable: live row count on the device (N is then the capacity)
};

// LDS-tiled: a work-group of 4 wavefronts (WR x WC) owns TM rows x TN columns; every KC-wide
// chunk of the reduction is staged once in LDS (X tile and W tile, 16-byte global loads held
// in registers while the previous chunk is multiplied) and read back as MFMA operands:
// lane (q, c) = (lane / 16, lane % 16) reads 16 bytes of row c of a 16-row tile at
// k = 16 s + 4 q, four MFMA steps per read, step r reducing over k = 16 s + 4 q' + r.
// KC = 32 for large problems (many work-groups per CU hide the staging latency); KC = 64 for
// the few thousand rows of a batch, where a work-group is nearly alone on its CU and every
// chunk costs a full memory round trip (a 128-wide layer is then two chunks; one chunk of 128
// is no faster and its 50 KB of LDS keep it from running beside the encoding kernel).
// The LDS row stride KC + 4 floats keeps the rows 16-byte aligned and staggers the banks.
template <int TM, int TN, int WR, int WC, int KC>
__global__ __launch_bounds__(256) void linear_rows_kernel(LinArgs p)
{
    constexpr int LD = KC + 4;
    constexpr int MT = TM / (16 * WR), NT = TN / (16 * WC);     // 16 x 16 tiles per wavefront
    constexpr int PPR = KC / 4, RPP = 256 / PPR;                // 16-byte pieces per tile row, rows per staging pass
    constexpr int XL = TM / RPP, WL = TN / RPP;                 // 16-byte loads per thread and chunk
    static_assert(XL >= 1 && WL >= 1, "tile too small for the staging pattern");
    __shared__ __align__(16) float xs[TM * LD];
    __shared__ __align__(16) float ws[TN * LD];
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int q = lane >> 4, c = lane & 15;
    const int wr = wave / WC, wc = wave - wr * WC;
    const int64_t N = live_count(p.live_N, p.N);
    const int col0 = blockIdx.y * TN;                           // column over all weights
    // (one row tile per work-group unless the grid was cut short: with a live row count the launch
    // covers a capacity, and a work-group then strides over the row tiles that exist)
    for (int64_t row0 = (int64_t)blockIdx.x * TM; row0 < N; row0 += (int64_t)gridDim.x * TM) {
    const int total_cols = p.nw * p.C;
    // staging role: thread -> (row t / PPR (+RPP u), 16-byte piece t % PPR) of a tile
    const int srow = threadIdx.x / PPR, spiece = threadIdx.x % PPR;
    const float *xg[XL];
    const float *wg[WL];
#pragma unroll
    for (int u = 0; u < XL; u++) xg[u] = p.x + min(row0 + srow + RPP * u, N - 1) * p.K + 4 * spiece;
#pragma unroll
    for (int u = 0; u < WL; u++) {
        const int col = min(col0 + srow + RPP * u, total_cols - 1);
        const int wi = col / p.C;
        wg[u] = p.w[wi] + (int64_t)(col - wi * p.C) * p.K + 4 * spiece;
    }
    float4_t acc[MT][NT];
#pragma unroll
    for (int mt = 0; mt < MT; mt++)
#pragma unroll
        for (int nt = 0; nt < NT; nt++) acc[mt][nt] = float4_t{0.f, 0.f, 0.f, 0.f};
    const float4_t zero4 = {0.f, 0.f, 0.f, 0.f};
    float4_t xr[XL], wrg[WL];
    auto fetch = [&](int k0) {
        const bool in = k0 + 4 * spiece < p.K;                  // K is a multiple of 4
#pragma unroll
        for (int u = 0; u < XL; u++) xr[u] = in ? *reinterpret_cast<const float4_t *>(xg[u] + k0) : zero4;
#pragma unroll
        for (int u = 0; u < WL; u++) wrg[u] = in ? *reinterpret_cast<const float4_t *>(wg[u] + k0) : zero4;
    };
    fetch(0);
    for (int k0 = 0; k0 < p.K; k0 += KC) {
        __syncthreads();                                        // previous chunk fully consumed
#pragma unroll
        for (int u = 0; u < XL; u++)
            *reinterpret_cast<float4_t *>(xs + (srow + RPP * u) * LD + 4 * spiece) = xr[u];
#pragma unroll
        for (int u = 0; u < WL; u++)
            *reinterpret_cast<float4_t *>(ws + (srow + RPP * u) * LD + 4 * spiece) = wrg[u];
        __syncthreads();
        if (k0 + KC < p.K) fetch(k0 + KC);                      // in flight during the MFMAs below
#pragma unroll
        for (int ss = 0; ss < KC / 16; ss++) {
            float4_t a[MT], b[NT];
#pragma unroll
            for (int mt = 0; mt < MT; mt++)
                a[mt] = *reinterpret_cast<const float4_t *>(xs + ((wr * MT + mt) * 16 + c) * LD + 16 * ss + 4 * q);
#pragma unroll
            for (int nt = 0; nt < NT; nt++)
                b[nt] = *reinterpret_cast<const float4_t *>(ws + ((wc * NT + nt) * 16 + c) * LD + 16 * ss + 4 * q);
#pragma unroll
            for (int r = 0; r < 4; r++)
#pragma unroll
                for (int mt = 0; mt < MT; mt++)
#pragma unroll
                    for (int nt = 0; nt < NT; nt++)
                        acc[mt][nt] = __builtin_amdgcn_mfma_f32_16x16x4f32(a[mt][r], b[nt][r], acc[mt][nt], 0, 0, 0);
        }
    }
    // lane (q, c) of tile (mt, nt) holds rows .. + 4 q + r, column .. + c
#pragma unroll
    for (int nt = 0; nt < NT; nt++) {
        const int col = col0 + (wc * NT + nt) * 16 + c;
        if (col >= total_cols) continue;
        const int wi = col / p.C;
        const int lc = col - wi * p.C;
        const float bv = p.bias ? p.bias[col] : 0.f;
        float *y = p.y[wi];
#pragma unroll
        for (int mt = 0; mt < MT; mt++)
#pragma unroll
            for (int r = 0; r < 4; r++) {
                const int64_t row = row0 + (wr * MT + mt) * 16 + 4 * q + r;
                if (row >= N) continue;
                float v = acc[mt][nt][r] + bv;
                if (p.res) v += p.res[row * p.C + lc];
                if (p.relu) v = v < 0.f ? 0.f : v;              // (a NaN stays one, as in torch.relu)
                y[row * p.C + lc] = v;
            }
    }
    }
}

// Input gradient of linear layers: Y (N, K) = mask(sum_i G_i W_i) + A with G_i (N, C), W_i (C, K)
// row-major, up to three terms sharing the shapes (the query / key / value projections feed one
// input), A an optional addend (the gradient arriving on a residual branch) and mask an optional
// (N, K) tensor whose non-positive entries zero the product (the ReLU in front of the layer).
// Same tiling as linear_rows_kernel (64 x 64 per work-group, 2 x 2 wavefronts), 64-wide chunks
// of the reduction staged in LDS; here the reduction runs over the rows of W, so its tile is
// staged as [reduction][column] and read four bytes at a time as the B operand.
constexpr int NN_T = 64;
constexpr int NN_KC = 64;          // reduction chunk: long enough for the next chunk's loads to land meanwhile
constexpr int NN_GLD = NN_KC + 4;  // G tile row stride (floats): 16-byte aligned, staggers the banks
constexpr int NN_WLD = NN_T + 4;   // 4 rows apart = 16 banks apart: the four rows of a B read cover all banks twice

struct LinNNArgs {
    const float *g[3];
    const float *w[3];
    const float *add, *mask;
    float *y;
    int64_t N;
    int C, K, terms;
};

// TM x TN outputs per work-group (64 or 32 each), 2 x 2 wavefronts of TM/2 x TN/2.
template <int TM, int TN>
__global__ __launch_bounds__(256) void linear_rows_nn_kernel(LinNNArgs p)
{
    constexpr int MT = TM / 32, NTL = TN / 32;                  // 16 x 16 tiles per wavefront
    constexpr int WLD = TN + 4;                                  // as NN_WLD for the 64-wide tile
    constexpr int GP = TM / 16;                                  // staging passes of the G tile (16 rows each)
    constexpr int WPR = TN / 4, WROWS = 256 / WPR, WP = NN_KC / WROWS;   // W tile: pieces per row, rows per pass, passes
    __shared__ __align__(16) float gs[TM * NN_GLD];
    __shared__ __align__(16) float ws[NN_KC * WLD];
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int q = lane >> 4, c = lane & 15;
    const int wr = wave >> 1, wc = wave & 1;
    const int64_t row0 = (int64_t)blockIdx.x * TM;
    const int col0 = blockIdx.y * TN;
    // staging roles: G tile (TM rows x 64 floats): row t / 16 (+16 u), piece t % 16;
    // W tile (64 rows x TN floats): row t / WPR (+WROWS u), piece t % WPR
    const int srow = threadIdx.x >> 4, spiece = threadIdx.x & 15;
    const int wrow = threadIdx.x / WPR, wpiece = threadIdx.x % WPR;
    int64_t grow[GP];
#pragma unroll
    for (int u = 0; u < GP; u++) grow[u] = min(row0 + srow + 16 * u, p.N - 1) * p.C + 4 * spiece;
    const int wcol = min(col0 + 4 * wpiece, p.K - 4);           // K is a multiple of 4

    float4_t acc[MT][NTL];
#pragma unroll
    for (int i = 0; i < MT; i++)
#pragma unroll
        for (int j = 0; j < NTL; j++) acc[i][j] = float4_t{0.f, 0.f, 0.f, 0.f};
    const int chunks = p.C / NN_KC;                              // C is a multiple of 64
    const int steps = p.terms * chunks;
    // Two register sets, each fetched two chunks ahead: few wavefronts share a SIMD for these
    // shapes, so nothing else hides the latency of the loads.
    float4_t gr[2][GP], wg[2][WP];
    auto fetch = [&](int step, float4_t *gdst, float4_t *wdst) {
        if (step >= steps) return;
        const int term = step / chunks, k0 = (step - term * chunks) * NN_KC;
        const float *g = p.g[term] + k0, *w = p.w[term] + (int64_t)(k0 + wrow) * p.K + wcol;
#pragma unroll
        for (int u = 0; u < GP; u++) gdst[u] = *reinterpret_cast<const float4_t *>(g + grow[u]);
#pragma unroll
        for (int u = 0; u < WP; u++) wdst[u] = *reinterpret_cast<const float4_t *>(w + (int64_t)(WROWS * u) * p.K);
    };
    auto chunk = [&](int step, float4_t *gset, float4_t *wset) {
        __syncthreads();                                         // previous chunk fully consumed
#pragma unroll
        for (int u = 0; u < GP; u++)
            *reinterpret_cast<float4_t *>(gs + (srow + 16 * u) * NN_GLD + 4 * spiece) = gset[u];
#pragma unroll
        for (int u = 0; u < WP; u++)
            *reinterpret_cast<float4_t *>(ws + (wrow + WROWS * u) * WLD + 4 * wpiece) = wset[u];
        __syncthreads();
        fetch(step + 2, gset, wset);                             // in flight during this and the next chunk
        // all operands of the chunk first (one wait), then the MFMAs: with one wavefront per SIMD a
        // wait per read would be paid in full
        float4_t a[NN_KC / 16][MT];
        float b[NN_KC / 16][4][NTL];
#pragma unroll
        for (int ss = 0; ss < NN_KC / 16; ss++) {
#pragma unroll
            for (int i = 0; i < MT; i++)
                a[ss][i] = *reinterpret_cast<const float4_t *>(gs + ((wr * MT + i) * 16 + c) * NN_GLD + 16 * ss + 4 * q);
#pragma unroll
            for (int r = 0; r < 4; r++)
#pragma unroll
                for (int j = 0; j < NTL; j++)   // step r reduces over the rows 16 ss + 4 q' + r of the W tile
                    b[ss][r][j] = ws[(16 * ss + 4 * q + r) * WLD + (wc * NTL + j) * 16 + c];
        }
#pragma unroll
        for (int ss = 0; ss < NN_KC / 16; ss++)
#pragma unroll
            for (int r = 0; r < 4; r++)
#pragma unroll
                for (int i = 0; i < MT; i++)
#pragma unroll
                    for (int j = 0; j < NTL; j++)
                        acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x4f32(a[ss][i][r], b[ss][r][j], acc[i][j], 0, 0, 0);
    };
    fetch(0, gr[0], wg[0]);
    fetch(1, gr[1], wg[1]);
    for (int step = 0; step < steps; step += 2) {
        chunk(step, gr[0], wg[0]);
        if (step + 1 < steps) chunk(step + 1, gr[1], wg[1]);
    }
#pragma unroll
    for (int j = 0; j < NTL; j++) {
        const int col = col0 + (wc * NTL + j) * 16 + c;
        if (col >= p.K) continue;
#pragma unroll
        for (int i = 0; i < MT; i++)
#pragma unroll
            for (int r = 0; r < 4; r++) {
                const int64_t row = row0 + (wr * MT + i) * 16 + 4 * q + r;
                if (row >= p.N) continue;
                float v = acc[i][j][r];
                if (p.mask && !(p.mask[row * p.K + col] > 0.f)) v = 0.f;
                if (p.add) v += p.add[row * p.K + col];
                p.y[row * p.K + col] = v;
            }
    }
}

// Column sums of a row-major (N, C) matrix (the bias gradient of a linear layer): 16 columns x
// 64 row groups per work-group of 1024 threads, each thread adds every 64th row into 4 running
// sums, the 64 partial sums of a column are then added in order.  No atomics, no scratch.
__global__ __launch_bounds__(1024) void column_sum_kernel(const float *g, int64_t N, int C, float *out)
{
    __shared__ float red[64][17];
    const int cx = threadIdx.x & 15, rg = threadIdx.x >> 4;
    const int col = blockIdx.x * 16 + cx;
    float acc[4] = {0.f, 0.f, 0.f, 0.f};
    if (col < C) {
        int64_t n = rg;
        for (; n + 192 < N; n += 256) {
#pragma unroll
            for (int u = 0; u < 4; u++) acc[u] += g[(n + 64 * u) * C + col];
        }
        for (; n < N; n += 64) acc[0] += g[n * C + col];
    }
    red[rg][cx] = (acc[0] + acc[1]) + (acc[2] + acc[3]);
    __syncthreads();
    if (rg == 0 && col < C) {
        float total = red[0][cx];
#pragma unroll 8
        for (int r = 1; r < 64; r++) total += red[r][cx];
        out[col] = total;
    }
}

// Weight gradient of a linear layer, gW (C, K) = g^T x with g (N, C), x (N, K): a short, wide
// product with a long reduction over the rows.  The rows are cut into slices whose partial
// products are written out and added by a second kernel in a fixed order (no atomics).  The
// slice kernel serves a group of layers at once (kernel further down); a single layer is a
// group of one.

// ---- grouped weight gradients -------------------------------------------------
// The weight (and bias) gradients of several linear layers in two launches: the layers'
// 64 x 64 output tiles are numbered consecutively and a work-group finds its layer by
// scanning the group's tile prefix.
constexpr int WG_GROUP = 32;       // layers per launch pair (64 bytes each of the 4 KB of kernel arguments)

struct WeightGradGroup {
    const float *g[WG_GROUP], *x[WG_GROUP];
    float *gw[WG_GROUP], *gb[WG_GROUP];
    int64_t part_off[WG_GROUP];      // floats from the workspace start to this layer's slices
    int N[WG_GROUP], C[WG_GROUP], K[WG_GROUP], slices[WG_GROUP];
    int tile0[WG_GROUP + 1];         // prefix over 64 x 64 tiles
    int cell0[WG_GROUP + 1];         // prefix over 256-element blocks of C (K + 1) outputs
    int count;
    float *part;
};
static_assert(sizeof(WeightGradGroup) <= 4096, "WeightGradGroup must fit the kernel-argument segment");

constexpr int WGT = 64;            // output tile of a work-group: 64 x 64
constexpr int WG_ROWS = 16;        // rows staged per step
constexpr int WG_LD = WGT + 16;    // LDS row stride, 16 mod 32: the four rows of an operand read cover all banks twice

// A work-group of 4 wavefronts (2 x 2, 32 x 32 outputs each) owns a 64 x 64 block of one
// layer's gW for one slice of rows.  16 rows of g (64 columns) and of x (64 columns) are staged
// in LDS per step with 16-byte global loads (one per thread and matrix) and read back as MFMA
// operands: lane (q, c) takes g[row 4 s + q][column c] and x[row 4 s + q][column c], four rows
// per v_mfma_f32_16x16x4_f32.  The bias gradient (column sums of g) comes from the operands of
// the wavefronts in the first block column.
__global__ __launch_bounds__(256) void weight_grad_group_slices_kernel(WeightGradGroup a)
{
    __shared__ __align__(16) float gs[WG_ROWS * WG_LD];
    __shared__ __align__(16) float xs[WG_ROWS * WG_LD];
    int t = 0;
    while (t + 1 < a.count && a.tile0[t + 1] <= (int)blockIdx.x) t++;
    if ((int)blockIdx.y >= a.slices[t]) return;
    const int tile = blockIdx.x - a.tile0[t];
    const int C = a.C[t], K = a.K[t];
    const int64_t N = a.N[t];
    const int tiles_k = (K + WGT - 1) / WGT;
    const int tc = tile / tiles_k, tk = tile - tc * tiles_k;
    const int slices = a.slices[t];
    int rows = (int)(((N + slices - 1) / slices + 3) / 4 * 4);
    if (rows < 4) rows = 4;
    const float *g = a.g[t], *x = a.x[t];
    float *part = a.part + a.part_off[t];
    float *part_b = a.gb[t] ? part + (int64_t)slices * C * K : nullptr;

    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int q = lane >> 4, c = lane & 15;
    const int wr = wave >> 1, wc = wave & 1;
    const int c0 = tc * WGT, k0 = tk * WGT;
    const int64_t n_begin = (int64_t)blockIdx.y * rows;
    const int64_t n_end = min(N, n_begin + rows);
    // staging role: thread -> row t / 16, four columns from 4 (t % 16)
    const int srow = threadIdx.x >> 4, scol = (threadIdx.x & 15) * 4;
    const bool vec_g = (C & 3) == 0 && c0 + scol + 3 < C, vec_x = (K & 3) == 0 && k0 + scol + 3 < K;

    float4_t acc[2][2];
#pragma unroll
    for (int i = 0; i < 2; i++)
#pragma unroll
        for (int j = 0; j < 2; j++) acc[i][j] = float4_t{0.f, 0.f, 0.f, 0.f};
    float colsum[2] = {0.f, 0.f};
    auto fetch = [&](const float *src, int64_t n, int ld, int col0, int width, bool vec) -> float4_t {
        float4_t v = {0.f, 0.f, 0.f, 0.f};
        if (n < n_end) {
            if (vec) {
                v = *reinterpret_cast<const float4_t *>(src + n * ld + col0);
            } else {
#pragma unroll
                for (int r = 0; r < 4; r++)
                    if (col0 + r < width) v[r] = src[n * ld + col0 + r];
            }
        }
        return v;
    };
    float4_t gn = fetch(g, n_begin + srow, C, c0 + scol, C, vec_g);
    float4_t xn = fetch(x, n_begin + srow, K, k0 + scol, K, vec_x);
    for (int64_t n0 = n_begin; n0 < n_end; n0 += WG_ROWS) {
        __syncthreads();                               // the previous step's operands have been read
        *reinterpret_cast<float4_t *>(gs + srow * WG_LD + scol) = gn;
        *reinterpret_cast<float4_t *>(xs + srow * WG_LD + scol) = xn;
        __syncthreads();
        gn = fetch(g, n0 + WG_ROWS + srow, C, c0 + scol, C, vec_g);
        xn = fetch(x, n0 + WG_ROWS + srow, K, k0 + scol, K, vec_x);
#pragma unroll
        for (int s4 = 0; s4 < WG_ROWS / 4; s4++) {
            float av[2], bv[2];
#pragma unroll
            for (int i = 0; i < 2; i++) av[i] = gs[(4 * s4 + q) * WG_LD + 32 * wr + 16 * i + c];
#pragma unroll
            for (int j = 0; j < 2; j++) bv[j] = xs[(4 * s4 + q) * WG_LD + 32 * wc + 16 * j + c];
#pragma unroll
            for (int i = 0; i < 2; i++) {
                colsum[i] += av[i];
#pragma unroll
                for (int j = 0; j < 2; j++)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x4f32(av[i], bv[j], acc[i][j], 0, 0, 0);
            }
        }
    }
    if (part_b && tk == 0 && wc == 0) {
#pragma unroll
        for (int i = 0; i < 2; i++) {
            // rows n = 4 s + q: add the four row classes in ascending q
            const float s = (colsum[i] + __shfl_xor(colsum[i], 16, 64)) +
                            (__shfl_xor(colsum[i], 32, 64) + __shfl_xor(colsum[i], 48, 64));
            const int cc = c0 + 32 * wr + 16 * i + c;
            if (q == 0 && cc < C) part_b[(int64_t)blockIdx.y * C + cc] = s;
        }
    }
    // lane (q, c) holds gW[c0 + 32 wr + 16 i + 4 q + r][k0 + 32 wc + 16 j + c]
    float *dst = part + (int64_t)blockIdx.y * C * K;
#pragma unroll
    for (int i = 0; i < 2; i++)
#pragma unroll
        for (int j = 0; j < 2; j++)
#pragma unroll
            for (int r = 0; r < 4; r++) {
                const int cc = c0 + 32 * wr + 16 * i + 4 * q + r, kk = k0 + 32 * wc + 16 * j + c;
                if (cc < C && kk < K) dst[(int64_t)cc * K + kk] = acc[i][j][r];
            }
}

__global__ __launch_bounds__(256) void weight_grad_group_add_kernel(WeightGradGroup a)
{
    int t = 0;
    while (t + 1 < a.count && a.cell0[t + 1] <= (int)blockIdx.x) t++;
    int64_t x = (int64_t)(blockIdx.x - a.cell0[t]) * 256 + threadIdx.x;
    const int slices = a.slices[t];
    int64_t total = (int64_t)a.C[t] * a.K[t];
    const float *part = a.part + a.part_off[t];
    float *out = a.gw[t];
    if (x >= total) {
        x -= total;
        if (!a.gb[t] || x >= a.C[t]) return;
        part += (int64_t)slices * total;
        total = a.C[t];
        out = a.gb[t];
    }
    float a0 = 0.f, a1 = 0.f;
    int s = 0;
    for (; s + 1 < slices; s += 2) {
        a0 += part[(int64_t)s * total + x];
        a1 += part[(int64_t)(s + 1) * total + x];
    }
    if (s < slices) a0 += part[(int64_t)s * total + x];
    out[x] = a0 + a1;
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
    p.live_N = cf::live_atoms(N);      // (rows are atoms when N is the atom capacity of a size header)
    // few rows (a tile grid that leaves CUs idle): 32 x 32 tiles, four to eight times the work-groups;
    // otherwise wide outputs take 64-column tiles (2 x 2 wavefronts), narrow ones 32-column tiles
    const int64_t total_cols = (int64_t)n_weights * C;
    const bool small = N <= 8192;
    const bool wide = !small && total_cols >= 256;
    int64_t gx = (N + (small ? 31 : 63)) / (small ? 32 : 64);
    // a capacity: most row tiles are beyond the live rows, so launch a bounded number of work-groups
    // per column tile and let them stride (empty work-groups cost a few microseconds per thousand)
    if (p.live_N && gx > 128) gx = 128;
    const int64_t gy = (total_cols + (wide ? 63 : 31)) / (wide ? 64 : 32);
    CF_REQUIRE(gx < (1ll << 31) && gy < 65536, CF_ERR_UNSUPPORTED, "cf_linear_rows: too large");
    const dim3 grid((unsigned)gx, (unsigned)gy);
    hipStream_t st = (hipStream_t)stream;
    if (small && K >= 64)
        linear_rows_kernel<32, 32, 2, 2, 64><<<grid, 256, 0, st>>>(p);
    else if (small)
        linear_rows_kernel<32, 32, 2, 2, 32><<<grid, 256, 0, st>>>(p);
    else if (wide)
        linear_rows_kernel<64, 64, 2, 2, 32><<<grid, 256, 0, st>>>(p);
    else
        linear_rows_kernel<64, 32, 4, 1, 32><<<grid, 256, 0, st>>>(p);
    CF_CHECK_LAUNCH("cf_linear_rows");
    return CF_OK;
}

extern "C" int cf_linear_rows_nn(const float *g0, const float *g1, const float *g2, int n_terms, const float *w0,
                                 const float *w1, const float *w2, int64_t N, int64_t C, int64_t K,
                                 const float *add, const float *mask, float *y, void *stream)
{
    CF_REQUIRE(N >= 0 && C >= 1 && K >= 1 && n_terms >= 1 && n_terms <= 3 && C <= (1 << 20) && K <= (1 << 20),
               CF_ERR_INVALID_ARGUMENT, "cf_linear_rows_nn: bad sizes N=%lld C=%lld K=%lld terms=%d", (long long)N,
               (long long)C, (long long)K, n_terms);
    if (N == 0) return CF_OK;
    CF_REQUIRE(C % 64 == 0 && K % 4 == 0, CF_ERR_UNSUPPORTED,
               "cf_linear_rows_nn: C must be a multiple of 64 and K of 4 (got %lld, %lld)", (long long)C,
               (long long)K);
    const float *g[3] = {g0, g1, g2}, *w[3] = {w0, w1, w2};
    LinNNArgs p{};
    for (int i = 0; i < n_terms; i++) {
        CF_REQUIRE(g[i] && w[i], CF_ERR_INVALID_ARGUMENT, "cf_linear_rows_nn: null operand %d", i);
        p.g[i] = g[i];
        p.w[i] = w[i];
    }
    CF_REQUIRE(y, CF_ERR_INVALID_ARGUMENT, "cf_linear_rows_nn: null output");
    p.add = add; p.mask = mask; p.y = y; p.N = N; p.C = (int)C; p.K = (int)K; p.terms = n_terms;
    // quarter tiles while full ones would leave most CUs without a work-group
    if (((N + 63) / 64) * ((K + 63) / 64) < 256) {
        dim3 grid((unsigned)((N + 31) / 32), (unsigned)((K + 31) / 32));
        linear_rows_nn_kernel<32, 32><<<grid, 256, 0, (hipStream_t)stream>>>(p);
    } else {
        dim3 grid((unsigned)((N + NN_T - 1) / NN_T), (unsigned)((K + NN_T - 1) / NN_T));
        linear_rows_nn_kernel<NN_T, NN_T><<<grid, 256, 0, (hipStream_t)stream>>>(p);
    }
    CF_CHECK_LAUNCH("cf_linear_rows_nn");
    return CF_OK;
}

extern "C" int cf_column_sum(const float *g, int64_t N, int64_t C, float *out, void *stream)
{
    CF_REQUIRE(N >= 0 && C >= 1 && C < (1ll << 30), CF_ERR_INVALID_ARGUMENT, "cf_column_sum: bad sizes");
    CF_REQUIRE(out && (N == 0 || g), CF_ERR_INVALID_ARGUMENT, "cf_column_sum: null pointer");
    column_sum_kernel<<<(int)((C + 15) / 16), 1024, 0, (hipStream_t)stream>>>(g, N, (int)C, out);
    CF_CHECK_LAUNCH("cf_column_sum");
    return CF_OK;
}

static int weight_grad_slices(int64_t N) { return N >= 512 ? 16 : (N >= 64 ? 4 : 1); }

extern "C" int64_t cf_linear_weight_grad_workspace(int64_t N, int64_t C, int64_t K)
{
    if (N < 0 || C < 1 || K < 1) return -1;
    return (int64_t)weight_grad_slices(N) * C * (K + 1) * (int64_t)sizeof(float);
}

extern "C" int cf_linear_weight_grad_grouped(int n_layers, const float *const *g, const float *const *x,
                                             const int64_t *N, const int64_t *C, const int64_t *K,
                                             float *const *gW, float *const *gb, void *workspace,
                                             int64_t workspace_bytes, void *stream);

extern "C" int cf_linear_weight_grad(const float *g, const float *x, int64_t N, int64_t C, int64_t K,
                                     void *workspace, int64_t workspace_bytes, float *gW, float *gb, void *stream)
{
    // a group of one layer: same kernels, same slicing, same summation order
    return cf_linear_weight_grad_grouped(1, &g, &x, &N, &C, &K, &gW, &gb, workspace, workspace_bytes, stream);
}

extern "C" int64_t cf_linear_weight_grad_grouped_workspace(int n_layers, const int64_t *N, const int64_t *C,
                                                           const int64_t *K)
{
    if (n_layers < 0 || (n_layers > 0 && (!N || !C || !K))) return -1;
    int64_t bytes = 0;
    for (int t = 0; t < n_layers; t++) {
        const int64_t b = cf_linear_weight_grad_workspace(N[t], C[t], K[t]);
        if (b < 0) return -1;
        bytes += b;
    }
    return bytes > 0 ? bytes : (int64_t)sizeof(float);
}

extern "C" int cf_linear_weight_grad_grouped(int n_layers, const float *const *g, const float *const *x,
                                             const int64_t *N, const int64_t *C, const int64_t *K,
                                             float *const *gW, float *const *gb, void *workspace,
                                             int64_t workspace_bytes, void *stream)
{
    CF_REQUIRE(n_layers >= 0, CF_ERR_INVALID_ARGUMENT, "cf_linear_weight_grad_grouped: negative layer count");
    if (n_layers == 0) return CF_OK;
    CF_REQUIRE(g && x && N && C && K && gW && gb, CF_ERR_INVALID_ARGUMENT,
               "cf_linear_weight_grad_grouped: null table");
    for (int t = 0; t < n_layers; t++) {
        CF_REQUIRE(N[t] >= 0 && N[t] < (1ll << 31) && C[t] >= 1 && K[t] >= 1 && C[t] < (1 << 20) && K[t] < (1 << 20),
                   CF_ERR_INVALID_ARGUMENT, "cf_linear_weight_grad_grouped: bad sizes of layer %d", t);
        CF_REQUIRE(gW[t] && (N[t] == 0 || (g[t] && x[t])), CF_ERR_INVALID_ARGUMENT,
                   "cf_linear_weight_grad_grouped: null pointer in layer %d", t);
    }
    const int64_t need = cf_linear_weight_grad_grouped_workspace(n_layers, N, C, K);
    CF_REQUIRE(workspace && workspace_bytes >= need, CF_ERR_INVALID_ARGUMENT,
               "cf_linear_weight_grad_grouped: workspace of %lld bytes needed", (long long)need);
    hipStream_t st = (hipStream_t)stream;
    int64_t off = 0;
    for (int first = 0; first < n_layers; first += WG_GROUP) {
        WeightGradGroup a;
        a.count = n_layers - first < WG_GROUP ? n_layers - first : WG_GROUP;
        a.part = (float *)workspace;
        int64_t tiles = 0, cells = 0;
        int max_slices = 1;
        for (int k = 0; k < WG_GROUP; k++) {
            const int t = first + k;
            const bool live = k < a.count;
            a.g[k] = live ? g[t] : nullptr;
            a.x[k] = live ? x[t] : nullptr;
            a.gw[k] = live ? gW[t] : nullptr;
            a.gb[k] = live ? gb[t] : nullptr;
            a.N[k] = live ? (int)N[t] : 0;
            a.C[k] = live ? (int)C[t] : 1;
            a.K[k] = live ? (int)K[t] : 1;
            a.slices[k] = live ? weight_grad_slices(N[t]) : 1;
            a.part_off[k] = off;
            a.tile0[k] = (int)tiles;
            a.cell0[k] = (int)cells;
            if (live) {
                off += cf_linear_weight_grad_workspace(N[t], C[t], K[t]) / (int64_t)sizeof(float);
                tiles += ((C[t] + WGT - 1) / WGT) * ((K[t] + WGT - 1) / WGT);
                cells += (C[t] * (K[t] + 1) + 255) / 256;
                if (a.slices[k] > max_slices) max_slices = a.slices[k];
                CF_REQUIRE(tiles < (1ll << 30) && cells < (1ll << 30), CF_ERR_UNSUPPORTED,
                           "cf_linear_weight_grad_grouped: too large");
            }
        }
        a.tile0[WG_GROUP] = (int)tiles;
        a.cell0[WG_GROUP] = (int)cells;
        weight_grad_group_slices_kernel<<<dim3((unsigned)tiles, (unsigned)max_slices), 256, 0, st>>>(a);
        CF_CHECK_LAUNCH("cf_linear_weight_grad_grouped: slices");
        weight_grad_group_add_kernel<<<(unsigned)cells, 256, 0, st>>>(a);
        CF_CHECK_LAUNCH("cf_linear_weight_grad_grouped: sum");
    }
    return CF_OK;
}
