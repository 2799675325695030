// Irregular (per-crystal) helpers for gfx950: mean pooling over the atoms of
// each crystal, its backward, and the dense intra-crystal edge list.
#include "cf_common.h"

namespace {

using namespace cf;

// One thread per (crystal, channel); atoms are summed in blocks of 8 combined
// by a fixed tree, blocks accumulated in order: deterministic and close to
// pairwise accuracy for crystals of any size.
__global__ void irregular_mean_fwd_kernel(const float *src, const int64_t *start_n, int64_t B, int64_t D,
                                          float *dst)
{
    int64_t tid = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (tid >= B * D) return;
    const int64_t n = tid / D, k = tid - n * D;
    const int64_t r0 = start_n[n], r1 = start_n[n + 1];
    const float *col = src + k;
    float total = 0.f;
    int64_t r = r0;
    for (; r + 8 <= r1; r += 8) {
        float t0 = col[r * D] + col[(r + 1) * D];
        float t1 = col[(r + 2) * D] + col[(r + 3) * D];
        float t2 = col[(r + 4) * D] + col[(r + 5) * D];
        float t3 = col[(r + 6) * D] + col[(r + 7) * D];
        total += (t0 + t1) + (t2 + t3);
    }
    float tail = 0.f;
    for (; r < r1; r++) tail += col[r * D];
    total += tail;
    dst[tid] = total / (float)(r1 - r0);
}

__global__ void irregular_mean_bwd_kernel(const float *go, const int64_t *batch_i, const int64_t *start_n,
                                          int64_t N, int64_t D, float *gx)
{
    int64_t tid = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (tid >= N * D) return;
    const int64_t i = tid / D, k = tid - i * D;
    const int64_t n = batch_i[i];
    gx[tid] = go[n * D + k] / (float)(start_n[n + 1] - start_n[n]);
}

// One thread per edge: locate the crystal by bisection over edge_start_n, then
// (i,j) = divmod(local edge, atoms in crystal).
// E is the row stride of `edges`; with `live_E` only the first *live_E edges exist.
__global__ void edge_index_kernel(const int64_t *atom_start, const int64_t *edge_start, int64_t B, int64_t E,
                                  const int64_t *live_E, const float *pos, int64_t *edges, float *rpos)
{
    int64_t e = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (e >= live_count(live_E, E)) return;
    const EdgeEnds r = edge_ends(atom_start, edge_start, B, e);
    const int64_t i = r.i, j = r.j;
    if (edges) {
        edges[e] = i;
        edges[E + e] = j;
    }
    if (pos && rpos) {
        rpos[e * 3 + 0] = pos[j * 3 + 0] - pos[i * 3 + 0];
        rpos[e * 3 + 1] = pos[j * 3 + 1] - pos[i * 3 + 1];
        rpos[e * 3 + 2] = pos[j * 3 + 2] - pos[i * 3 + 2];
    }
}

// Leading-zero cumulative sums of the crystal sizes, their squares and n (n + 1) / 2, in one
// work-group: each thread sums a contiguous run of crystals, the run totals are scanned in
// LDS, each thread then writes the prefixes of its run.
constexpr int SCAN_THREADS = 256;
// With `header` (4 words) the totals are left there for the kernels that follow: atoms, edges, atom
// pairs and a status word -- 0, or 1 with the three counts set to 0 when a size is negative or the
// totals exceed the capacities N_cap / E_cap (every kernel that reads the header then does nothing).
__global__ __launch_bounds__(SCAN_THREADS) void layout_scan_kernel(const int64_t *sizes, int64_t B, int64_t *atom_start,
                                                                   int64_t *edge_start, int64_t *unit_start,
                                                                   int64_t *header, int64_t N_cap, int64_t E_cap)
{
    __shared__ int64_t tot[3][SCAN_THREADS];
    __shared__ int64_t grand[3];
    __shared__ int negative;
    const int t = threadIdx.x;
    if (t == 0) negative = 0;
    __syncthreads();
    const int64_t run = (B + SCAN_THREADS - 1) / SCAN_THREADS;
    const int64_t b0 = min((int64_t)t * run, B), b1 = min(b0 + run, B);
    int64_t a = 0, e = 0, u = 0;
    bool neg = false;
    for (int64_t b = b0; b < b1; b++) {
        const int64_t n = sizes[b];
        neg = neg || n < 0 || n > (1ll << 24);
        a += n;
        e += n * n;
        u += n * (n + 1) / 2;
    }
    if (neg) atomicOr(&negative, 1);
    tot[0][t] = a; tot[1][t] = e; tot[2][t] = u;
    __syncthreads();
    if (t < 3) {                                     // exclusive scan of one row per thread
        int64_t acc = 0;
        for (int x = 0; x < SCAN_THREADS; x++) {
            const int64_t v = tot[t][x];
            tot[t][x] = acc;
            acc += v;
        }
        grand[t] = acc;
    }
    __syncthreads();
    // (with a header the capacities bind: a batch beyond them is turned into one of empty crystals,
    // so that nothing downstream indexes past a buffer)
    const bool ok = !header || (!negative && grand[0] <= N_cap && grand[1] <= E_cap);
    if (header && t == 0) {
        header[0] = ok ? grand[0] : 0;
        header[1] = ok ? grand[1] : 0;
        header[2] = ok ? grand[2] : 0;
        header[3] = ok ? 0 : 1;
    }
    a = tot[0][t]; e = tot[1][t]; u = tot[2][t];
    if (t == 0) atom_start[0] = edge_start[0] = unit_start[0] = 0;
    for (int64_t b = b0; b < b1; b++) {
        const int64_t n = sizes[b];
        a += n;
        e += n * n;
        u += n * (n + 1) / 2;
        atom_start[b + 1] = ok ? a : 0;
        edge_start[b + 1] = ok ? e : 0;
        unit_start[b + 1] = ok ? u : 0;
    }
}

// CSR offsets of the atoms' edge rows in the dense blocks: atom i of crystal b (found by
// bisection) starts at edge_start[b] + (i - atom_start[b]) n_b; entry N is the edge count.
__global__ void layout_rows_kernel(const int64_t *atom_start, const int64_t *edge_start, int64_t B, int64_t N_cap,
                                   const int64_t *live_N, int64_t *e_start, int64_t *batch)
{
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    const int64_t N = live_count(live_N, N_cap);
    if (i > N) return;
    if (i == N) {
        e_start[N] = edge_start[B];
        return;
    }
    int64_t lo;
    e_start[i] = row_start(atom_start, edge_start, B, i, &lo);
    if (batch) batch[i] = lo;
}

// Up to COPY_SEGMENTS device-to-device copies (or zero fills, src == NULL) in one launch: a
// work-group strides over the 16-byte pieces of every segment, bytes beyond the last whole piece
// (and segments that are not 16-byte aligned) go one at a time.
constexpr int COPY_SEGMENTS = 8;
struct CopyTable {
    const unsigned char *src[COPY_SEGMENTS];
    unsigned char *dst[COPY_SEGMENTS];
    int64_t bytes[COPY_SEGMENTS];
    int n;
};

__global__ __launch_bounds__(256) void copy_segments_kernel(CopyTable t)
{
    typedef unsigned int uint4_v __attribute__((ext_vector_type(4)));
    const int64_t tid = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    const int64_t nthreads = (int64_t)gridDim.x * blockDim.x;
    for (int s = 0; s < t.n; s++) {
        const unsigned char *src = t.src[s];
        unsigned char *dst = t.dst[s];
        const int64_t bytes = t.bytes[s];
        const bool aligned = (((uintptr_t)src | (uintptr_t)dst) & 15) == 0;
        const int64_t pieces = aligned ? bytes / 16 : 0;
        const uint4_v zero = {0u, 0u, 0u, 0u};
        for (int64_t x = tid; x < pieces; x += nthreads)
            reinterpret_cast<uint4_v *>(dst)[x] = src ? reinterpret_cast<const uint4_v *>(src)[x] : zero;
        for (int64_t x = pieces * 16 + tid; x < bytes; x += nthreads) dst[x] = src ? src[x] : (unsigned char)0;
    }
}

}  // namespace

extern "C" int cf_irregular_mean_fwd(const float *src, const int64_t *start_n, int64_t B, int64_t D,
                                     float *dst, void *stream)
{
    CF_REQUIRE(B >= 0 && D >= 0, CF_ERR_INVALID_ARGUMENT, "cf_irregular_mean_fwd: negative size");
    if (B * D == 0) return CF_OK;
    CF_REQUIRE(src && start_n && dst, CF_ERR_INVALID_ARGUMENT, "cf_irregular_mean_fwd: null pointer");
    int64_t total = B * D;
    irregular_mean_fwd_kernel<<<(int)((total + 127) / 128), 128, 0, (hipStream_t)stream>>>(src, start_n, B, D, dst);
    CF_CHECK_LAUNCH("cf_irregular_mean_fwd");
    return CF_OK;
}

extern "C" int cf_irregular_mean_bwd(const float *go, const int64_t *batch_i, const int64_t *start_n,
                                     int64_t N, int64_t D, float *gx, void *stream)
{
    CF_REQUIRE(N >= 0 && D >= 0, CF_ERR_INVALID_ARGUMENT, "cf_irregular_mean_bwd: negative size");
    if (N * D == 0) return CF_OK;
    CF_REQUIRE(go && batch_i && start_n && gx, CF_ERR_INVALID_ARGUMENT, "cf_irregular_mean_bwd: null pointer");
    int64_t total = N * D;
    irregular_mean_bwd_kernel<<<(int)((total + 255) / 256), 256, 0, (hipStream_t)stream>>>(go, batch_i, start_n,
                                                                                          N, D, gx);
    CF_CHECK_LAUNCH("cf_irregular_mean_bwd");
    return CF_OK;
}

extern "C" int cf_edge_index(const int64_t *atom_start_n, const int64_t *edge_start_n, int64_t B, int64_t E,
                             const float *pos, int64_t *edge_ij_e, float *rpos_ij_e, void *stream)
{
    CF_REQUIRE(B >= 0 && E >= 0, CF_ERR_INVALID_ARGUMENT, "cf_edge_index: negative size");
    if (E == 0) return CF_OK;
    CF_REQUIRE(B > 0 && atom_start_n && edge_start_n, CF_ERR_INVALID_ARGUMENT,
               "cf_edge_index: null pointer or no crystals");
    CF_REQUIRE(edge_ij_e || (pos && rpos_ij_e), CF_ERR_INVALID_ARGUMENT, "cf_edge_index: no output requested");
    edge_index_kernel<<<(int)((E + 255) / 256), 256, 0, (hipStream_t)stream>>>(atom_start_n, edge_start_n, B, E,
                                                                              cf::live_edges(E), pos, edge_ij_e,
                                                                              rpos_ij_e);
    CF_CHECK_LAUNCH("cf_edge_index");
    return CF_OK;
}

extern "C" int cf_copy_segments(int n_segments, const void *const *src, void *const *dst, const int64_t *bytes,
                                void *stream)
{
    CF_REQUIRE(n_segments >= 0 && n_segments <= COPY_SEGMENTS, CF_ERR_INVALID_ARGUMENT,
               "cf_copy_segments: 0..%d segments, got %d", COPY_SEGMENTS, n_segments);
    CF_REQUIRE(n_segments == 0 || (src && dst && bytes), CF_ERR_INVALID_ARGUMENT, "cf_copy_segments: null table");
    CopyTable t{};
    int64_t most = 0;
    for (int s = 0; s < n_segments; s++) {
        CF_REQUIRE(bytes[s] >= 0 && (bytes[s] == 0 || dst[s]), CF_ERR_INVALID_ARGUMENT,
                   "cf_copy_segments: segment %d has no destination or a negative size", s);
        if (bytes[s] == 0) continue;
        t.src[t.n] = (const unsigned char *)src[s];
        t.dst[t.n] = (unsigned char *)dst[s];
        t.bytes[t.n] = bytes[s];
        most = bytes[s] > most ? bytes[s] : most;
        t.n++;
    }
    if (t.n == 0) return CF_OK;
    int64_t blocks = (most / 16 + 255) / 256;
    blocks = blocks < 1 ? 1 : (blocks > 1024 ? 1024 : blocks);
    copy_segments_kernel<<<(int)blocks, 256, 0, (hipStream_t)stream>>>(t);
    CF_CHECK_LAUNCH("cf_copy_segments");
    return CF_OK;
}

extern "C" int cf_batch_layout(const int64_t *sizes_n, int64_t B, int64_t N, int64_t E, int64_t *atom_start_n,
                               int64_t *edge_start_n, int64_t *unit_start_n, int64_t *e_start_i, int64_t *edge_ij_e,
                               int64_t *pairs_u, int64_t *batch_i, void *stream)
{
    CF_REQUIRE(B >= 1 && N >= 1 && E >= 1, CF_ERR_INVALID_ARGUMENT, "cf_batch_layout: B, N and E must be positive");
    CF_REQUIRE(sizes_n && atom_start_n && edge_start_n && unit_start_n && e_start_i && edge_ij_e,
               CF_ERR_INVALID_ARGUMENT, "cf_batch_layout: null pointer");
    CF_REQUIRE(N < (1ll << 31) * 256, CF_ERR_UNSUPPORTED, "cf_batch_layout: too many atoms");
    hipStream_t st = (hipStream_t)stream;
    // with a size header set for these capacities the totals are whatever `sizes_n` holds when the
    // kernels run: the scan leaves them in the header and everything downstream reads them there
    int64_t *header = cf::size_header_for_layout(N, E);
    layout_scan_kernel<<<1, SCAN_THREADS, 0, st>>>(sizes_n, B, atom_start_n, edge_start_n, unit_start_n, header, N, E);
    CF_CHECK_LAUNCH("cf_batch_layout: scan");
    layout_rows_kernel<<<(int)((N + 1 + 255) / 256), 256, 0, st>>>(atom_start_n, edge_start_n, B, N,
                                                                    header, e_start_i, batch_i);
    CF_CHECK_LAUNCH("cf_batch_layout: rows");
    int rc = cf_edge_index(atom_start_n, edge_start_n, B, E, nullptr, edge_ij_e, nullptr, stream);
    if (rc) return rc;
    if (pairs_u) rc = cf_edge_pairs(atom_start_n, edge_start_n, unit_start_n, B, E, pairs_u, stream);
    return rc;
}
