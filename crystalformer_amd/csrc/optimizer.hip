// One training-step update for gfx950: global gradient-norm clip, AdamW and the inverse
// square-root learning-rate schedule over a list of small tensors (a few dozen, 128 to
// 65 536 elements each), as two kinds of launch instead of the hundred-odd element-wise
// launches of a per-tensor optimiser loop.  The step counter lives in device memory, so a
// captured graph of these launches advances it on every replay.
//
// Tensors are handed over by value in the kernel arguments, ADAM_GROUP at a time; a
// work-group owns one ADAM_CHUNK-element chunk of one tensor and finds it by scanning the
// group's chunk prefix (a scalar loop over at most ADAM_GROUP entries).  The model of the
// benchmark has 53 parameter tensors: one launch of each kind.
#include "cf_common.h"

namespace {

using namespace cf;

constexpr int ADAM_GROUP = 64;      // tensors per launch (kernel-argument table: 44 bytes each of the 4 KB)
constexpr int ADAM_CHUNK = 2048;    // elements per work-group: 256 threads x 8
constexpr int ADAM_THREADS = 256;

struct AdamGroup {                    // passed by value: has to fit the 4 KB of kernel arguments
    float *p[ADAM_GROUP];
    const float *g[ADAM_GROUP];
    float *m[ADAM_GROUP];
    float *v[ADAM_GROUP];
    int n[ADAM_GROUP];               // elements
    int chunk0[ADAM_GROUP + 1];      // first chunk of tensor t inside this launch
    float wd[ADAM_GROUP];            // decoupled weight decay
    int count;
    int first_partial;               // index of this launch's chunk 0 in the partial array
    int total_partials;              // chunks over all launches of the step
    int advance;                     // 1: this launch's work-group 0 advances the step counter
    float *partial;                  // (total_partials) sums of squares, one per chunk
    float *state;                    // [0] steps taken (counted as float), [1] gradient norm, [2] lr used
    float lr0, sch_decay, beta1, beta2, eps, clip_norm;
};
static_assert(sizeof(AdamGroup) <= 4096, "AdamGroup must fit the kernel-argument segment");

__device__ __forceinline__ float block_sum(float v, float *lds)
{
    v = wave_sum(v);
    const int wave = threadIdx.x >> 6;
    if ((threadIdx.x & 63) == 0) lds[wave] = v;
    __syncthreads();
    const float s = (lds[0] + lds[1]) + (lds[2] + lds[3]);
    __syncthreads();
    return s;
}

__device__ __forceinline__ int find_tensor(const AdamGroup &a, int chunk)
{
    int t = 0;
    while (t + 1 < a.count && a.chunk0[t + 1] <= chunk) t++;
    return t;
}

// Sum of squares of one chunk of one gradient, fixed order inside the chunk.
__global__ __launch_bounds__(ADAM_THREADS) void grad_sqnorm_kernel(AdamGroup a)
{
    __shared__ float lds[4];
    const int t = find_tensor(a, blockIdx.x);
    const int base = (blockIdx.x - a.chunk0[t]) * ADAM_CHUNK;
    const float *g = a.g[t];
    const int n = a.n[t];
    float s = 0.f;
#pragma unroll
    for (int u = 0; u < ADAM_CHUNK / ADAM_THREADS; u++) {
        const int x = base + u * ADAM_THREADS + threadIdx.x;
        const float gv = x < n ? g[x] : 0.f;
        s += gv * gv;
    }
    s = block_sum(s, lds);
    if (threadIdx.x == 0) {
        a.partial[a.first_partial + blockIdx.x] = s;
        if (a.advance && blockIdx.x == 0) a.state[0] += 1.f;     // read by the update launches only
    }
}

// Every work-group re-adds the chunk sums in one fixed order (identical in all of them), then
// updates its chunk: p *= 1 - lr wd; m += (g - m)(1 - b1); v = b2 v + (1 - b2) g g;
// p -= lr / (1 - b1^t) * m / (sqrt(v) / sqrt(1 - b2^t) + eps), g scaled by the clip factor first.
__global__ __launch_bounds__(ADAM_THREADS) void adamw_update_kernel(AdamGroup a)
{
    __shared__ float lds[4];
    float s = 0.f;
    for (int x = threadIdx.x; x < a.total_partials; x += ADAM_THREADS) s += a.partial[x];
    const float sq = block_sum(s, lds);
    const float norm = sqrtf(sq);
    float clip = 1.f;
    if (a.clip_norm > 0.f) clip = fminf(a.clip_norm / (norm + 1e-6f), 1.f);
    const float step = a.state[0];                               // 1-based number of this update
    const float lr = a.sch_decay > 0.f ? a.lr0 * sqrtf(a.sch_decay / (a.sch_decay + (step - 1.f))) : a.lr0;
    const float bc1 = (float)(1.0 - pow((double)a.beta1, (double)step));
    const float bc2 = (float)(1.0 - pow((double)a.beta2, (double)step));
    const float step_size = lr / bc1;
    const float bc2_sqrt = sqrtf(bc2);
    if (a.advance && blockIdx.x == 0 && threadIdx.x == 0) { a.state[1] = norm; a.state[2] = lr; }

    const int t = find_tensor(a, blockIdx.x);
    const int base = (blockIdx.x - a.chunk0[t]) * ADAM_CHUNK;
    float *p = a.p[t], *m = a.m[t], *v = a.v[t];
    const float *g = a.g[t];
    const int n = a.n[t];
    const float decay = 1.f - lr * a.wd[t];
    const float b1 = a.beta1, b2 = a.beta2;
#pragma unroll
    for (int u = 0; u < ADAM_CHUNK / ADAM_THREADS; u++) {
        const int x = base + u * ADAM_THREADS + threadIdx.x;
        if (x < n) {
            const float gv = g[x] * clip;
            float pv = p[x] * decay;
            float mv = m[x];
            mv = mv + (gv - mv) * (1.f - b1);
            const float vv = v[x] * b2 + (1.f - b2) * gv * gv;
            const float denom = sqrtf(vv) / bc2_sqrt + a.eps;
            pv = pv - step_size * (mv / denom);
            p[x] = pv;
            m[x] = mv;
            v[x] = vv;
        }
    }
}

int64_t chunks_of(int64_t n) { return (n + ADAM_CHUNK - 1) / ADAM_CHUNK; }

// Mean absolute error over the batch, summed over the targets, and its gradient, in one
// work-group: loss = (1/B) sum_b sum_i |pred[b,i] - target[b,i]|, grad = sign(pred - target) / B.
// Each thread adds its elements in ascending order, the threads are added in a fixed order.
__global__ __launch_bounds__(ADAM_THREADS) void l1_mean_loss_kernel(const float *pred, const float *target, int64_t B,
                                                                    int64_t total, float *loss, float *grad)
{
    __shared__ float lds[4];
    const float inv = 1.0f / (float)B;
    float s = 0.f;
    for (int64_t x = threadIdx.x; x < total; x += ADAM_THREADS) {
        const float d = pred[x] - target[x];
        s += fabsf(d);
        if (grad) grad[x] = d > 0.f ? inv : (d < 0.f ? -inv : 0.f);
    }
    s = block_sum(s, lds);
    if (threadIdx.x == 0) loss[0] = s * inv;
}

}  // namespace

extern "C" int64_t cf_adamw_step_workspace(int n_tensors, const int64_t *numel)
{
    if (n_tensors < 0 || (n_tensors > 0 && !numel)) return -1;
    int64_t chunks = 0;
    for (int t = 0; t < n_tensors; t++) {
        if (numel[t] < 0 || numel[t] > (1LL << 30)) return -1;
        chunks += chunks_of(numel[t]);
    }
    return (chunks > 0 ? chunks : 1) * (int64_t)sizeof(float);
}

extern "C" int cf_adamw_step(int n_tensors, float *const *params, const float *const *grads, float *const *exp_avg,
                             float *const *exp_avg_sq, const int64_t *numel, const float *weight_decay, float lr0,
                             float sch_decay, float beta1, float beta2, float eps, float clip_norm, float *state_3,
                             void *workspace, int64_t workspace_bytes, void *stream)
{
    CF_REQUIRE(n_tensors >= 0, CF_ERR_INVALID_ARGUMENT, "cf_adamw_step: negative tensor count");
    if (n_tensors == 0) return CF_OK;
    CF_REQUIRE(params && grads && exp_avg && exp_avg_sq && numel && weight_decay && state_3 && workspace,
               CF_ERR_INVALID_ARGUMENT, "cf_adamw_step: null pointer");
    CF_REQUIRE(beta1 >= 0.f && beta1 < 1.f && beta2 >= 0.f && beta2 < 1.f && eps >= 0.f && lr0 >= 0.f,
               CF_ERR_INVALID_ARGUMENT, "cf_adamw_step: bad hyper-parameters");
    const int64_t need = cf_adamw_step_workspace(n_tensors, numel);
    CF_REQUIRE(need > 0 && workspace_bytes >= need, CF_ERR_INVALID_ARGUMENT,
               "cf_adamw_step: workspace of %lld bytes needed", (long long)need);
    const int64_t total = need / (int64_t)sizeof(float);
    CF_REQUIRE(total < (1 << 24), CF_ERR_UNSUPPORTED, "cf_adamw_step: too many elements");
    for (int t = 0; t < n_tensors; t++)
        CF_REQUIRE(numel[t] == 0 || (params[t] && grads[t] && exp_avg[t] && exp_avg_sq[t]), CF_ERR_INVALID_ARGUMENT,
                   "cf_adamw_step: tensor %d has a null pointer", t);
    hipStream_t st = (hipStream_t)stream;

    // two passes over the same grouping: all norms first, then all updates
    for (int pass = 0; pass < 2; pass++) {
        int first_partial = 0;
        bool advance = true;
        int t = 0;
        while (t < n_tensors) {
            AdamGroup a;
            a.count = 0;
            int chunks = 0;
            for (; t < n_tensors && a.count < ADAM_GROUP; t++) {
                if (numel[t] == 0) continue;
                const int k = a.count++;
                a.p[k] = params[t];
                a.g[k] = grads[t];
                a.m[k] = exp_avg[t];
                a.v[k] = exp_avg_sq[t];
                a.n[k] = (int)numel[t];
                a.wd[k] = weight_decay[t];
                a.chunk0[k] = chunks;
                chunks += (int)chunks_of(numel[t]);
            }
            if (a.count == 0) break;
            for (int k = a.count; k <= ADAM_GROUP; k++) a.chunk0[k] = chunks;
            for (int k = a.count; k < ADAM_GROUP; k++) {
                a.p[k] = nullptr; a.g[k] = nullptr; a.m[k] = nullptr; a.v[k] = nullptr; a.n[k] = 0; a.wd[k] = 0.f;
            }
            a.first_partial = first_partial;
            a.total_partials = (int)total;
            a.advance = advance ? 1 : 0;
            a.partial = (float *)workspace;
            a.state = state_3;
            a.lr0 = lr0; a.sch_decay = sch_decay; a.beta1 = beta1; a.beta2 = beta2; a.eps = eps; a.clip_norm = clip_norm;
            if (pass == 0) {
                grad_sqnorm_kernel<<<chunks, ADAM_THREADS, 0, st>>>(a);
                CF_CHECK_LAUNCH("cf_adamw_step: norm");
            } else {
                adamw_update_kernel<<<chunks, ADAM_THREADS, 0, st>>>(a);
                CF_CHECK_LAUNCH("cf_adamw_step: update");
            }
            first_partial += chunks;
            advance = false;
        }
    }
    return CF_OK;
}

extern "C" int cf_l1_mean_loss(const float *pred, const float *target, int64_t B, int64_t T, float *loss, float *grad,
                               void *stream)
{
    CF_REQUIRE(B >= 1 && T >= 1 && B * T < (1ll << 40), CF_ERR_INVALID_ARGUMENT, "cf_l1_mean_loss: bad sizes B=%lld T=%lld",
               (long long)B, (long long)T);
    CF_REQUIRE(pred && target && loss, CF_ERR_INVALID_ARGUMENT, "cf_l1_mean_loss: null pointer");
    l1_mean_loss_kernel<<<1, ADAM_THREADS, 0, (hipStream_t)stream>>>(pred, target, B, B * T, loss, grad);
    CF_CHECK_LAUNCH("cf_l1_mean_loss");
    return CF_OK;
}
