// hip_train.inl — the batched training step on the device: forward keeping every layer, output and
// hidden deltas, weight and bias gradients, optional clipping by the global norm, one of five
// optimizer updates.  Part of hip_forward.hip's translation unit (included near its end): it uses
// that file's device helpers, launch wrappers and net structure.
//
// What the reference does per step (Src/Spingalett.Training.c): batch_forward :313-345,
// batch_compute_deltas :347-394 (one sgemm NN per hidden layer + apply_derivative_batch),
// batch_accumulate_gradients :396-419 (one sgemm TN + one sgemv T per layer),
// apply_gradients_batch_prescaled :439-507 with the update rules of Src/Spingalett.SIMD.c:279-520.
// Everything stays FP32, as there: products on the FP32 matrix cores, sums in FP32.

namespace {

enum { TR_EPI_DELTA = 0, TR_EPI_SCALE = 1 };

// derivative of an activation as a function of its output (Activation.c:40-56, SIMD.c:90-188)
__device__ __forceinline__ float act_derivative(float a, int act)
{
    switch (act) {
    case A_RELU:    return a > 0.0f ? 1.0f : 0.0f;
    case A_LEAKY:   return a > 0.0f ? 1.0f : 0.01f;
    case A_SIGMOID:
    case A_SOFTMAX: return a * (1.0f - a);
    case A_TANH:    return 1.0f - a * a;
    case A_FOO52:   return (a > 1.0f || a < 0.0f) ? 0.01f : 1.0f;
    default:        return 1.0f;
    }
}

struct TrGemmArgs {
    const float *A, *B;
    float *C;              // [M][N]
    float *ws;             // [splits][M][N] partial sums when the grid splits K, else nullptr
    const float *aux;      // TR_EPI_DELTA: activations [M][N] whose derivative multiplies the product
    uint32_t M, N, K, lda, ldb;
    uint32_t kper;         // k range of one split (multiple of 32)
    int act;               // TR_EPI_DELTA: activation kind of aux
    float scale;           // TR_EPI_SCALE
    int vecA, vecB;        // operand may be read as float4 (leading dimension and base 16-byte aligned)
};

// C[m][n] = sum_k A(m, k) B(n, k) on the FP32 matrix cores.  Tile (64 TM) x (64 TM) x 32, four waves in a
// 2 x 2 grid, TM x TM 32 x 32 accumulators per wave (TM is fixed to 1 below).  Each operand is either k-contiguous (element (r, k) at
// r * ld + k; LDS tile [row][33]) or row-contiguous (element (r, k) at k * ld + r; LDS tile [k][64 TM + 32]):
// the hidden deltas read the weights row-contiguous, the gradients read both operands so.  Both LDS layouts
// are conflict-free for the matrix-core operand reads (lane -> row, half-wave -> k).
template <bool AMC, bool BMC, int EPI>
__global__ __launch_bounds__(256) void sp_train_gemm32(const TrGemmArgs g)
{
    // TM = 2 (128 x 128 tiles) was measured on the 784-512-1000-10 net at batch 20000: 255 us against 227 us for the
    // 20000 x 512 x 1000 product (628 large tiles fill 256 compute units unevenly), no gain on the gradient products.
    constexpr int TM = 1;
    constexpr int BM = 64 * TM, BN = 64 * TM, BK = 32, LDK = BK + 1, LDM = BM + 32;
    constexpr int TILE = BK * LDM > BM * LDK ? BK * LDM : BM * LDK;
    constexpr int PIECES = BM * BK / 4 / 256;            // float4 pieces per thread and operand
    __shared__ __attribute__((aligned(16))) float As[TILE];
    __shared__ __attribute__((aligned(16))) float Bs[TILE];
    const uint32_t M = g.M, N = g.N, K = g.K;
    const int t = threadIdx.x, lane = t & 63, wave = t >> 6;
    const int wm = wave >> 1, wn = wave & 1;
    const uint32_t tiles_n = (N + BN - 1) / BN;
    // consecutive workgroups go to different XCDs: give each XCD a contiguous run of tiles, so that the tiles that
    // share a row panel of A meet in one L2
    uint32_t bid = blockIdx.x;
    {
        const uint32_t per = gridDim.x / 8u;
        if (bid < per * 8u) bid = (bid & 7u) * per + (bid >> 3);
    }
    const uint32_t m0 = (bid / tiles_n) * BM, n0 = (bid % tiles_n) * BN;
    const uint32_t kbeg = blockIdx.y * g.kper;
    const uint32_t kend = kbeg + g.kper < K ? kbeg + g.kper : K;

    f32x16 acc[TM][TM];
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TM; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.0f;

    // four consecutive elements starting at p, of which the first `valid` exist
    auto load4 = [](const float *p, bool vec, int valid) -> float4 {
        if (vec && valid >= 4) return *reinterpret_cast<const float4 *>(p);
        float v[4] = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
        for (int e = 0; e < 4; ++e)
            if (e < valid) v[e] = p[e];
        return make_float4(v[0], v[1], v[2], v[3]);
    };
    // piece p of a tile: k-contiguous -> row p / 8, k (p % 8) * 4; row-contiguous -> k p / (BM / 4), row (p % (BM / 4)) * 4
    auto fetch_one = [&](const float *base, uint32_t ld, bool mc, bool vec, uint32_t r0, uint32_t R, uint32_t k0, int p) -> float4 {
        if (mc) {
            const uint32_t k = k0 + (uint32_t)(p / (BM / 4)), r = r0 + (uint32_t)(p % (BM / 4)) * 4u;
            const int valid = (k < kend && r < R) ? (int)(R - r < 4u ? R - r : 4u) : 0;
            return load4(base + (size_t)(k < K ? k : K - 1) * ld + (r < R ? r : 0u), vec, valid);
        }
        const uint32_t r = r0 + (uint32_t)(p >> 3), k = k0 + (uint32_t)(p & 7) * 4u;
        const int valid = (r < R && k < kend) ? (int)(kend - k < 4u ? kend - k : 4u) : 0;
        return load4(base + (size_t)(r < R ? r : R - 1) * ld + (k < kend ? k : 0u), vec, valid);
    };
    float4 ra[PIECES], rb[PIECES];
    auto fetch = [&](uint32_t k0) {
#pragma unroll
        for (int i = 0; i < PIECES; ++i) {
            ra[i] = fetch_one(g.A, g.lda, AMC, g.vecA != 0, m0, M, k0, t + 256 * i);
            rb[i] = fetch_one(g.B, g.ldb, BMC, g.vecB != 0, n0, N, k0, t + 256 * i);
        }
    };
    auto stash_one = [&](float *tile, bool mc, const float4 &v, int p) {
        if (mc) {
            *reinterpret_cast<float4 *>(tile + (p / (BM / 4)) * LDM + (p % (BM / 4)) * 4) = v;
        } else {
            float *d = tile + (p >> 3) * LDK + (p & 7) * 4;
            d[0] = v.x; d[1] = v.y; d[2] = v.z; d[3] = v.w;
        }
    };
    auto stash = [&]() {
#pragma unroll
        for (int i = 0; i < PIECES; ++i) {
            stash_one(As, AMC, ra[i], t + 256 * i);
            stash_one(Bs, BMC, rb[i], t + 256 * i);
        }
    };

    fetch(kbeg);
    for (uint32_t k0 = kbeg; k0 < kend; k0 += BK) {
        stash();
        __syncthreads();
        if (k0 + BK < kend) fetch(k0 + BK);
#pragma unroll
        for (int ks = 0; ks < BK; ks += 2) {
            const int k = ks + (lane >> 5);
            float a[TM], b[TM];
#pragma unroll
            for (int i = 0; i < TM; ++i) {
                const int ar = (wm * TM + i) * 32 + (lane & 31), br = (wn * TM + i) * 32 + (lane & 31);
                a[i] = AMC ? As[k * LDM + ar] : As[ar * LDK + k];
                b[i] = BMC ? Bs[k * LDM + br] : Bs[br * LDK + k];
            }
#pragma unroll
            for (int i = 0; i < TM; ++i)
#pragma unroll
                for (int j = 0; j < TM; ++j) acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[i], b[j], acc[i][j], 0, 0, 0);
        }
        __syncthreads();
    }

#pragma unroll
    for (int j = 0; j < TM; ++j) {
        const uint32_t col = n0 + (wn * TM + j) * 32 + (lane & 31);
        if (col >= N) continue;
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const uint32_t row = m0 + (wm * TM + i) * 32 + 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3);
                if (row >= M) continue;
                const size_t o = (size_t)row * N + col;
                if (g.ws) g.ws[(size_t)blockIdx.y * M * N + o] = acc[i][j][r];
                else if (EPI == TR_EPI_DELTA) g.C[o] = acc[i][j][r] * act_derivative(g.aux[o], g.act);
                else g.C[o] = g.scale * acc[i][j][r];
            }
    }
}

// adds the K splits of sp_train_gemm32 in split order and applies its epilogue
template <int EPI>
__global__ __launch_bounds__(256) void sp_train_gemm32_reduce(const TrGemmArgs g, uint32_t splits)
{
    const uint64_t idx = (uint64_t)blockIdx.x * 256u + threadIdx.x;
    const uint64_t total = (uint64_t)g.M * g.N;
    if (idx >= total) return;
    float sum = 0.0f;
    for (uint32_t sp = 0; sp < splits; ++sp) sum += g.ws[(uint64_t)sp * total + idx];
    if (EPI == TR_EPI_DELTA) g.C[idx] = sum * act_derivative(g.aux[idx], g.act);
    else g.C[idx] = g.scale * sum;
}

// Deltas of the output layer (Training.c:357-378), one wavefront per sample.
//   mode 0: squared error through a softmax: d_j = a_j ((a_j - t_j) - sum_i (a_i - t_i) a_i)
//   mode 1: cross-entropy through softmax / sigmoid: d = a - t
//   mode 2: every other combination: d = (a - t) f'(a)
__global__ __launch_bounds__(256) void sp_train_out_delta(const float *__restrict__ a, const float *__restrict__ tg,
                                                          float *__restrict__ d, uint32_t n, uint32_t width, int mode, int act)
{
    const int lane = threadIdx.x & 63;
    const uint32_t row = blockIdx.x * 4u + (threadIdx.x >> 6);
    if (row >= n) return;
    const float *ar = a + (size_t)row * width, *tr = tg + (size_t)row * width;
    float *dr = d + (size_t)row * width;
    float sum = 0.0f;
    if (mode == 0) {
        for (uint32_t j = lane; j < width; j += kWave) sum += (ar[j] - tr[j]) * ar[j];
        sum = wave_sum(sum);
    }
    for (uint32_t j = lane; j < width; j += kWave) {
        const float av = ar[j], diff = av - tr[j];
        dr[j] = mode == 0 ? av * (diff - sum) : mode == 1 ? diff : diff * act_derivative(av, act);
    }
}

// Column sums of delta [n][width] (the sgemv against a vector of ones, Training.c:412-417) in two
// passes: kColsumRows rows per workgroup into part[chunk][col], then the chunks in order, times scale.
constexpr uint32_t kColsumRows = 256;
__global__ __launch_bounds__(256) void sp_train_colsum_part(const float *__restrict__ d, float *__restrict__ part, uint32_t n,
                                                            uint32_t width)
{
    __shared__ float s[4][64];
    const int c = threadIdx.x & 63, rl = threadIdx.x >> 6;
    const uint32_t col = blockIdx.x * 64u + c;
    const uint32_t r0 = blockIdx.y * kColsumRows, r1 = r0 + kColsumRows < n ? r0 + kColsumRows : n;
    float sum = 0.0f;
    if (col < width) {
        // four independent partial sums keep four loads in flight per lane
        float p[4] = {0.0f, 0.0f, 0.0f, 0.0f};
        uint32_t r = r0 + rl;
        for (; r + 12u < r1; r += 16u) {
#pragma unroll
            for (int u = 0; u < 4; ++u) p[u] += d[(size_t)(r + 4u * u) * width + col];
        }
        for (; r < r1; r += 4u) p[0] += d[(size_t)r * width + col];
        sum = (p[0] + p[1]) + (p[2] + p[3]);
    }
    s[rl][c] = sum;
    __syncthreads();
    if (rl == 0 && col < width) part[(size_t)blockIdx.y * width + col] = (s[0][c] + s[1][c]) + (s[2][c] + s[3][c]);
}

__global__ __launch_bounds__(256) void sp_train_colsum_fin(const float *__restrict__ part, float *__restrict__ out, uint32_t chunks,
                                                           uint32_t width, float scale)
{
    const uint32_t col = blockIdx.x * 256u + threadIdx.x;
    if (col >= width) return;
    // eight independent sums keep eight loads in flight (the chunks are added in a fixed order all the same)
    float p[8] = {0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f};
    uint32_t ch = 0;
    for (; ch + 8u <= chunks; ch += 8u) {
#pragma unroll
        for (int u = 0; u < 8; ++u) p[u] += part[(size_t)(ch + u) * width + col];
    }
    for (; ch < chunks; ++ch) p[0] += part[(size_t)ch * width + col];
    out[col] = scale * (((p[0] + p[1]) + (p[2] + p[3])) + ((p[4] + p[5]) + (p[6] + p[7])));
}

// Sum of squares of one array in FP64, one value per workgroup (first pass of clip_grad_norm, SIMD.c:496-520)
__global__ __launch_bounds__(256) void sp_train_sumsq_part(const float *__restrict__ g, uint64_t cnt, double *__restrict__ part)
{
    __shared__ double s[4];
    double sum = 0.0;
    for (uint64_t i = (uint64_t)blockIdx.x * 256u + threadIdx.x; i < cnt; i += (uint64_t)gridDim.x * 256u) sum += (double)g[i] * (double)g[i];
#pragma unroll
    for (int sft = 32; sft > 0; sft >>= 1) sum += __shfl_xor(sum, sft, kWave);
    if ((threadIdx.x & 63) == 0) s[threadIdx.x >> 6] = sum;
    __syncthreads();
    if (threadIdx.x == 0) part[blockIdx.x] = (s[0] + s[1]) + (s[2] + s[3]);
}

// scal[0] = factor the gradients are multiplied by (max_norm / norm when the norm exceeds max_norm, else 1), scal[1] = norm
__global__ __launch_bounds__(64) void sp_train_clip_fin(const double *__restrict__ part, uint32_t count, float max_norm, float *__restrict__ scal)
{
    double sum = 0.0;
    for (uint32_t i = threadIdx.x; i < count; i += kWave) sum += part[i];
#pragma unroll
    for (int sft = 32; sft > 0; sft >>= 1) sum += __shfl_xor(sum, sft, kWave);
    if (threadIdx.x == 0) {
        const float norm = sqrtf((float)sum);
        scal[0] = norm > max_norm ? max_norm / norm : 1.0f;
        scal[1] = norm;
    }
}

struct OptArgs {
    float *W, *g, *m, *v;
    uint64_t cnt;
    const float *clip;     // device scalar the gradient is multiplied by first, or nullptr
    int opt;               // OptimizerType, Spingalett.h:76-83
    int decay_in_grad;     // RMSprop: decay * W joins the gradient before the second moment (per-sample rule)
    float lr, decay, momentum, b1, b2, omb1, omb2, mf, vf, eps;
};

// One optimizer step over one array: the scalar forms of SIMD.c:279-494 as called from
// apply_gradients_batch_prescaled (Training.c:439-507).  The gradient array keeps what the reference
// leaves in it (clipped, and with decay * W added for Adam with weight decay).
__global__ __launch_bounds__(256) void sp_train_opt(const OptArgs a)
{
    const uint64_t i = (uint64_t)blockIdx.x * 256u + threadIdx.x;
    if (i >= a.cnt) return;
    float w = a.W[i], g = a.g[i];
    if (a.clip) { g *= *a.clip; a.g[i] = g; }
    switch (a.opt) {
    case 0:     // SGD
        w -= a.lr * (a.decay > 0.0f ? g + a.decay * w : g);
        break;
    case 1: {   // momentum
        const float m = a.momentum * a.m[i] + a.decay * w + g;
        a.m[i] = m;
        w -= a.lr * m;
        break;
    }
    case 2: {   // RMSprop
        if (a.decay_in_grad && a.decay > 0.0f) g += a.decay * w;
        const float v = a.b2 * a.v[i] + a.omb2 * (g * g);
        a.v[i] = v;
        w -= a.decay_in_grad ? a.lr * g / sqrtf(v + a.eps) : a.lr * (a.decay * w + g / sqrtf(v + a.eps));
        break;
    }
    default: {  // Adam (3): decay joins the gradient; AdamW (4): decay shrinks the weight
        const bool adamw = a.opt == 4;
        if (!adamw && a.decay > 0.0f) { g += a.decay * w; a.g[i] = g; }
        const float m = a.b1 * a.m[i] + a.omb1 * g;
        const float v = a.b2 * a.v[i] + a.omb2 * (g * g);
        a.m[i] = m;
        a.v[i] = v;
        const float step = a.lr * ((m * a.mf) / sqrtf(v * a.vf + a.eps));
        w = (adamw && a.decay > 0.0f) ? w * (1.0f - a.lr * a.decay) - step : w - step;
        break;
    }
    }
    a.W[i] = w;
}

__global__ __launch_bounds__(256) void sp_train_fill0(float *p, uint64_t cnt)
{
    const uint64_t i = (uint64_t)blockIdx.x * 256u + threadIdx.x;
    if (i < cnt) p[i] = 0.0f;
}

}  // namespace

// Device state of a net being trained: gradients and optimizer moments laid out like the host net's
// flat arrays (layer l at woff[l] / boff[l]), activations and deltas of every layer for the largest
// batch seen so far.
struct sphip_train_state {
    std::vector<uint64_t> woff, boff;
    uint64_t total_w = 0, total_b = 0;
    float *gW = nullptr, *gB = nullptr, *mW = nullptr, *vW = nullptr, *mB = nullptr, *vB = nullptr;
    uint32_t cap_n = 0;
    std::vector<float *> act, delta;       // [layers]; act[0] stages host inputs, delta[0] is unused
    float *targets = nullptr;              // staged host targets [cap_n][topo[last]]
    uint32_t staged_n = 0;                 // samples of the batch staged last (0: none)
    float *ws = nullptr;                   // split-K partials, column-sum partials
    uint64_t ws_cap = 0;
    double *sq_part = nullptr;             // per-workgroup sums of squares (clipping)
    float *scal = nullptr;                 // clip factor, gradient norm
    float *loss_buf = nullptr;             // per-sample loss / prediction / hit, totals
    uint64_t loss_cap = 0;
};

namespace {

constexpr uint32_t kSqBlocks = 1024;

void train_free(sphip_net *net)
{
    sphip_train_state *ts = net->train;
    if (!ts) return;
    float *flat[] = {ts->gW, ts->gB, ts->mW, ts->vW, ts->mB, ts->vB, ts->targets, ts->ws, ts->scal, ts->loss_buf};
    for (float *p : flat) if (p) (void)hipFree(p);
    if (ts->sq_part) (void)hipFree(ts->sq_part);
    for (float *p : ts->act) if (p) (void)hipFree(p);
    for (float *p : ts->delta) if (p) (void)hipFree(p);
    delete ts;
    net->train = nullptr;
}

int train_reserve(sphip_net *net, uint32_t n)
{
    sphip_train_state *ts = net->train;
    if (n > ts->cap_n) {
        for (uint32_t l = 0; l < net->layers; ++l) {
            if (ts->act[l]) { HCHECK(hipFree(ts->act[l])); ts->act[l] = nullptr; }
            if (ts->delta[l]) { HCHECK(hipFree(ts->delta[l])); ts->delta[l] = nullptr; }
        }
        if (ts->targets) { HCHECK(hipFree(ts->targets)); ts->targets = nullptr; }
        ts->cap_n = 0;
        ts->staged_n = 0;
        for (uint32_t l = 0; l < net->layers; ++l) {
            HCHECK(hipMalloc((void **)&ts->act[l], (size_t)n * net->topo[l] * sizeof(float)));
            if (l) HCHECK(hipMalloc((void **)&ts->delta[l], (size_t)n * net->topo[l] * sizeof(float)));
        }
        HCHECK(hipMalloc((void **)&ts->targets, (size_t)n * net->topo[net->layers - 1] * sizeof(float)));
        ts->cap_n = n;
    }
    // workspace: K splits of the delta and gradient products, column-sum partials
    uint64_t ws = 0;
    uint32_t kper = 0;
    for (uint32_t l = 1; l + 1 < net->layers; ++l) {
        const uint32_t sp = gemm32_splits(n, net->topo[l], net->topo[l + 1], &kper);
        if (sp > 1 && (uint64_t)sp * n * net->topo[l] > ws) ws = (uint64_t)sp * n * net->topo[l];
    }
    for (uint32_t l = 0; l + 1 < net->layers; ++l) {
        const uint32_t sp = gemm32_splits(net->topo[l + 1], net->topo[l], n, &kper);
        const uint64_t wcnt = (uint64_t)net->topo[l] * net->topo[l + 1];
        if (sp > 1 && sp * wcnt > ws) ws = sp * wcnt;
        const uint64_t cs = (uint64_t)((n + kColsumRows - 1) / kColsumRows) * net->topo[l + 1];
        if (cs > ws) ws = cs;
    }
    if (grow(&ts->ws, &ts->ws_cap, ws)) return 1;
    return 0;
}

template <bool AMC, bool BMC, int EPI>
void launch_train_gemm(TrGemmArgs g, float *ws, uint64_t ws_floats)
{
    uint32_t splits = gemm32_splits(g.M, g.N, g.K, &g.kper);
    if (splits > 1 && (uint64_t)splits * g.M * g.N > ws_floats) { splits = 1; g.kper = (g.K + 31u) / 32u * 32u; }
    g.ws = splits > 1 ? ws : nullptr;
    g.vecA = g.lda % 4u == 0 && (reinterpret_cast<uintptr_t>(g.A) & 15u) == 0;
    g.vecB = g.ldb % 4u == 0 && (reinterpret_cast<uintptr_t>(g.B) & 15u) == 0;
    const dim3 grid(((g.M + 63) / 64) * ((g.N + 63) / 64), splits);
    sp_train_gemm32<AMC, BMC, EPI><<<grid, 256, 0, g_stream>>>(g);
    if (splits > 1)
        sp_train_gemm32_reduce<EPI><<<(uint32_t)(((uint64_t)g.M * g.N + 255) / 256), 256, 0, g_stream>>>(g, splits);
}

void launch_opt(const sphip_train_args &a, float *W, float *g, float *m, float *v, uint64_t cnt, float decay, const float *clip)
{
    OptArgs o{};
    o.W = W; o.g = g; o.m = m; o.v = v; o.cnt = cnt; o.clip = clip;
    o.opt = a.optimizer;
    o.decay_in_grad = a.decay_in_grad;
    o.lr = a.learning_rate; o.decay = decay; o.momentum = a.momentum;
    o.b1 = a.beta1; o.b2 = a.beta2;
    // formed in FP32 like the reference's locals (Training.c:447-448, 479-480)
    o.omb1 = 1.0f - a.beta1;
    o.omb2 = 1.0f - a.beta2;
    o.mf = 1.0f / (1.0f - a.beta1_pow_t);
    o.vf = 1.0f / (1.0f - a.beta2_pow_t);
    o.eps = a.epsilon;
    sp_train_opt<<<(uint32_t)((cnt + 255) / 256), 256, 0, g_stream>>>(o);
}

}  // namespace

extern "C" {

int sphip_train_begin(sphip_net *net)
{
    if (!net) return fail_msg("sphip_train_begin: invalid argument");
    if (net->prec != F32) return fail_msg("sphip_train_begin: training needs the FP32 arrays on the device (this net holds a packed format)");
    for (uint32_t l = 1; l + 1 < net->layers; ++l)
        if (net->act[l - 1] == A_SOFTMAX) return fail_msg("sphip_train_begin: softmax is not supported in hidden layers");
    if (check_uploaded(net)) return 1;
    if (net->train) return 0;
    sphip_train_state *ts = new (std::nothrow) sphip_train_state;
    if (!ts) return fail_msg("sphip_train_begin: out of host memory");
    net->train = ts;
    ts->act.assign(net->layers, nullptr);
    ts->delta.assign(net->layers, nullptr);
    for (uint32_t l = 0; l + 1 < net->layers; ++l) {
        ts->woff.push_back(ts->total_w);
        ts->boff.push_back(ts->total_b);
        ts->total_w += (uint64_t)net->topo[l] * net->topo[l + 1];
        ts->total_b += net->topo[l + 1];
    }
    float **flat[] = {&ts->gW, &ts->mW, &ts->vW, &ts->gB, &ts->mB, &ts->vB};
    for (int i = 0; i < 6; ++i) {
        const uint64_t cnt = i < 3 ? ts->total_w : ts->total_b;
        hipError_t e = hipMalloc((void **)flat[i], cnt * sizeof(float));
        if (e != hipSuccess) { train_free(net); return fail_hip("sphip_train_begin: device allocation", e); }
        sp_train_fill0<<<(uint32_t)((cnt + 255) / 256), 256, 0, g_stream>>>(*flat[i], cnt);
    }
    hipError_t e = hipMalloc((void **)&ts->sq_part, 2u * kSqBlocks * sizeof(double));
    if (e == hipSuccess) e = hipMalloc((void **)&ts->scal, 4 * sizeof(float));
    if (e == hipSuccess) e = hipGetLastError();
    if (e == hipSuccess) e = hipStreamSynchronize(g_stream);
    if (e != hipSuccess) { train_free(net); return fail_hip("sphip_train_begin", e); }
    return 0;
}

void sphip_train_end(sphip_net *net)
{
    if (!net || !net->train) return;
    if (g_stream) (void)hipStreamSynchronize(g_stream);
    train_free(net);
}

static float *train_array(sphip_net *net, int which, uint32_t l, uint64_t *cnt)
{
    sphip_train_state *ts = net->train;
    const uint64_t wc = (uint64_t)net->topo[l] * net->topo[l + 1], bc = net->topo[l + 1];
    switch (which) {
    case SPHIP_TRAIN_W:  *cnt = wc; return reinterpret_cast<float *>(net->W[l].base);
    case SPHIP_TRAIN_B:  *cnt = bc; return reinterpret_cast<float *>(net->B[l].base);
    case SPHIP_TRAIN_MW: *cnt = wc; return ts->mW + ts->woff[l];
    case SPHIP_TRAIN_VW: *cnt = wc; return ts->vW + ts->woff[l];
    case SPHIP_TRAIN_MB: *cnt = bc; return ts->mB + ts->boff[l];
    case SPHIP_TRAIN_VB: *cnt = bc; return ts->vB + ts->boff[l];
    case SPHIP_TRAIN_GW: *cnt = wc; return ts->gW + ts->woff[l];
    case SPHIP_TRAIN_GB: *cnt = bc; return ts->gB + ts->boff[l];
    default: *cnt = 0; return nullptr;
    }
}

int sphip_train_set(sphip_net *net, int which, uint32_t l, const float *host)
{
    if (!net || !net->train || l + 1 >= net->layers || !host) return fail_msg("sphip_train_set: invalid argument");
    uint64_t cnt = 0;
    float *dst = train_array(net, which, l, &cnt);
    if (!dst) return fail_msg("sphip_train_set: unknown array");
    HCHECK(hipMemcpyAsync(dst, host, cnt * sizeof(float), hipMemcpyHostToDevice, g_stream));
    HCHECK(hipStreamSynchronize(g_stream));
    if (which == SPHIP_TRAIN_W) net->W[l].cat3_valid = false;      // the FP16 parts describe the old weights
    return 0;
}

int sphip_train_get(sphip_net *net, int which, uint32_t l, float *host)
{
    if (!net || !net->train || l + 1 >= net->layers || !host) return fail_msg("sphip_train_get: invalid argument");
    uint64_t cnt = 0;
    const float *src = train_array(net, which, l, &cnt);
    if (!src) return fail_msg("sphip_train_get: unknown array");
    HCHECK(hipMemcpyAsync(host, src, cnt * sizeof(float), hipMemcpyDeviceToHost, g_stream));
    HCHECK(hipStreamSynchronize(g_stream));
    return 0;
}

int sphip_train_step(sphip_net *net, const float *x, const float *targets, uint32_t n, const sphip_train_args *args,
                     uint32_t flags, float *total_loss)
{
    const bool restage = (flags & SPHIP_TRAIN_SAME_BATCH) != 0;
    if (!net || ((!x || !targets) && !restage) || n == 0 || !args) return fail_msg("sphip_train_step: invalid argument");
    if (!net->train) return fail_msg("sphip_train_step: sphip_train_begin was not called for this net");
    if (args->optimizer > 4 || (args->loss_func != 0 && args->loss_func != 1)) return fail_msg("sphip_train_step: invalid optimizer or loss");
    sphip_train_state *ts = net->train;
    if (reserve(net, n, false) || train_reserve(net, n)) return 1;
    const uint32_t last = net->layers - 1, width = net->topo[last];
    const bool on_dev = (flags & SPHIP_X_ON_DEVICE) != 0;
    const float *d_x = x, *d_t = targets;
    if (restage) {
        if (ts->staged_n != n) return fail_msg("sphip_train_step: SPHIP_TRAIN_SAME_BATCH without a staged batch of this size");
        d_x = ts->act[0];
        d_t = ts->targets;
    } else if (!on_dev) {
        if (upload_from_host(ts->act[0], x, (size_t)n * net->topo[0] * sizeof(float))) return 1;
        HCHECK(hipMemcpyAsync(ts->targets, targets, (size_t)n * width * sizeof(float), hipMemcpyHostToDevice, g_stream));
        d_x = ts->act[0];
        d_t = ts->targets;
        ts->staged_n = n;
    }

    // forward, every layer kept (Training.c:313-345)
    const float *in = d_x;
    for (uint32_t l = 1; l <= last; ++l) {
        const LayerArgs L = make_layer_args(net, l);
        const bool softmax = net->act[l - 1] == A_SOFTMAX;
        float *main_out = softmax ? net->soft_tmp : ts->act[l];
        bool soft_done = false;
        if (n <= kF32VectorMax || f32_thin_vector(L, n)) launch_gemv(net->prec, net->workspace(), L, in, main_out, n, false);
        else soft_done = launch_gemm32(L, in, main_out, n, net->split_ws, net->split_cap, softmax ? ts->act[l] : nullptr);
        if (softmax && !soft_done) sp_softmax_rows<<<(n + 3) / 4, 256, 0, g_stream>>>(net->soft_tmp, ts->act[l], 0, n, net->topo[l]);
        in = ts->act[l];
    }

    if (total_loss) {
        if (grow(&ts->loss_buf, &ts->loss_cap, 3ull * n + 8u)) return 1;
        float *d_loss = ts->loss_buf;
        uint32_t *d_pred = reinterpret_cast<uint32_t *>(d_loss + n), *d_hit = d_pred + n;
        double *d_tot = reinterpret_cast<double *>((reinterpret_cast<uintptr_t>(d_hit + n) + 7u) & ~(uintptr_t)7u);
        EvalArgs ea{ts->act[last], d_t, d_loss, d_pred, d_hit, n, width, args->loss_func, net->act[last - 1] == A_SIGMOID ? 1 : 0};
        sp_eval_rows<<<(n + 3) / 4, 256, 0, g_stream>>>(ea);
        sp_eval_total<<<1, 1024, 0, g_stream>>>(d_loss, d_hit, n, d_tot, reinterpret_cast<uint32_t *>(d_tot + 1));
        double tot = 0.0;
        HCHECK(hipMemcpyAsync(&tot, d_tot, sizeof(double), hipMemcpyDeviceToHost, g_stream));
        HCHECK(hipStreamSynchronize(g_stream));
        *total_loss = (float)tot;
    }

    // deltas (Training.c:347-394)
    const int last_act = net->act[last - 1];
    const int mode = (args->loss_func == 0 && last_act == A_SOFTMAX) ? 0
                   : (args->loss_func == 1 && (last_act == A_SOFTMAX || last_act == A_SIGMOID)) ? 1 : 2;
    sp_train_out_delta<<<(n + 3) / 4, 256, 0, g_stream>>>(ts->act[last], d_t, ts->delta[last], n, width, mode, last_act);
    for (uint32_t l = last - 1; l > 0; --l) {
        TrGemmArgs g{};
        g.A = ts->delta[l + 1]; g.lda = net->topo[l + 1];
        g.B = reinterpret_cast<const float *>(net->W[l].base); g.ldb = net->topo[l];
        g.C = ts->delta[l]; g.aux = ts->act[l]; g.act = net->act[l - 1];
        g.M = n; g.N = net->topo[l]; g.K = net->topo[l + 1];
        launch_train_gemm<false, true, TR_EPI_DELTA>(g, ts->ws, ts->ws_cap);
    }

    // gradients (Training.c:396-419)
    const float grad_scale = 1.0f / (float)n;
    for (uint32_t l = 0; l < last; ++l) {
        const uint32_t in_sz = net->topo[l], out_sz = net->topo[l + 1];
        TrGemmArgs g{};
        g.A = ts->delta[l + 1]; g.lda = out_sz;
        g.B = l == 0 ? d_x : ts->act[l]; g.ldb = in_sz;
        g.C = ts->gW + ts->woff[l];
        g.M = out_sz; g.N = in_sz; g.K = n; g.scale = grad_scale;
        launch_train_gemm<true, true, TR_EPI_SCALE>(g, ts->ws, ts->ws_cap);
        const uint32_t chunks = (n + kColsumRows - 1) / kColsumRows;
        sp_train_colsum_part<<<dim3((out_sz + 63) / 64, chunks), 256, 0, g_stream>>>(ts->delta[l + 1], ts->ws, n, out_sz);
        sp_train_colsum_fin<<<(out_sz + 255) / 256, 256, 0, g_stream>>>(ts->ws, ts->gB + ts->boff[l], chunks, out_sz, grad_scale);
    }
    HCHECK(hipGetLastError());
    if (args->optimizer < 0) return 0;          // gradients only

    // update (Training.c:439-507)
    const float *clip = nullptr;
    if (args->max_grad_norm > 0.0f) {
        uint32_t bw = (uint32_t)((ts->total_w + 255) / 256), bb = (uint32_t)((ts->total_b + 255) / 256);
        if (bw > kSqBlocks) bw = kSqBlocks;
        if (bb > kSqBlocks) bb = kSqBlocks;
        sp_train_sumsq_part<<<bw, 256, 0, g_stream>>>(ts->gW, ts->total_w, ts->sq_part);
        sp_train_sumsq_part<<<bb, 256, 0, g_stream>>>(ts->gB, ts->total_b, ts->sq_part + bw);
        sp_train_clip_fin<<<1, 64, 0, g_stream>>>(ts->sq_part, bw + bb, args->max_grad_norm, ts->scal);
        clip = ts->scal;
    }
    for (uint32_t l = 0; l < last; ++l) {
        const uint64_t wc = (uint64_t)net->topo[l] * net->topo[l + 1], bc = net->topo[l + 1];
        launch_opt(*args, reinterpret_cast<float *>(net->W[l].base), ts->gW + ts->woff[l], ts->mW + ts->woff[l], ts->vW + ts->woff[l],
                   wc, args->weight_decay, clip);
        net->W[l].cat3_valid = false;                               // the FP16 parts of a split-mode forward describe the old weights
        launch_opt(*args, reinterpret_cast<float *>(net->B[l].base), ts->gB + ts->boff[l], ts->mB + ts->boff[l], ts->vB + ts->boff[l],
                   bc, 0.0f, clip);
    }
    HCHECK(hipGetLastError());
    return 0;
}

// `iters` training steps on device-resident inputs between two HIP events on the library's stream; *ms = total elapsed.
// With args->beta*_pow_t fixed the moments keep their first-step correction; the arithmetic per step is the same.
int sphip_time_train_step(sphip_net *net, const float *d_x, const float *d_targets, uint32_t n, const sphip_train_args *args,
                          int iters, float *ms)
{
    if (!net || !d_x || !d_targets || n == 0 || !args || iters <= 0 || !ms) return fail_msg("sphip_time_train_step: invalid argument");
    if (sphip_train_step(net, d_x, d_targets, n, args, SPHIP_X_ON_DEVICE, nullptr)) return 1;      // sizes every buffer
    TimingEvents ev;
    if (ev.create()) return 1;
    hipEvent_t e0 = ev.e0, e1 = ev.e1;
    int rc = 0;
    HCHECK(hipEventRecord(e0, g_stream));
    for (int it = 0; it < iters && !rc; ++it) rc = sphip_train_step(net, d_x, d_targets, n, args, SPHIP_X_ON_DEVICE, nullptr);
    hipError_t e = hipEventRecord(e1, g_stream);
    if (e == hipSuccess) e = hipEventSynchronize(e1);
    if (e == hipSuccess) e = hipEventElapsedTime(ms, e0, e1);
    if (rc) return rc;
    if (e != hipSuccess) return fail_hip("sphip_time_train_step", e);
    return 0;
}

}  // extern "C"
