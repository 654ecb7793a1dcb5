// hip_gemm32.inl — the FP32 MFMA GEMM for FP32 weights beyond 64 samples (sp_gemm32_f32,
// sp_gemm32_reduce).  Part of hip_forward.hip's translation unit (included there, inside its unnamed
// namespace); not compiled on its own.

// ---------------------------------------------------------------------------
// FP32 MFMA GEMM for FP32 weights (n > 64): 64 x 64 x 16 tile, 4 waves
// ---------------------------------------------------------------------------
struct Gemm32Args {
    LayerArgs L;
    const float *A;
    float *C;
    float *ws;             // [splits][M][N] partial sums when the grid splits K, else nullptr
    uint32_t M;
    uint32_t kper;         // k range of one split (multiple of 32)
};

// 64 x 64 x 32 tile, one 32 x 32 MFMA accumulator per wave.  The next K tile is fetched into
// registers while the current one is multiplied from LDS; small problems split K over grid y
// (a layer of this path is often a few dozen tiles only) and a second launch adds the parts.
// VEC: rows are 16-byte aligned (K % 4 == 0) and are read as float4.
template <bool VEC>
__global__ __launch_bounds__(256) void sp_gemm32_f32(const Gemm32Args g)
{
    constexpr int BM = 64, BN = 64, BK = 32, LDK = BK + 1;
    __shared__ float As[BM * LDK];
    __shared__ float Ws[BN * LDK];
    const uint32_t M = g.M, N = g.L.N, K = g.L.K;
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
    const float *Wf = reinterpret_cast<const float *>(g.L.w);

    f32x16 acc;
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[r] = 0.0f;

    // each thread carries two 4-element pieces of A and of W per tile: piece p -> row p / 8, k (p % 8) * 4
    float4 ra[2], rw[2];
    auto fetch = [&](uint32_t k0) {
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            const int p = t + 256 * i, row = p >> 3;
            const uint32_t k = k0 + (uint32_t)(p & 7) * 4u;
            const uint32_t m = m0 + row, n = n0 + row;
            if constexpr (VEC) {
                const bool kin = k < kend;                       // whole pieces: K and the split are multiples of 4
                const float4 va = *reinterpret_cast<const float4 *>(g.A + (size_t)(m < M ? m : M - 1) * K + (kin ? k : 0u));
                const float4 vw = *reinterpret_cast<const float4 *>(Wf + (size_t)(n < N ? n : N - 1) * K + (kin ? k : 0u));
                ra[i] = (kin && m < M) ? va : make_float4(0.0f, 0.0f, 0.0f, 0.0f);
                rw[i] = (kin && n < N) ? vw : make_float4(0.0f, 0.0f, 0.0f, 0.0f);
            } else {
                float a4[4], w4[4];
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    const bool kin = k + e < kend;
                    a4[e] = (kin && m < M) ? g.A[(size_t)m * K + k + e] : 0.0f;
                    w4[e] = (kin && n < N) ? Wf[(size_t)n * K + k + e] : 0.0f;
                }
                ra[i] = make_float4(a4[0], a4[1], a4[2], a4[3]);
                rw[i] = make_float4(w4[0], w4[1], w4[2], w4[3]);
            }
        }
    };
    auto stash = [&]() {
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            const int p = t + 256 * i, row = p >> 3, kk = (p & 7) * 4;
            float *da = As + row * LDK + kk, *dw = Ws + row * LDK + kk;
            da[0] = ra[i].x; da[1] = ra[i].y; da[2] = ra[i].z; da[3] = ra[i].w;
            dw[0] = rw[i].x; dw[1] = rw[i].y; dw[2] = rw[i].z; dw[3] = rw[i].w;
        }
    };

    fetch(kbeg);
    for (uint32_t k0 = kbeg; k0 < kend; k0 += BK) {
        stash();
        __syncthreads();
        if (k0 + BK < kend) fetch(k0 + BK);
#pragma unroll
        for (int ks = 0; ks < BK; ks += 2) {
            const float a = As[(wm * 32 + (lane & 31)) * LDK + ks + (lane >> 5)];
            const float b = Ws[(wn * 32 + (lane & 31)) * LDK + ks + (lane >> 5)];
            acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a, b, acc, 0, 0, 0);
        }
        __syncthreads();
    }

    const uint32_t col = n0 + wn * 32 + (lane & 31);
    if (col >= N) return;
    const float bias = elem_value_rt(g.L.bias_fmt, g.L.bias, col) * g.L.bscale;
#pragma unroll
    for (int r = 0; r < 16; ++r) {
        const uint32_t row = m0 + wm * 32 + 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3);
        if (row >= M) continue;
        if (g.ws) g.ws[((size_t)blockIdx.y * M + row) * N + col] = acc[r];
        else g.C[(size_t)row * N + col] = apply_act(acc[r] + bias, g.L.act);
    }
}

// The same product for layers whose weights exceed the L2s, at 512 samples and more: 128 x 128 x 32 tile (each wave
// 64 x 64 = 2 x 2 accumulators), two LDS stages and one barrier per K tile, rows of 36 floats in LDS.  MFMA step
// (j, t), t = 0 .. 3, of a K tile multiplies k = 8 j + 4 h + t on the lanes of half h for both operands alike (a sum
// over k in any order), so that a lane reads the four k of four steps with one 16-byte LDS load.  Half the bytes per
// flop of the 64 x 64 tile, through LDS and through the fabric (8192 x 4096 x 4096: 9.2 GB fetched per launch with
// 64 x 64 tiles).  Rows are 16-byte aligned (K % 4 == 0); no K split.
__global__ __launch_bounds__(256) void sp_gemm32_f32_big(const Gemm32Args g)
{
    constexpr int BM = 128, BN = 128, BK = 32, LD = 36, SIZE = BM * LD;
    extern __shared__ __attribute__((aligned(16))) float smem32[];
    float *As = smem32, *Ws = smem32 + 2 * SIZE;
    const uint32_t M = g.M, N = g.L.N, K = g.L.K;
    const int t = threadIdx.x, lane = t & 63, wave = t >> 6;
    const int wm = wave >> 1, wn = wave & 1, q = lane & 31, h = lane >> 5;
    const uint32_t tiles_n = (N + BN - 1) / BN;
    uint32_t bid = blockIdx.x;
    {
        const uint32_t per = gridDim.x / 8u;          // each XCD a contiguous run of tiles
        if (bid < per * 8u) bid = (bid & 7u) * per + (bid >> 3);
    }
    // ... walked in groups of 8 row tiles x all column tiles, the 8 row tiles of a column tile one after the other:
    // the 64 workgroups an XCD holds share 8 + 8 panels (1.76 GB fetched per 8192 x 4096 x 4096 launch instead of 4.45)
    uint32_t m0, n0;
    {
        constexpr uint32_t GM = 8;
        const uint32_t tiles_m = (M + BM - 1) / BM;
        const uint32_t group = bid / (GM * tiles_n), first = group * GM;
        const uint32_t rows = tiles_m - first < GM ? tiles_m - first : GM;
        const uint32_t in = bid - group * GM * tiles_n;
        m0 = (first + in % rows) * BM;
        n0 = (in / rows) * BN;
    }
    const float *Wf = reinterpret_cast<const float *>(g.L.w);

    f32x16 acc[2][2];
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.0f;

    // piece p of a tile: row p / 8, k (p % 8) * 4; four pieces of A and of W per thread
    float4 ra[4], rw[4];
    auto fetch = [&](uint32_t k0) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int p = t + 256 * i;
            const uint32_t row = (uint32_t)(p >> 3), k = k0 + (uint32_t)(p & 7) * 4u;
            const uint32_t m = m0 + row, n = n0 + row;
            const bool kin = k < K;
            const float4 va = *reinterpret_cast<const float4 *>(g.A + (size_t)(m < M ? m : M - 1) * K + (kin ? k : 0u));
            const float4 vw = *reinterpret_cast<const float4 *>(Wf + (size_t)(n < N ? n : N - 1) * K + (kin ? k : 0u));
            ra[i] = (kin && m < M) ? va : make_float4(0.0f, 0.0f, 0.0f, 0.0f);
            rw[i] = (kin && n < N) ? vw : make_float4(0.0f, 0.0f, 0.0f, 0.0f);
        }
    };
    auto stash = [&](int stage) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int p = t + 256 * i, o = (p >> 3) * LD + (p & 7) * 4;
            *reinterpret_cast<float4 *>(As + stage * SIZE + o) = ra[i];
            *reinterpret_cast<float4 *>(Ws + stage * SIZE + o) = rw[i];
        }
    };
    auto compute = [&](int stage) {
        const float *as = As + stage * SIZE + (wm * 64 + q) * LD + 4 * h, *ws = Ws + stage * SIZE + (wn * 64 + q) * LD + 4 * h;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            float a[2][4], b[2][4];
#pragma unroll
            for (int i = 0; i < 2; ++i) {
                const float4 va = *reinterpret_cast<const float4 *>(as + i * 32 * LD + 8 * j);
                const float4 vb = *reinterpret_cast<const float4 *>(ws + i * 32 * LD + 8 * j);
                a[i][0] = va.x; a[i][1] = va.y; a[i][2] = va.z; a[i][3] = va.w;
                b[i][0] = vb.x; b[i][1] = vb.y; b[i][2] = vb.z; b[i][3] = vb.w;
            }
#pragma unroll
            for (int tt = 0; tt < 4; ++tt)
#pragma unroll
                for (int i = 0; i < 2; ++i)
#pragma unroll
                    for (int jn = 0; jn < 2; ++jn) acc[i][jn] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[i][tt], b[jn][tt], acc[i][jn], 0, 0, 0);
        }
    };

    const uint32_t nk = (K + BK - 1) / BK;
    fetch(0);
    stash(0);
    __syncthreads();
    for (uint32_t kt = 0; kt < nk; ++kt) {
        const bool more = kt + 1 < nk;
        if (more) fetch((kt + 1) * BK);
        compute((int)(kt & 1u));
        if (more) stash((int)((kt + 1) & 1u));     // the other stage: every wave left it before the last barrier
        __syncthreads();
    }

#pragma unroll
    for (int jn = 0; jn < 2; ++jn) {
        const uint32_t col = n0 + wn * 64 + jn * 32 + q;
        if (col >= N) continue;
        const float bias = elem_value_rt(g.L.bias_fmt, g.L.bias, col) * g.L.bscale;
#pragma unroll
        for (int i = 0; i < 2; ++i)
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const uint32_t row = m0 + wm * 64 + i * 32 + 8 * (r >> 2) + 4 * h + (r & 3);
                if (row < M) g.C[(size_t)row * N + col] = apply_act(acc[i][jn][r] + bias, g.L.act);
            }
    }
}

// Small FP32 layers in one launch: a workgroup owns a 32 x 32 tile of the output, its eight waves split K in whole
// steps of eight, and their sums meet in LDS.  No operand staging: lane (r, h) loads four consecutive k of row r of both
// operands (k = 8 s + 4 h .. + 3 of step s) straight into registers and feeds them to four MFMA steps (a sum over k in
// any order).  For outputs of up to 512 tiles and K up to 1024, where sp_gemm32_f32 needs a K split over the grid and a
// second launch to fill the chip (256 x 512 x 784: 8 us against 12 us for the two).  A softmax layer of at most 32
// outputs is normalised here (Activation.c:5-21), soft_out != nullptr.  Rows are 16-byte aligned (K % 4 == 0).
__global__ __launch_bounds__(512) void sp_gemm32_small(const Gemm32Args g, float *__restrict__ soft_out)
{
    constexpr int NW = 8, U = 4;
    __shared__ float part[NW][32 * 33];
    const uint32_t M = g.M, N = g.L.N, K = g.L.K;
    const int t = threadIdx.x, lane = t & 63, wave = t >> 6, q = lane & 31, h = lane >> 5;
    const uint32_t tiles_n = (N + 31u) / 32u;
    const uint32_t m0 = (blockIdx.x / tiles_n) * 32u, n0 = (blockIdx.x % tiles_n) * 32u;
    const uint32_t steps = (K + 7u) / 8u, per = (steps + NW - 1) / NW;
    const uint32_t s0 = wave * per, s1 = s0 + per < steps ? s0 + per : steps;
    const uint32_t am = m0 + q < M ? m0 + q : M - 1, wn = n0 + q < N ? n0 + q : N - 1;
    const float *ap = g.A + (size_t)am * K + 4 * h;
    const float *wp = reinterpret_cast<const float *>(g.L.w) + (size_t)wn * K + 4 * h;
    f32x16 acc;
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[r] = 0.0f;
    auto ld = [&](const float *p, uint32_t s) -> float4 {       // K % 4 == 0: a piece is inside the row or beyond it
        return 8u * s + 4u * h < K ? *reinterpret_cast<const float4 *>(p + 8u * s) : make_float4(0.0f, 0.0f, 0.0f, 0.0f);
    };
    auto fma4 = [&](const float4 &a, const float4 &b) {
        acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a.x, b.x, acc, 0, 0, 0);
        acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a.y, b.y, acc, 0, 0, 0);
        acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a.z, b.z, acc, 0, 0, 0);
        acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a.w, b.w, acc, 0, 0, 0);
    };
    uint32_t s = s0;
    for (; s + U <= s1; s += U) {
        float4 a[U], b[U];
#pragma unroll
        for (int u = 0; u < U; ++u) { a[u] = ld(ap, s + u); b[u] = ld(wp, s + u); }
#pragma unroll
        for (int u = 0; u < U; ++u) fma4(a[u], b[u]);
    }
    for (; s < s1; ++s) fma4(ld(ap, s), ld(wp, s));
#pragma unroll
    for (int r = 0; r < 16; ++r) part[wave][(8 * (r >> 2) + 4 * h + (r & 3)) * 33 + q] = acc[r];
    __syncthreads();
    // the waves' sums in wave order, bias, activation; 512 threads, two outputs each
#pragma unroll
    for (int i = 0; i < 2; ++i) {
        const int e = t + 512 * i, row = e >> 5, col = e & 31;
        float v = 0.0f;
#pragma unroll
        for (int w = 0; w < NW; ++w) v += part[w][row * 33 + col];
        const uint32_t n = n0 + col < N ? n0 + col : N - 1;
        v = apply_act(v + elem_value_rt(g.L.bias_fmt, g.L.bias, n) * g.L.bscale, g.L.act);
        if (soft_out) part[0][row * 33 + col] = v;               // (every thread has read part[0][its own two slots] only)
        else if (m0 + row < M && n0 + col < N) g.C[(size_t)(m0 + row) * N + n0 + col] = v;
    }
    if (!soft_out) return;                                        // (uniform)
    __syncthreads();
    if (t < 32 && m0 + t < M) {                                   // N <= 32: the tile holds whole rows of logits
        const float *lr = &part[0][t * 33];
        float mx = lr[0];
        for (uint32_t c = 1; c < N; ++c) mx = fmaxf(mx, lr[c]);
        float sum = 0.0f;
        for (uint32_t c = 0; c < N; ++c) sum += expf(lr[c] - mx);
        const float inv = sum > 0.0f ? 1.0f / sum : 1.0f;
        for (uint32_t c = 0; c < N; ++c) soft_out[(size_t)(m0 + t) * N + c] = expf(lr[c] - mx) * inv;
    }
}

// adds the K splits of sp_gemm32_f32 (in split order) and applies bias and activation
__global__ __launch_bounds__(256) void sp_gemm32_reduce(const Gemm32Args g, uint32_t splits)
{
    const uint64_t idx = (uint64_t)blockIdx.x * 256u + threadIdx.x;
    const uint64_t total = (uint64_t)g.M * g.L.N;
    if (idx >= total) return;
    float sum = 0.0f;
    for (uint32_t sp = 0; sp < splits; ++sp) sum += g.ws[(uint64_t)sp * total + idx];
    const uint32_t col = (uint32_t)(idx % g.L.N);
    const float bias = elem_value_rt(g.L.bias_fmt, g.L.bias, col) * g.L.bscale;
    g.C[idx] = apply_act(sum + bias, g.L.act);
}

// The same for a softmax layer of at most 64 outputs: 16 lanes per sample (lane i takes outputs i, i + 16, ...)
// add the splits of their logits and normalise them together (Activation.c:5-21: largest logit subtracted,
// exponentials, one division by their sum), so that the layer needs no separate softmax pass.
__global__ __launch_bounds__(256) void sp_gemm32_reduce_softmax(const Gemm32Args g, uint32_t splits, float *__restrict__ out)
{
    const uint32_t row = blockIdx.x * 16u + (threadIdx.x >> 4), sub = threadIdx.x & 15u;
    const uint32_t N = g.L.N;
    const uint64_t total = (uint64_t)g.M * N;
    float v[4];
    float m = -3.402823466e+38f;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const uint32_t c = sub + 16u * j;
        const bool valid = row < g.M && c < N;
        float sum = 0.0f;
        if (valid) {
            for (uint32_t sp = 0; sp < splits; ++sp) sum += g.ws[(uint64_t)sp * total + (uint64_t)row * N + c];
            sum += elem_value_rt(g.L.bias_fmt, g.L.bias, c) * g.L.bscale;
        }
        v[j] = valid ? sum : -3.402823466e+38f;
        m = fmaxf(m, v[j]);
    }
#pragma unroll
    for (int off = 8; off >= 1; off >>= 1) m = fmaxf(m, __shfl_xor(m, off));
    float s = 0.0f;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const uint32_t c = sub + 16u * j;
        v[j] = (row < g.M && c < N) ? expf(v[j] - m) : 0.0f;
        s += v[j];
    }
#pragma unroll
    for (int off = 8; off >= 1; off >>= 1) s += __shfl_xor(s, off);
    const float inv = s > 0.0f ? 1.0f / s : 1.0f;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const uint32_t c = sub + 16u * j;
        if (row < g.M && c < N) out[(uint64_t)row * N + c] = v[j] * inv;
    }
}
