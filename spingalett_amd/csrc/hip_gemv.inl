// hip_gemv.inl — the kernels for 1..4 samples (FP32 weights: up to 64): vector GEMV and the
// integer GEMV on the INT8 matrix cores.  Part of hip_forward.hip's translation unit (included there,
// inside its unnamed namespace); not compiled on its own.

// ---------------------------------------------------------------------------
// GEMV family (n <= 64): y[b][j] = act(bias[j] + scale * sum_k q[j][k] x[b][k])
// ---------------------------------------------------------------------------
struct LayerArgs {
    const uint8_t *w;      // serialized weight codes, row-major [N][K]
    const uint8_t *bias;   // serialized bias codes [N]
    float wscale;          // folded weight scale
    float bscale;          // folded bias scale
    int bias_fmt;
    int act;               // activation applied in the epilogue (A_NONE for softmax layers)
    uint32_t N, K;         // out, in
};

// unpack one 16-byte chunk into its 128/bits unscaled float values
template <int FMT>
__device__ __forceinline__ void unpack16(const uint4 v, float *o)
{
    const uint32_t w[4] = {v.x, v.y, v.z, v.w};
    if constexpr (FMT == F32) {
#pragma unroll
        for (int i = 0; i < 4; ++i) o[i] = bits_to_float(w[i]);
    } else if constexpr (FMT == BF16) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            o[2 * i]     = bits_to_float(w[i] << 16);
            o[2 * i + 1] = bits_to_float(w[i] & 0xFFFF0000u);
        }
    } else if constexpr (FMT == F16) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            _Float16 lo, hi;
            uint16_t a = (uint16_t)(w[i] & 0xFFFFu), b = (uint16_t)(w[i] >> 16);
            __builtin_memcpy(&lo, &a, 2);
            __builtin_memcpy(&hi, &b, 2);
            o[2 * i] = (float)lo;
            o[2 * i + 1] = (float)hi;
        }
    } else if constexpr (FMT == I8) {
#pragma unroll
        for (int i = 0; i < 4; ++i)
#pragma unroll
            for (int j = 0; j < 4; ++j) o[4 * i + j] = (float)((int)(w[i] << (24 - 8 * j)) >> 24);
    } else if constexpr (FMT == I4) {
#pragma unroll
        for (int i = 0; i < 4; ++i)
#pragma unroll
            for (int j = 0; j < 8; ++j) o[8 * i + j] = (float)((int)(w[i] << (28 - 4 * j)) >> 28);
    } else {
#pragma unroll
        for (int i = 0; i < 4; ++i)
#pragma unroll
            for (int j = 0; j < 16; ++j) o[16 * i + j] = (float)((int)(w[i] << (30 - 2 * j)) >> 30);
    }
}

// Aligned path: every row is a whole number of 16-byte chunks.  One wave owns
// R rows at a time; lane c takes chunks c, c+64, ... of each row, so a wave reads
// 1 KiB contiguous per row and instruction.  Partial sums meet in a
// wavefront-shuffle reduction; lane 0 applies scale, bias and activation.
template <int FMT, int BT, int R>
__global__ __launch_bounds__(256) void sp_gemv(const LayerArgs L, const float *__restrict__ x,
                                               float *__restrict__ y, int nb)
{
    constexpr int EPC = 128 / fmt_bits(FMT);
    const int lane = threadIdx.x & 63;
    const uint32_t wave = blockIdx.x * 4u + (threadIdx.x >> 6);
    const uint32_t row0 = wave * R;
    if (row0 >= L.N) return;
    const uint32_t nchunks = L.K / EPC;
    const size_t row_bytes = (size_t)nchunks * 16u;

    const uint8_t *rp[R];
#pragma unroll
    for (int r = 0; r < R; ++r) {
        uint32_t row = row0 + r < L.N ? row0 + r : L.N - 1;
        rp[r] = L.w + (size_t)row * row_bytes;
    }

    float acc[R][BT];
#pragma unroll
    for (int r = 0; r < R; ++r)
#pragma unroll
        for (int b = 0; b < BT; ++b) acc[r][b] = 0.0f;

    for (uint32_t c = lane; c < nchunks; c += kWave) {
        uint4 wv[R];
#pragma unroll
        for (int r = 0; r < R; ++r) wv[r] = *reinterpret_cast<const uint4 *>(rp[r] + (size_t)c * 16u);
        float wf[R][EPC];
#pragma unroll
        for (int r = 0; r < R; ++r) unpack16<FMT>(wv[r], wf[r]);
        // BF16 weights, three or four samples: left to itself the compiler waits for each sample's activations
        // before it asks for the next one's (8192 x 8192: 65 us against 45 us for FP16 weights); all of a chunk's
        // activation loads first, then the arithmetic
        constexpr bool HOIST = FMT == BF16 && BT == 4;
        float4 xs[HOIST ? BT : 1][HOIST ? EPC / 4 : 1];
        if constexpr (HOIST) {
#pragma unroll
            for (int b = 0; b < BT; ++b) {
                const int bb = b < nb ? b : nb - 1;
                const float4 *xp = reinterpret_cast<const float4 *>(x + (size_t)bb * L.K + (size_t)c * EPC);
#pragma unroll
                for (int e = 0; e < EPC / 4; ++e) xs[b][e] = xp[e];
            }
            __builtin_amdgcn_sched_barrier(0);
        }
#pragma unroll
        for (int b = 0; b < BT; ++b) {
            const int bb = b < nb ? b : nb - 1;
            const float4 *xp = reinterpret_cast<const float4 *>(x + (size_t)bb * L.K + (size_t)c * EPC);
#pragma unroll
            for (int e = 0; e < EPC / 4; ++e) {
                float4 xv;
                if constexpr (HOIST) xv = xs[b][e];
                else xv = xp[e];
#pragma unroll
                for (int r = 0; r < R; ++r) {
                    acc[r][b] = fmaf(wf[r][4 * e + 0], xv.x, acc[r][b]);
                    acc[r][b] = fmaf(wf[r][4 * e + 1], xv.y, acc[r][b]);
                    acc[r][b] = fmaf(wf[r][4 * e + 2], xv.z, acc[r][b]);
                    acc[r][b] = fmaf(wf[r][4 * e + 3], xv.w, acc[r][b]);
                }
            }
        }
    }

#pragma unroll
    for (int r = 0; r < R; ++r)
#pragma unroll
        for (int b = 0; b < BT; ++b) acc[r][b] = wave_sum(acc[r][b]);

    if (lane == 0) {
#pragma unroll
        for (int r = 0; r < R; ++r) {
            const uint32_t row = row0 + r;
            if (row >= L.N) break;
            const float bias = elem_value_rt(L.bias_fmt, L.bias, row) * L.bscale;
#pragma unroll
            for (int b = 0; b < BT; ++b)
                if (b < nb) y[(size_t)b * L.N + row] = apply_act(fmaf(acc[r][b], L.wscale, bias), L.act);
        }
    }
}

// Rows of whole 32-bit words, a word per lane: `lpr` lanes (a power of two) share a row, 64 / lpr rows per wave.  For rows of a few hundred bytes, of which sp_gemv's 16-byte chunks occupy a handful of lanes (a 256-code INT2
// row is four chunks), and for rows that are whole words but not whole 16-byte units (784 INT4 codes), which would
// otherwise be fetched an element per lane.  K codes = K bits / 32 words; the activations of an integer word's codes
// are 16-byte aligned (4, 8 or 16 floats).  FP32 and 16-bit rows (one or two values per word) come here for thin
// layers only, a workgroup per row.
template <int FMT, int BT>
__global__ __launch_bounds__(256) void sp_gemv_words(const LayerArgs L, const float *__restrict__ x, float *__restrict__ y, int nb,
                                                     uint32_t lpr)
{
    constexpr int bits = fmt_bits(FMT), CW = 32 / bits;      // codes per word
    const int lane = threadIdx.x & 63;
    // lpr <= 64: 64 / lpr rows per wave; lpr = 128 or 256: a row spans two or four waves, whose sums meet in LDS
    const uint32_t sub = threadIdx.x & (lpr - 1u);
    const uint32_t row = lpr <= 64u ? (blockIdx.x * 4u + (threadIdx.x >> 6)) * (64u / lpr) + (uint32_t)lane / lpr
                                    : blockIdx.x * (256u / lpr) + threadIdx.x / lpr;
    const uint32_t wpr = L.K / CW;                            // words per row
    const uint32_t rowc = row < L.N ? row : L.N - 1;
    const uint32_t *wp = reinterpret_cast<const uint32_t *>(L.w) + (size_t)rowc * wpr;
    float acc[BT];
#pragma unroll
    for (int b = 0; b < BT; ++b) acc[b] = 0.0f;
    for (uint32_t w = sub; w < wpr; w += lpr) {
        const uint32_t word = wp[w];
        float q[CW];
        if constexpr (FMT == F32) {
            q[0] = __uint_as_float(word);
        } else if constexpr (FMT == F16) {
            _Float16 lo, hi;
            const uint16_t a = (uint16_t)(word & 0xFFFFu), b = (uint16_t)(word >> 16);
            __builtin_memcpy(&lo, &a, 2);
            __builtin_memcpy(&hi, &b, 2);
            q[0] = (float)lo;
            q[1] = (float)hi;
        } else if constexpr (FMT == BF16) {
            q[0] = __uint_as_float(word << 16);
            q[1] = __uint_as_float(word & 0xFFFF0000u);
        } else {
#pragma unroll
            for (int j = 0; j < CW; ++j) q[j] = (float)((int)(word << (32 - bits - bits * j)) >> (32 - bits));
        }
#pragma unroll
        for (int b = 0; b < BT; ++b) {
            const int bb = b < nb ? b : nb - 1;
            const float *xw = x + (size_t)bb * L.K + (size_t)w * CW;
            if constexpr (CW >= 4) {
                const float4 *xp = reinterpret_cast<const float4 *>(xw);
#pragma unroll
                for (int e = 0; e < CW / 4; ++e) {
                    const float4 xv = xp[e];
                    acc[b] = fmaf(q[4 * e + 0], xv.x, acc[b]);
                    acc[b] = fmaf(q[4 * e + 1], xv.y, acc[b]);
                    acc[b] = fmaf(q[4 * e + 2], xv.z, acc[b]);
                    acc[b] = fmaf(q[4 * e + 3], xv.w, acc[b]);
                }
            } else {
#pragma unroll
                for (int e = 0; e < CW; ++e) acc[b] = fmaf(q[e], xw[e], acc[b]);
            }
        }
    }
    for (uint32_t off = (lpr < 64u ? lpr : 64u) >> 1; off; off >>= 1) {
#pragma unroll
        for (int b = 0; b < BT; ++b) acc[b] += __shfl_xor(acc[b], (int)off, kWave);
    }
    if (lpr > 64u) {                                          // (uniform over the workgroup)
        __shared__ float part[4][BT];
        const uint32_t wave = threadIdx.x >> 6, wpr_waves = lpr / 64u;
        if (lane == 0) {
#pragma unroll
            for (int b = 0; b < BT; ++b) part[wave][b] = acc[b];
        }
        __syncthreads();
        if (sub == 0) {
#pragma unroll
            for (int b = 0; b < BT; ++b) {
                float sum = part[wave][b];
                for (uint32_t v = 1; v < wpr_waves; ++v) sum += part[wave + v][b];
                acc[b] = sum;
            }
        }
    }
    if (sub == 0 && row < L.N) {
        const float bias = elem_value_rt(L.bias_fmt, L.bias, row) * L.bscale;
#pragma unroll
        for (int b = 0; b < BT; ++b)
            if (b < nb) y[(size_t)b * L.N + row] = apply_act(fmaf(acc[b], L.wscale, bias), L.act);
    }
}

// Generic path: any K, rows may start inside a byte.  One wave per row, one
// element per lane and step.
template <int FMT, int BT>
__global__ __launch_bounds__(256) void sp_gemv_generic(const LayerArgs L, const float *__restrict__ x,
                                                       float *__restrict__ y, int nb)
{
    const int lane = threadIdx.x & 63;
    const uint32_t row = blockIdx.x * 4u + (threadIdx.x >> 6);
    if (row >= L.N) return;
    float acc[BT];
#pragma unroll
    for (int b = 0; b < BT; ++b) acc[b] = 0.0f;
    const uint64_t base = (uint64_t)row * L.K;
    for (uint32_t k = lane; k < L.K; k += kWave) {
        const float w = elem_value<FMT>(L.w, base + k);
#pragma unroll
        for (int b = 0; b < BT; ++b) {
            const int bb = b < nb ? b : nb - 1;
            acc[b] = fmaf(w, x[(size_t)bb * L.K + k], acc[b]);
        }
    }
#pragma unroll
    for (int b = 0; b < BT; ++b) acc[b] = wave_sum(acc[b]);
    if (lane == 0) {
        const float bias = elem_value_rt(L.bias_fmt, L.bias, row) * L.bscale;
#pragma unroll
        for (int b = 0; b < BT; ++b)
            if (b < nb) y[(size_t)b * L.N + row] = apply_act(fmaf(acc[b], L.wscale, bias), L.act);
    }
}

// ---------------------------------------------------------------------------
// Integer-weight GEMV on the INT8 matrix cores (n <= 64, INT8 / INT4 / INT2)
// ---------------------------------------------------------------------------
// The packed codes are (nearly) MFMA operands already: INT8 bytes as they are,
// INT4 / INT2 after a mask-and-shift that leaves one code per byte.  The FP32
// activations are turned into exact integers instead of the weights into floats:
// per sample and K chunk, X = rint(x * 2^p) with |X| < 2^22, written as three
// balanced base-256 digits d0 + 256 d1 + 65536 d2, each an INT8.  Then
//     sum_k q_k x_k = 2^-p * (S0 + 256 S1 + 65536 S2),  S_i = sum_k q_k d_i,k
// and the S_i are exact INT32 dot products from v_mfma_i32_16x16x64_i8.  One
// 16-row A tile carries four samples (three digit rows + one zero row each), the
// B operand is 16 weight rows x 64 codes, so a wave needs no reduction across
// lanes: lane (n, s) ends up holding S0, S1, S2 of output row n and sample s.
// The unsigned fields of INT4 / INT2 are biased codes (q + 8, q + 2 after an XOR
// of the sign bits); the bias is removed exactly with sum_k d_i,k.
//
// Work split: a wave owns 16 output rows over the whole K; the waves of a
// workgroup (1, 2 or 4, chosen so that the grid fills the chip) share the digit
// planes of the current K chunk in LDS.  No workgroup ever waits for another:
// device-scope fences cost an L2 write-back on this multi-die part.
struct GemvI8Args {
    LayerArgs L;
    const float *x;        // [nb][K] activations (quantise kernel)
    uint8_t *aq;           // digit planes, see sp_quant_x
    float *inv;            // [chunks][nb] 2^-p
    int *dsum;             // [chunks][nb][4] digit sums (bias removal)
    float *y;              // [nb][N]
    int nb;
    uint32_t kc;           // K chunk = one scale block (multiple of the 64-byte block)
    uint32_t nchunks;      // ceil(K / kc)
    uint32_t stage_blocks; // 64-byte blocks whose digit planes are held in LDS at a time
    uint32_t rw, ks;       // waves of a workgroup that multiply: row groups x K shares
    uint32_t qw;           // self-quantising form: waves of a workgroup that quantise the activations (after the rw x ks others)
    uint32_t meta_bytes;   // LDS bytes of the per-chunk scale records (multiple of 16)
};

typedef int i32x4v __attribute__((ext_vector_type(4)));

template <int FMT>
struct I8Fmt {
    static constexpr int bits = fmt_bits(FMT);
    static constexpr int KL = 512 / bits;      // codes per 64-byte row segment (one wave load)
    static constexpr int NMF = KL / 64;        // MFMAs one lane-load feeds
    static constexpr int WK = 32 / bits;       // codes per 32-bit word
    static constexpr int BIAS = FMT == I8 ? 0 : FMT == I4 ? 8 : 2;
};

// Digits of the WK activations that meet one 32-bit weight word.  X = rint(x * scale);
// X + 0x808080 written in plain base 256 has the balanced digits of X, each offset by
// 128: gather the bytes per digit, then flip the top bits.  Byte i of the operand word
// of MFMA u comes from code i * NMF + u.
template <int FMT>
__device__ __forceinline__ void quant_word(const float4 (&v)[I8Fmt<FMT>::WK / 4], float scale,
                                           uint32_t (&d0)[I8Fmt<FMT>::NMF], uint32_t (&d1)[I8Fmt<FMT>::NMF],
                                           uint32_t (&d2)[I8Fmt<FMT>::NMF], int &ds0, int &ds1, int &ds2)
{
    constexpr int WK = I8Fmt<FMT>::WK, NMF = I8Fmt<FMT>::NMF;
    uint32_t Xo[WK];
#pragma unroll
    for (int c4 = 0; c4 < WK / 4; ++c4) {
        Xo[4 * c4 + 0] = (uint32_t)((int)rintf(v[c4].x * scale) + 0x808080);
        Xo[4 * c4 + 1] = (uint32_t)((int)rintf(v[c4].y * scale) + 0x808080);
        Xo[4 * c4 + 2] = (uint32_t)((int)rintf(v[c4].z * scale) + 0x808080);
        Xo[4 * c4 + 3] = (uint32_t)((int)rintf(v[c4].w * scale) + 0x808080);
    }
#pragma unroll
    for (int u = 0; u < NMF; ++u) {
        const uint32_t x0 = Xo[u], x1 = Xo[NMF + u], x2 = Xo[2 * NMF + u], x3 = Xo[3 * NMF + u];
        const uint32_t lo01 = __builtin_amdgcn_perm(x1, x0, 0x05040100u);   // x0.b0 x0.b1 x1.b0 x1.b1
        const uint32_t lo23 = __builtin_amdgcn_perm(x3, x2, 0x05040100u);
        const uint32_t hi01 = __builtin_amdgcn_perm(x1, x0, 0x0c060c02u);   // x0.b2 0 x1.b2 0
        const uint32_t hi23 = __builtin_amdgcn_perm(x3, x2, 0x0c060c02u);
        d0[u] = __builtin_amdgcn_perm(lo23, lo01, 0x06040200u) ^ 0x80808080u;
        d1[u] = __builtin_amdgcn_perm(lo23, lo01, 0x07050301u) ^ 0x80808080u;
        d2[u] = __builtin_amdgcn_perm(hi23, hi01, 0x06040200u) ^ 0x80808080u;
        ds0 = __builtin_amdgcn_sdot4((int)d0[u], 0x01010101, ds0, false);
        ds1 = __builtin_amdgcn_sdot4((int)d1[u], 0x01010101, ds1, false);
        ds2 = __builtin_amdgcn_sdot4((int)d2[u], 0x01010101, ds2, false);
    }
}

// One wave quantises up to 2048 consecutive activations of one sample (a scale chunk, or a slice of one: `len` codes
// starting at code kbase of row xr): every lane fetches its words' activations in one batch of loads (quant_load),
// the wave finds the largest magnitude (quant_amax), and each lane converts what it holds with the scale that the
// chunk's largest magnitude gives (quant_digits).
// A 64-byte weight segment (block) is spread over 4 lane groups g of 16 bytes = 4 words w;
// word w holds WK codes; after unpacking, MFMA u of that block takes byte i of word w from code
//   INT8: 4w+i (u = 0)      INT4: 8w + 2i + u      INT2: 16w + 4i + u
// of the lane group.  store(block, u, g, w, d0, d1, d2) receives the operand words (block counted from kbase);
// the result is the scale record {bits of 2^-p, sum d0, sum d1, sum d2} of what this wave converted (same in every lane).
template <int FMT>
struct QuantRegs {
    static constexpr int MAXIT = 2048 / (64 * I8Fmt<FMT>::WK);
    static constexpr int F4 = I8Fmt<FMT>::WK / 4;
    float4 v[MAXIT][F4];
};

template <int FMT>
__device__ __forceinline__ void quant_load(QuantRegs<FMT> &q, const float *xr, uint32_t K, uint32_t kbase, uint32_t len, int lane)
{
    using F = I8Fmt<FMT>;
    constexpr int KL = F::KL, WK = F::WK, F4 = WK / 4, MAXIT = QuantRegs<FMT>::MAXIT;
    constexpr uint32_t WPB = KL / WK;                            // words per block (16)
    const uint32_t iters = len / (64u * WK);
#pragma unroll
    for (int it = 0; it < MAXIT; ++it) {
        const uint32_t wl = (uint32_t)it * 64u + (uint32_t)lane;
        const uint32_t blk = wl / WPB, r = wl % WPB, gg = r >> 2, w = r & 3u;
        const uint32_t kw = kbase + blk * KL + gg * (KL / 4) + w * WK;     // first code of the word
        const bool valid = (uint32_t)it < iters && kw < K;                  // rows are whole numbers of words
        const float4 *src = reinterpret_cast<const float4 *>(xr + (valid ? kw : 0u));
#pragma unroll
        for (int c = 0; c < F4; ++c) {
            float4 t = src[c];
            if (!valid) t = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
            q.v[it][c] = t;
        }
    }
}

// largest |x| the wave holds, as its bit pattern: orders like the value, and infinities and NaNs sort last
template <int FMT>
__device__ __forceinline__ uint32_t quant_amax(const QuantRegs<FMT> &q)
{
    uint32_t lm = 0u;
#pragma unroll
    for (int it = 0; it < QuantRegs<FMT>::MAXIT; ++it)
#pragma unroll
        for (int c = 0; c < QuantRegs<FMT>::F4; ++c) {
            const float4 t = q.v[it][c];
            const uint32_t mx = max(__float_as_uint(t.x) & 0x7FFFFFFFu, __float_as_uint(t.y) & 0x7FFFFFFFu);
            const uint32_t mz = max(__float_as_uint(t.z) & 0x7FFFFFFFu, __float_as_uint(t.w) & 0x7FFFFFFFu);
            lm = max(lm, max(mx, mz));
        }
    return wave_max_u(lm);
}

template <int FMT, class Store>
__device__ __forceinline__ int4 quant_digits(const QuantRegs<FMT> &q, uint32_t amax, uint32_t len, int lane, Store store)
{
    using F = I8Fmt<FMT>;
    constexpr int KL = F::KL, NMF = F::NMF, WK = F::WK, MAXIT = QuantRegs<FMT>::MAXIT;
    constexpr uint32_t WPB = KL / WK;
    const uint32_t iters = len / (64u * WK);
    int e = (int)(amax >> 23) - 127;
    if (e < -126) e = -126;
    int p = 21 - e;                                              // |X| < 2^22: the top digit stays inside INT8
    p = p > 126 ? 126 : p;
    // A chunk that holds an infinity or a NaN cannot be written in digits: its record carries a NaN instead of
    // 2^-p, which turns the sample's sums into NaN, and the epilogue redoes those outputs in FP32 arithmetic so
    // that infinities and NaNs come out as cblas_sgemv / the FP32 dot product give them (Network.c:229-245).
    const bool finite = amax < 0x7F800000u;
    const bool live = amax != 0u && finite;                      // an all-zero chunk contributes nothing
    const float scale = live ? __uint_as_float((uint32_t)(p + 127) << 23) : 0.0f;
    int ds0 = 0, ds1 = 0, ds2 = 0;
#pragma unroll
    for (int it = 0; it < MAXIT; ++it) {
        if ((uint32_t)it < iters) {
            const uint32_t wl = (uint32_t)it * 64u + (uint32_t)lane;
            const uint32_t blk = wl / WPB, r = wl % WPB, gg = r >> 2, w = r & 3u;
            uint32_t d0[NMF], d1[NMF], d2[NMF];
            quant_word<FMT>(q.v[it], scale, d0, d1, d2, ds0, ds1, ds2);
#pragma unroll
            for (int u = 0; u < NMF; ++u) store(blk, (uint32_t)u, gg, w, d0[u], d1[u], d2[u]);
        }
    }
    ds0 = wave_sum_i(ds0);
    ds1 = wave_sum_i(ds1);
    ds2 = wave_sum_i(ds2);
    return make_int4(live ? (int)((uint32_t)(127 - p) << 23) : finite ? 0 : 0x7FC00000, ds0, ds1, ds2);
}

// Quantise kernel (n > 4): one wave per sample and scale chunk, four to a workgroup.
// Output order = the order the A operand is read: per (block, u, g) the planes are stored as
//   [sample][digit 0..2][16 bytes]
// i.e. 3 bytes per element and sample; the GEMV kernel copies them verbatim.
template <int FMT>
__global__ __launch_bounds__(256) void sp_quant_x(const GemvI8Args a)
{
    using F = I8Fmt<FMT>;
    constexpr int KL = F::KL, NMF = F::NMF;
    const int lane = threadIdx.x & 63;
    const uint32_t rec = blockIdx.x * 4u + (threadIdx.x >> 6);
    if (rec >= a.nchunks * (uint32_t)a.nb) return;
    const uint32_t ch = rec / (uint32_t)a.nb, s0 = rec % (uint32_t)a.nb;
    const uint32_t nblk = a.kc / KL;                         // blocks per chunk (last chunk zero-padded)
    QuantRegs<FMT> qr;
    quant_load<FMT>(qr, a.x + (size_t)s0 * a.L.K, a.L.K, ch * a.kc, a.kc, lane);
    const int4 md = quant_digits<FMT>(qr, quant_amax<FMT>(qr), a.kc, lane,
        [&](uint32_t blk, uint32_t u, uint32_t g, uint32_t w, uint32_t d0, uint32_t d1, uint32_t d2) {
            uint8_t *dst = a.aq + (((((size_t)ch * nblk + blk) * NMF + u) * 4 + g) * (size_t)a.nb + s0) * 48 + w * 4;
            *reinterpret_cast<uint32_t *>(dst) = d0;
            *reinterpret_cast<uint32_t *>(dst + 16) = d1;
            *reinterpret_cast<uint32_t *>(dst + 32) = d2;
        });
    if (lane == 0) {
        a.inv[rec] = __int_as_float(md.x);
        int *d = a.dsum + (size_t)rec * 4;
        d[0] = md.y; d[1] = md.z; d[2] = md.w; d[3] = 0;
    }
}

// Self-quantising form for up to four samples: one launch per layer, the waves of a workgroup specialised.
//   * Quant waves (the qw waves after the stream waves) request the activations of their first scale chunk before
//     anything else in the workgroup touches memory, and only when those have arrived are the stream waves let go
//     (barrier "go"): a compute unit's memory pipeline returns data in request order, and activations queued behind
//     megabytes of weight requests arrived 1.3 us later per fetch group in flight.  They then quantise into LDS, one
//     scale chunk of one sample at a time, and meet the stream waves at barrier 0.
//   * Stream waves (rw row groups x ks K shares; wave = ks_id * rw + rw_id) request D fetch groups of G 64-byte blocks
//     of their 16 rows, wait at barrier 0 for the digit planes, then multiply group by group; a group's registers are
//     reloaded with the group D further on as soon as it has been multiplied (D register sets, rotated by unrolling:
//     no copies, and the counted wait before a group leaves the younger requests in flight).  The weight stream so
//     runs while the activations are quantised (about 1.5 us during which memory used to sit idle).
//   * Which blocks a K share takes (PAIRS): pairs of blocks ks_id, ks_id + ks, ... (whole 128-byte lines per wave;
//     with three groups of one pair in flight the better choice up to 64 MiB of weights: 8192 x 8192 INT8 17.1
//     against 18.2 us, INT2 8.9 against 9.6 us, 4096 x 16384 INT4 11.5 against 13.3 us) or single blocks ks_id,
//     ks_id + ks, ... (two groups of four blocks; the halves of a line then come from two waves at about the same
//     time, which the memory system serves faster on large layers: 16384 x 16384 INT4 30.2 against 31.8 us, INT8 56
//     against 64 us).  Deeper prefetch than these was measured and is slower in either form.
// Digit planes of more than one LDS buffer (a.stage_blocks) take two buffers, stage s in buffer s & 1: the quant
// waves fill stage s + 1 while stage s is multiplied, and barrier s separates "stage s written" from "stage s read"
// for every wave (a buffer is refilled only after the barrier that ends its reading).
// 16 bytes per lane from a 64-bit lane address.  Inline assembly: the compiler's wait-count bookkeeping does not see
// the load (it would wait for every outstanding one where only the oldest set is needed); the caller waits with
// s_waitcnt vmcnt before it reads dst, and before the registers can be reused for anything else.
__device__ __forceinline__ void gload16_async(u32x4 &dst, const void *p)
{
    asm volatile("global_load_dwordx4 %0, %1, off" : "=v"(dst) : "v"(p) : "memory");
}

template <int FMT, int D, int G, bool PAIRS>
__device__ __forceinline__ void gemv_i8_specialised(const GemvI8Args &a)
{
    using F = I8Fmt<FMT>;
    constexpr int KL = F::KL, NMF = F::NMF;
    static_assert(G == 2 || G == 4, "fetch groups of two or four blocks");
    extern __shared__ __attribute__((aligned(16))) uint8_t lds_all[];
    int4 *meta = reinterpret_cast<int4 *>(lds_all);               // [nchunks][nb] {2^-p bits, d0 sum, d1 sum, d2 sum}
    uint8_t *A_lds = lds_all + a.meta_bytes;                      // [2][stage blocks][NMF][4 g][nb][3][16 bytes]

    const int t = threadIdx.x, lane = t & 63;
    const uint32_t wave = (uint32_t)__builtin_amdgcn_readfirstlane(t >> 6);
    const uint32_t N = a.L.N, K = a.L.K;
    const uint32_t nb = (uint32_t)a.nb;
    const uint32_t rw = a.rw, ks = a.ks, sw = rw * ks;
    const uint32_t kcb = a.kc / KL;                               // blocks per scale chunk
    const uint32_t blk_bytes = (uint32_t)NMF * 4u * nb * 48u;     // digit planes of one block
    const uint32_t u_bytes = 4u * nb * 48u;
    const uint32_t cps = a.stage_blocks / kcb;                    // chunks per stage
    const uint32_t nstages = (a.nchunks + cps - 1) / cps;
    const uint32_t buf_bytes = a.stage_blocks * blk_bytes;

    if (wave >= sw) {
        // ---- quant wave
        const uint32_t qid = wave - sw;
        QuantRegs<FMT> qr;
        auto store_to = [&](uint8_t *buf, uint32_t blk0, uint32_t smp) {
            return [=](uint32_t blk, uint32_t u, uint32_t gg, uint32_t w, uint32_t d0, uint32_t d1, uint32_t d2) {
                uint8_t *dst = buf + ((((size_t)(blk0 + blk) * NMF + u) * 4 + gg) * (size_t)nb + smp) * 48 + w * 4;
                *reinterpret_cast<uint32_t *>(dst) = d0;
                *reinterpret_cast<uint32_t *>(dst + 16) = d1;
                *reinterpret_cast<uint32_t *>(dst + 32) = d2;
            };
        };
        // The activations of a wave's first unit are requested before any weight: the stream waves are let go
        // (barrier "go") as soon as the requests are out, not when the data is in.  A compute unit's memory pipeline
        // returns data in request order, so the order of the requests is all that has to be right, and the weights
        // start 0.3-0.45 us earlier per launch (8192 x 8192 INT2 7.86 -> 7.46 us, 16384 x 16384 INT4 29.8 -> 29.4).
        const uint32_t nch0 = cps <= a.nchunks ? cps : a.nchunks;
        if (qid < nch0 * nb) {
            quant_load<FMT>(qr, a.x + (size_t)(qid % nb) * K, K, (qid / nb) * a.kc, a.kc, lane);
        }
        __syncthreads();                                      // barrier "go"
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        for (uint32_t s = 0; s < nstages; ++s) {
            const uint32_t ch0 = s * cps, nch = ch0 + cps <= a.nchunks ? cps : a.nchunks - ch0;
            uint8_t *buf = A_lds + (size_t)(s & 1u) * buf_bytes;
            for (uint32_t ui = qid; ui < nch * nb; ui += a.qw) {
                const uint32_t chl = ui / nb, smp = ui % nb;
                if (s != 0 || ui != qid)                      // the first unit is in the registers already
                    quant_load<FMT>(qr, a.x + (size_t)smp * K, K, (ch0 + chl) * a.kc, a.kc, lane);
                const int4 md = quant_digits<FMT>(qr, quant_amax<FMT>(qr), a.kc, lane, store_to(buf, chl * kcb, smp));
                if (lane == 0) meta[(size_t)(ch0 + chl) * nb + smp] = md;
            }
            __syncthreads();                                  // barrier s: stage s is written
        }
        if (ks > 1) {                                             // the two barriers of the K-share reduction
            __syncthreads();
            __syncthreads();
        }
        return;
    }

    // ---- stream wave
    const uint32_t ks_id = wave / rw, rw_id = wave % rw;
    const uint32_t nrow = (blockIdx.x * rw + rw_id) * 16u + (lane & 15);
    const uint32_t g = lane >> 4;
    const size_t row_bytes = (size_t)K * F::bits / 8u;
    const uint8_t *wrow = a.L.w + (size_t)(nrow < N ? nrow : N - 1) * row_bytes + g * 16u;
    // largest offset (from wrow) whose 16 bytes stay inside the row; reads past it are clamped there and meet zero digits
    const int64_t row_last = (int64_t)row_bytes - 16 - (int64_t)(g * 16u);
    const uint32_t groups_per_chunk = kcb / (ks * G);             // host guarantees divisibility
    const uint32_t ngroups = a.nchunks * groups_per_chunk;

    // Block u of this wave's fetch group j is block first + j * adv + du(u) of the row:
    //   PAIRS: block (u & 1) of pair ((G / 2) j + (u >> 1)) * ks + ks_id;  else block (G j + u) * ks + ks_id
    const uint32_t first = PAIRS ? 2u * ks_id : ks_id;
    const uint32_t adv = (uint32_t)G * ks;
    auto du = [&](int u) { return PAIRS ? (uint32_t)(u >> 1) * 2u * ks + (uint32_t)(u & 1) : (uint32_t)u * ks; };
    auto load_group = [&](u32x4 (&dst)[G], uint32_t j) {
#pragma unroll
        for (int u = 0; u < G; ++u) {
            int64_t off = (int64_t)((first + j * adv + du(u)) * 64u);
            off = off < row_last ? off : row_last;
            off = off > 0 ? off : 0;
            gload16_async(dst[u], wrow + off);
        }
    };
    __syncthreads();                                              // barrier "go": the quant waves have requested their activations
    u32x4 R[D][G];
#pragma unroll
    for (int d = 0; d < D; ++d)
        if ((uint32_t)d < ngroups) load_group(R[d], (uint32_t)d);

    // lane (m, g): row m of the A tile is digit m & 3 of sample m >> 2 (fourth rows and samples beyond nb are never
    // read from D: they point at the start of the block)
    uint32_t a_off;
    {
        const uint32_t m = lane & 15u, slot = m >> 2, d = m & 3u;
        a_off = (slot < nb && d < 3u) ? ((g * nb + slot) * 3u + d) * 16u : 0u;
    }
    float yacc = 0.0f;
    i32x4v acc[2] = {(i32x4v){0, 0, 0, 0}, (i32x4v){0, 0, 0, 0}};

    auto process = [&](const u32x4 wv, const uint8_t *rec) {
        const uint32_t w[4] = {wv.x, wv.y, wv.z, wv.w};
        i32x4v bop[NMF];
        if constexpr (FMT == I8) {
            bop[0] = (i32x4v){(int)w[0], (int)w[1], (int)w[2], (int)w[3]};
        } else if constexpr (FMT == I4) {
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                const uint32_t x8 = w[q] ^ 0x88888888u;          // nibble -> q + 8
                bop[0][q] = (int)(x8 & 0x0F0F0F0Fu);
                bop[1][q] = (int)((x8 >> 4) & 0x0F0F0F0Fu);
            }
        } else {
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                const uint32_t x2 = w[q] ^ 0xAAAAAAAAu;          // field -> q + 2
                bop[0][q] = (int)(x2 & 0x03030303u);
                bop[1][q] = (int)((x2 >> 2) & 0x03030303u);
                bop[2][q] = (int)((x2 >> 4) & 0x03030303u);
                bop[3][q] = (int)((x2 >> 6) & 0x03030303u);
            }
        }
#pragma unroll
        for (int f = 0; f < NMF; ++f) {
            const i32x4v aop = *reinterpret_cast<const i32x4v *>(rec + f * u_bytes + a_off);
            acc[f & 1] = __builtin_amdgcn_mfma_i32_16x16x64_i8(aop, bop[f], acc[f & 1], 0, 0, 0);
        }
    };
    auto fold = [&](uint32_t ch) {
        if (g < nb) {
            const int4 md = meta[(size_t)ch * nb + g];
            int S0 = acc[0][0] + acc[1][0], S1 = acc[0][1] + acc[1][1], S2 = acc[0][2] + acc[1][2];
            if (F::BIAS != 0 && ks_id == 0) {           // one K share removes the code bias of the whole chunk
                S0 -= F::BIAS * md.y;
                S1 -= F::BIAS * md.z;
                S2 -= F::BIAS * md.w;
            }
            const float tsum = fmaf((float)S2, 65536.0f, fmaf((float)S1, 256.0f, (float)S0));
            yacc = fmaf(tsum, __int_as_float(md.x), yacc);
        }
        acc[0] = acc[1] = (i32x4v){0, 0, 0, 0};
    };

    __syncthreads();                                              // barrier 0
    const uint8_t *rec = A_lds + (size_t)first * blk_bytes;       // digit planes of the first block of the current group
    uint32_t jnext = (uint32_t)D;                                 // next fetch group to request
    uint32_t gi = 0, ch = 0, cis = 0, stage = 0;
    // waits until at most `groups` fetch groups are outstanding (a uniform choice among the constants the
    // instruction can carry)
    auto wait_groups = [&](uint32_t groups) {
        static_for<D>([&](auto yc) {
            constexpr int y = decltype(yc)::value;
            if (groups == (uint32_t)y) asm volatile("s_waitcnt vmcnt(%0)" ::"n"(y * G) : "memory");
        });
    };
    uint32_t jcur = 0;                                            // fetch group about to be multiplied
    auto step = [&](auto dc) {
        constexpr int d = decltype(dc)::value;
        // this set's requests are the oldest outstanding; younger ones: the groups requested after it, at most D - 1
        // and fewer near the end of the row, where nothing is requested any more
        const uint32_t younger = ngroups - 1u - jcur;
        wait_groups(younger < (uint32_t)(D - 1) ? younger : (uint32_t)(D - 1));
#pragma unroll
        for (int u = 0; u < G; ++u) asm volatile("" : "+v"(R[d][u]));      // nothing that reads them moves above the wait
#pragma unroll
        for (int u = 0; u < G; ++u) process(R[d][u], rec + (size_t)du(u) * blk_bytes);
        if (jnext < ngroups) load_group(R[d], jnext);
        ++jnext;
        ++jcur;
        rec += (size_t)adv * blk_bytes;
        if (++gi == groups_per_chunk) {
            gi = 0;
            fold(ch);
            ++ch;
            if (++cis == cps && ch < a.nchunks) {                 // next stage: the other buffer, once it is written
                cis = 0;
                ++stage;
                __syncthreads();
                rec = A_lds + (size_t)(stage & 1u) * buf_bytes + (size_t)first * blk_bytes;
            }
        }
    };
    for (uint32_t gdone = 0; gdone < ngroups; gdone += D) {
        static_for<D>([&](auto dc) {
            if (gdone + (uint32_t)decltype(dc)::value < ngroups) step(dc);
        });
    }

    // add the K shares of a row group (in share order) through LDS
    if (ks > 1) {
        __syncthreads();
        float *red = reinterpret_cast<float *>(A_lds);             // [ks][rw][64]
        if (ks_id > 0) red[((size_t)ks_id * rw + rw_id) * 64 + lane] = yacc;
        __syncthreads();
        if (ks_id > 0) return;
        for (uint32_t o = 1; o < ks; ++o) yacc += red[((size_t)o * rw + rw_id) * 64 + lane];
    }
    if (nrow < N && g < nb) {
        const float bias = elem_value_rt(a.L.bias_fmt, a.L.bias, nrow) * a.L.bscale;
        float dot = yacc;
        if (dot != dot) {
            // the sample's input holds an infinity or a NaN (the integer sums themselves are always finite):
            // plain FP32 multiply-adds over the row, in k order
            const float *xs = a.x + (size_t)g * K;
            const uint64_t base = (uint64_t)nrow * K;
            dot = 0.0f;
            for (uint32_t k = 0; k < K; ++k) dot = fmaf((float)int_code<FMT>(a.L.w, base + k), xs[k], dot);
        }
        a.y[(size_t)g * N + nrow] = apply_act(fmaf(dot, a.L.wscale, bias), a.L.act);
    }
}

// Two-launch form (planes prepared by sp_quant_x; more than four samples, reachable with SPHIP_FORCE_GEMV).
// MT = 16-row A tiles (four samples each).  Rows of D that belong to no sample
// (fourth row of a slot, slots beyond nb) are never read, so their lanes may load
// anything: they are pointed at the start of the block.
// The waves of a workgroup are rw row groups x ks K shares (wave = ks_id * rw +
// rw_id); share ks_id takes the 64-byte blocks ks_id, ks_id + ks, ... of its rows.
// Weights are fetched in groups of four blocks, the next group in flight while
// the current one is multiplied; scale chunks are whole numbers of groups.
//
// FQ = 1, 2 select the self-quantising form above instead (one launch per layer; 1: K shares of whole lines, 2: of blocks).
template <int FMT, int MT, int FQ>
__global__ __launch_bounds__(FQ ? 1024 : MT <= 4 ? 1024 : 256) void sp_gemv_i8mfma(const GemvI8Args a)
{
    if constexpr (FQ != 0) {
        static_assert(FQ == 0 || MT == 1, "the self-quantising form carries at most four samples");
        if constexpr (FQ == 1) gemv_i8_specialised<FMT, 3, 2, true>(a);
        else gemv_i8_specialised<FMT, 2, 4, false>(a);
        return;
    }
    using F = I8Fmt<FMT>;
    constexpr int KL = F::KL, NMF = F::NMF, G = 4;
    extern __shared__ __attribute__((aligned(16))) uint8_t lds_all[];
    // [nchunks][nb] {2^-p bits, d0 sum, d1 sum, d2 sum}, then the digit planes of one stage:
    // [stage blocks][NMF][4 g][nb][3][16 bytes]
    int4 *meta = reinterpret_cast<int4 *>(lds_all);
    uint8_t *A_lds = lds_all + a.meta_bytes;

    const int t = threadIdx.x, lane = t & 63, wave = t >> 6;
    const uint32_t nthreads = blockDim.x;
    const uint32_t N = a.L.N, K = a.L.K;
    const int nb = a.nb;
    const uint32_t rw = a.rw, ks = a.ks, ks_id = (uint32_t)wave / rw, rw_id = (uint32_t)wave % rw;
    const uint32_t nrow = (blockIdx.x * rw + rw_id) * 16u + (lane & 15);
    const uint32_t g = lane >> 4;
    const size_t row_bytes = (size_t)K * F::bits / 8u;
    const uint8_t *wrow = a.L.w + (size_t)(nrow < N ? nrow : N - 1) * row_bytes + g * 16u + ks_id * 64u;
    // largest offset (from wrow) whose 16 bytes stay inside the row; reads past it are clamped there
    // and meet zero digits
    const int64_t row_last = (int64_t)row_bytes - 16 - (int64_t)(g * 16u + ks_id * 64u);
    const uint32_t kcb = a.kc / KL;                           // blocks per scale chunk
    const uint32_t blk_bytes = (uint32_t)NMF * 4u * (uint32_t)nb * 48u;   // digit planes of one block
    const uint32_t u_bytes = 4u * (uint32_t)nb * 48u;
    const uint32_t qstep = ks * 64u;                          // byte distance of this wave's consecutive blocks
    const uint32_t groups_per_chunk = kcb / (ks * G);         // host guarantees divisibility
    const uint32_t chunks_per_stage = a.stage_blocks / kcb;

    uint32_t a_off[MT];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
        const uint32_t m = lane & 15u, slot = (uint32_t)mt * 4u + (m >> 2), d = m & 3u;
        a_off[mt] = (slot < (uint32_t)nb && d < 3u) ? ((g * (uint32_t)nb + slot) * 3u + d) * 16u : 0u;
    }

    float yacc[MT];
    i32x4v acc[2][MT];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
        yacc[mt] = 0.0f;
        acc[0][mt] = acc[1][mt] = (i32x4v){0, 0, 0, 0};
    }

    auto load_blk = [&](uint32_t q) {                          // q-th block of this wave
        int64_t off = (int64_t)q * qstep;
        off = off < row_last ? off : row_last;
        off = off > 0 ? off : 0;
        return *reinterpret_cast<const uint4 *>(wrow + off);
    };
    auto process = [&](const uint4 wv, const uint8_t *rec) {
        const uint32_t w[4] = {wv.x, wv.y, wv.z, wv.w};
        i32x4v bop[NMF];
        if constexpr (FMT == I8) {
            bop[0] = (i32x4v){(int)w[0], (int)w[1], (int)w[2], (int)w[3]};
        } else if constexpr (FMT == I4) {
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                const uint32_t x8 = w[q] ^ 0x88888888u;          // nibble -> q + 8
                bop[0][q] = (int)(x8 & 0x0F0F0F0Fu);
                bop[1][q] = (int)((x8 >> 4) & 0x0F0F0F0Fu);
            }
        } else {
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                const uint32_t x2 = w[q] ^ 0xAAAAAAAAu;          // field -> q + 2
                bop[0][q] = (int)(x2 & 0x03030303u);
                bop[1][q] = (int)((x2 >> 2) & 0x03030303u);
                bop[2][q] = (int)((x2 >> 4) & 0x03030303u);
                bop[3][q] = (int)((x2 >> 6) & 0x03030303u);
            }
        }
#pragma unroll
        for (int f = 0; f < NMF; ++f)
#pragma unroll
            for (int mt = 0; mt < MT; ++mt) {
                const i32x4v aop = *reinterpret_cast<const i32x4v *>(rec + f * u_bytes + a_off[mt]);
                acc[f & 1][mt] = __builtin_amdgcn_mfma_i32_16x16x64_i8(aop, bop[f], acc[f & 1][mt], 0, 0, 0);
            }
    };
    auto fold = [&](uint32_t ch) {
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
            const int s0 = mt * 4 + (int)g;
            if (s0 < nb) {
                const int4 md = meta[(size_t)ch * nb + s0];
                int S0 = acc[0][mt][0] + acc[1][mt][0], S1 = acc[0][mt][1] + acc[1][mt][1], S2 = acc[0][mt][2] + acc[1][mt][2];
                if (F::BIAS != 0 && ks_id == 0) {       // one K share removes the code bias of the whole chunk
                    S0 -= F::BIAS * md.y;
                    S1 -= F::BIAS * md.z;
                    S2 -= F::BIAS * md.w;
                }
                const float tsum = fmaf((float)S2, 65536.0f, fmaf((float)S1, 256.0f, (float)S0));
                yacc[mt] = fmaf(tsum, __int_as_float(md.x), yacc[mt]);
            }
            acc[0][mt] = acc[1][mt] = (i32x4v){0, 0, 0, 0};
        }
    };

    // the first weight group
    constexpr int PD = 1;
    uint4 nxt[PD][G];
#pragma unroll
    for (int d = 0; d < PD; ++d)
#pragma unroll
        for (int u = 0; u < G; ++u) nxt[d][u] = load_blk((uint32_t)(d * G + u));

    // scale records of all chunks
    for (uint32_t i = t; i < a.nchunks * (uint32_t)nb; i += nthreads) {
        const int *d = a.dsum + (size_t)i * 4;
        meta[i] = make_int4(__float_as_int(a.inv[i]), d[0], d[1], d[2]);
    }

    uint32_t q = 0;                                            // this wave's block counter
    for (uint32_t ch0 = 0; ch0 < a.nchunks; ch0 += chunks_per_stage) {
        const uint32_t nch = ch0 + chunks_per_stage <= a.nchunks ? chunks_per_stage : a.nchunks - ch0;
        if (ch0) __syncthreads();                             // previous stage fully consumed
        {
            const uint4 *src = reinterpret_cast<const uint4 *>(a.aq + (size_t)ch0 * kcb * blk_bytes);
            const uint32_t pieces = nch * kcb * (blk_bytes / 16u);
            for (uint32_t i = t; i < pieces; i += nthreads) reinterpret_cast<uint4 *>(A_lds)[i] = src[i];
        }
        __syncthreads();
        const uint8_t *rec = A_lds + (size_t)ks_id * blk_bytes;
        const size_t rstep = (size_t)ks * blk_bytes;
        for (uint32_t ch = ch0; ch < ch0 + nch; ++ch) {
            for (uint32_t gi = 0; gi < groups_per_chunk; ++gi) {
                uint4 cur[G];
#pragma unroll
                for (int u = 0; u < G; ++u) cur[u] = nxt[0][u];
                q += G;
#pragma unroll
                for (int d = 0; d + 1 < PD; ++d)
#pragma unroll
                    for (int u = 0; u < G; ++u) nxt[d][u] = nxt[d + 1][u];
#pragma unroll
                for (int u = 0; u < G; ++u) nxt[PD - 1][u] = load_blk(q + (PD - 1) * G + u);
#pragma unroll
                for (int u = 0; u < G; ++u) process(cur[u], rec + (size_t)u * rstep);
                rec += G * rstep;
            }
            fold(ch);
        }
    }

    // add the K shares of a row group (in share order) through LDS
    if (ks > 1) {
        __syncthreads();
        float *red = reinterpret_cast<float *>(A_lds);         // [ks][rw][MT][64]
        if (ks_id > 0) {
#pragma unroll
            for (int mt = 0; mt < MT; ++mt) red[(((size_t)ks_id * rw + rw_id) * MT + mt) * 64 + lane] = yacc[mt];
        }
        __syncthreads();
        if (ks_id > 0) return;
        for (uint32_t o = 1; o < ks; ++o)
#pragma unroll
            for (int mt = 0; mt < MT; ++mt) yacc[mt] += red[(((size_t)o * rw + rw_id) * MT + mt) * 64 + lane];
    }

    if (nrow < N) {
        const float bias = elem_value_rt(a.L.bias_fmt, a.L.bias, nrow) * a.L.bscale;
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
            const int s0 = mt * 4 + (int)g;
            if (s0 >= nb) continue;
            float dot = yacc[mt];
            if (dot != dot) {
                // the sample's input holds an infinity or a NaN (the integer sums themselves are always finite):
                // plain FP32 multiply-adds over the row, in k order
                const float *xs = a.x + (size_t)s0 * K;
                const uint64_t base = (uint64_t)nrow * K;
                dot = 0.0f;
                for (uint32_t k = 0; k < K; ++k) dot = fmaf((float)int_code<FMT>(a.L.w, base + k), xs[k], dot);
            }
            a.y[(size_t)s0 * N + nrow] = apply_act(fmaf(dot, a.L.wscale, bias), a.L.act);
        }
    }
}
