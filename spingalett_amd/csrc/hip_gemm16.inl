// hip_gemm16.inl — the LDS-tiled 16-bit MFMA GEMM for larger batches (sp_gemm16, sp_gemm16_big,
// sp_gemm16_reduce).  Part of hip_forward.hip's translation unit (included there, inside its unnamed
// namespace); not compiled on its own.

// ---------------------------------------------------------------------------
// 16-bit MFMA GEMM (n > 64): C[M][N] = act(bias + scale * A[M][K] . Wq[N][K]^T)
// ---------------------------------------------------------------------------
typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8;
typedef __attribute__((__vector_size__(8 * sizeof(_Float16)))) _Float16 f16x8;
typedef __attribute__((__vector_size__(16 * sizeof(float)))) float f32x16;

struct GemmArgs {
    LayerArgs L;
    const uint16_t *A;     // [M][K] 16-bit activations
    void *C;               // [M][N] 16-bit, or FP32 when out_f32
    uint32_t M;
    int out_f32;
    float *ws;             // [grid y][M][N] partial sums when grid y splits the product, else nullptr
    uint32_t kper;         // k range of one K split, a multiple of 64 (0: all of K)
    // Split activations: the layer input is two 16-bit matrices, hi and (a - hi) 2^11, the second M K elements
    // behind the first; grid y = halves x ksplits, y / ksplits picks the matrix, y % ksplits the K range.
    uint32_t ksplits;      // K splits (>= 1)
    uint32_t halves;       // 1, or 2 with split activations
};

// 2^-11: what the partial sums of the second activation matrix are scaled by
constexpr float kLoScale = 1.0f / 2048.0f;

// hi and lo of a split activation: hi = v rounded to FP16, lo = (v - hi) 2^11 rounded to FP16 (v - hi is exact in FP32)
__device__ __forceinline__ void split_f16(float v, uint16_t &hi, uint16_t &lo)
{
    hi = f32_to_f16_sat(v);
    _Float16 hh;
    __builtin_memcpy(&hh, &hi, 2);
    const float rest = (v - (float)hh) * 2048.0f;
    lo = (rest == rest && fabsf(rest) != __builtin_inff()) ? f32_to_f16_sat(rest) : (uint16_t)0;   // inf / NaN live in hi
}

// (float)q as a 16-bit float; exact for |q| <= 128 in either type
template <bool F16T>
__device__ __forceinline__ uint32_t int_to_t16(int q)
{
    if constexpr (F16T) {
        _Float16 h = (_Float16)q;
        uint16_t r;
        __builtin_memcpy(&r, &h, 2);
        return r;
    } else {
        return __float_as_uint((float)q) >> 16;
    }
}

// packed FP16 subtraction a - c (two lanes at once)
__device__ __forceinline__ uint32_t h2_sub(uint32_t v, uint32_t c)
{
    typedef _Float16 h2 __attribute__((ext_vector_type(2)));
    h2 a, b;
    __builtin_memcpy(&a, &v, 4);
    __builtin_memcpy(&b, &c, 4);
    a = a - b;
    uint32_t r;
    __builtin_memcpy(&r, &a, 4);
    return r;
}

// unpack one 32-bit word of codes into 16-bit floats, written as packed pairs (codes 0 1, 2 3, ...)
template <int FMT, bool F16T>
__device__ __forceinline__ void unpack_word16(uint32_t w, uint32_t *o)
{
    constexpr int bits = fmt_bits(FMT);
    constexpr int cnt = 32 / bits;
    if constexpr (F16T && (FMT == I8 || FMT == I4 || FMT == I2)) {
        // A field masked in place and XORed onto an FP16 constant whose last mantissa bit weighs as much as
        // the field's lowest bit (the same XOR flips the sign bit: two's complement -> offset binary) reads
        // as constant + offset + code; one packed subtraction leaves the codes of two fields, exactly.  The
        // pairs come out as (code k, code k + cnt/2) and a byte permute puts neighbours together.
        constexpr uint32_t LO = 0x05040100u, HI = 0x07060302u;      // low / high halves of two words
        if constexpr (FMT == I8) {
            const uint32_t t0 = h2_sub((w & 0x00FF00FFu) ^ 0x64806480u, 0x64806480u);            // codes 0, 2
            const uint32_t t1 = h2_sub(((w >> 8) & 0x00FF00FFu) ^ 0x64806480u, 0x64806480u);     // codes 1, 3
            o[0] = __builtin_amdgcn_perm(t1, t0, LO);
            o[1] = __builtin_amdgcn_perm(t1, t0, HI);
        } else if constexpr (FMT == I4) {
            const uint32_t y = w >> 8;
            const uint32_t t0 = h2_sub((w & 0x000F000Fu) ^ 0x64086408u, 0x64086408u);            // codes 0, 4
            const uint32_t t1 = h2_sub((w & 0x00F000F0u) ^ 0x54805480u, 0x54805480u);            // codes 1, 5
            const uint32_t t2 = h2_sub((y & 0x000F000Fu) ^ 0x64086408u, 0x64086408u);            // codes 2, 6
            const uint32_t t3 = h2_sub((y & 0x00F000F0u) ^ 0x54805480u, 0x54805480u);            // codes 3, 7
            o[0] = __builtin_amdgcn_perm(t1, t0, LO);
            o[1] = __builtin_amdgcn_perm(t3, t2, LO);
            o[2] = __builtin_amdgcn_perm(t1, t0, HI);
            o[3] = __builtin_amdgcn_perm(t3, t2, HI);
        } else {
            const uint32_t y = w >> 10;
            uint32_t p[8];                                                                        // codes k, k + 8
            p[0] = h2_sub((w & 0x00030003u) ^ 0x64026402u, 0x64026402u);
            p[1] = h2_sub((w & 0x000C000Cu) ^ 0x5C085C08u, 0x5C085C08u);
            p[2] = h2_sub((w & 0x00300030u) ^ 0x54205420u, 0x54205420u);
            p[3] = h2_sub((w & 0x00C000C0u) ^ 0x4C804C80u, 0x4C804C80u);
            p[4] = h2_sub((w & 0x03000300u) ^ 0x46004600u, 0x46004600u);
            p[5] = h2_sub((y & 0x00030003u) ^ 0x64026402u, 0x64026402u);
            p[6] = h2_sub((y & 0x000C000Cu) ^ 0x5C085C08u, 0x5C085C08u);
            p[7] = h2_sub((y & 0x00300030u) ^ 0x54205420u, 0x54205420u);
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                o[q]     = __builtin_amdgcn_perm(p[2 * q + 1], p[2 * q], LO);
                o[4 + q] = __builtin_amdgcn_perm(p[2 * q + 1], p[2 * q], HI);
            }
        }
        return;
    }
#pragma unroll
    for (int j = 0; j < cnt; j += 2) {
        int q0 = (int)(w << (32 - bits - bits * j)) >> (32 - bits);
        int q1 = (int)(w << (32 - bits - bits * (j + 1))) >> (32 - bits);
        o[j / 2] = int_to_t16<F16T>(q0) | (int_to_t16<F16T>(q1) << 16);
    }
}

// Tile: BM x BN x BK (BK = 64, or 128 for a K of 1024 and more), 256 threads = 2 x 2 waves, each wave TM x TN tiles of
// 32x32.  A K split (g.kper, whole tiles of 64) goes with BK = 64 only.
// LDS rows are padded by 8 elements so that 128-bit fragment reads of 32
// consecutive rows spread over the banks.
// W4 (integer codes, ALIGNED activations): the weight rows are whole 32-bit words but not whole 16-byte units
// (784 INT4 codes = 392 bytes): the codes are fetched a word at a time instead of element by element.
template <int FMT, bool F16T, int TM, int TN, bool ALIGNED, bool W4 = false, int BK = 64>
__global__ __launch_bounds__(256) void sp_gemm16(const GemmArgs g)
{
    static_assert(!W4 || (ALIGNED && (FMT == I8 || FMT == I4 || FMT == I2)), "word loads: integer codes, aligned activations");
    constexpr int BM = 64 * TM, BN = 64 * TN, LDK = BK + 8;
    constexpr int KCH = BK / 8;                     // 16-byte pieces of a tile row of activations
    constexpr int bits = fmt_bits(FMT);
    constexpr int EPL = 128 / bits;                 // weight elements per 16-byte load
    constexpr int W_LOADS = (BN * BK / EPL + 255) / 256;
    constexpr int A_LOADS = BM * BK / 8 / 256;
    constexpr int CW = 32 / bits;                   // codes per 32-bit word
    constexpr int W4_LOADS = (BN * BK / CW + 255) / 256;

    __shared__ __attribute__((aligned(16))) uint16_t As[BM * LDK];
    __shared__ __attribute__((aligned(16))) uint16_t Ws[BN * LDK];

    const uint32_t M = g.M, N = g.L.N, K = g.L.K;
    const int t = threadIdx.x, lane = t & 63, wave = t >> 6;
    const int wm = wave >> 1, wn = wave & 1;
    // grid y = halves x K splits: y / ksplits picks the matrix of a split activation, y % ksplits the K range (whole tiles)
    const uint16_t *const A = g.A + (size_t)(blockIdx.y / g.ksplits) * M * K;
    const uint32_t kbeg = g.kper ? (blockIdx.y % g.ksplits) * g.kper : 0u;
    const uint32_t kend = g.kper && kbeg + g.kper < K ? kbeg + g.kper : K;

    // tile index: consecutive workgroups go to different XCDs, so give each XCD a
    // contiguous band of tiles (shared A rows / W rows stay in one L2)
    const uint32_t tiles_n = (N + BN - 1) / BN, tiles_m = (M + BM - 1) / BM;
    const uint32_t ntiles = tiles_m * tiles_n;
    uint32_t bid = blockIdx.x;
    {
        const uint32_t per = ntiles / 8u;
        if (bid < per * 8u) bid = (bid & 7u) * per + (bid >> 3);
    }
    const uint32_t tm = bid / tiles_n, tn = bid % tiles_n;
    const uint32_t m0 = tm * BM, n0 = tn * BN;

    f32x16 acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.0f;

    uint4 ra[A_LOADS], rw[W4 ? 1 : W_LOADS];
    uint32_t rw4[W4 ? W4_LOADS : 1];
    const size_t w_row_bytes = (size_t)K * bits / 8u;

    auto load_tiles = [&](uint32_t k0) {
        if constexpr (ALIGNED) {
#pragma unroll
            for (int i = 0; i < A_LOADS; ++i) {
                const int c = t + 256 * i, row = c / KCH, kc = c % KCH;
                const uint32_t m = m0 + row < M ? m0 + row : M - 1;
                const uint32_t k = k0 + kc * 8;
                ra[i] = k < K ? *reinterpret_cast<const uint4 *>(A + (size_t)m * K + k) : make_uint4(0, 0, 0, 0);
            }
            if constexpr (W4) {
#pragma unroll
                for (int i = 0; i < W4_LOADS; ++i) {
                    const int c = t + 256 * i;
                    constexpr int LPR = BK / CW;        // words per tile row
                    const int row = c / LPR, kc = c % LPR;
                    const uint32_t n = n0 + row < N ? n0 + row : N - 1;
                    const uint32_t k = k0 + kc * CW;
                    const bool ok = (row < BN) && (k < K);      // K is a whole number of words: k < K means k + CW <= K
                    rw4[i] = ok ? *reinterpret_cast<const uint32_t *>(g.L.w + (size_t)n * w_row_bytes + (size_t)k * bits / 8u) : 0u;
                }
            } else {
#pragma unroll
                for (int i = 0; i < W_LOADS; ++i) {
                    const int c = t + 256 * i;
                    constexpr int LPR = BK / EPL;           // loads per tile row
                    const int row = c / LPR, kc = c % LPR;
                    const uint32_t n = n0 + row < N ? n0 + row : N - 1;
                    const uint32_t k = k0 + kc * EPL;
                    const bool ok = (row < BN) && (k < K);
                    rw[i] = ok ? *reinterpret_cast<const uint4 *>(g.L.w + (size_t)n * w_row_bytes + (size_t)k * bits / 8u)
                               : make_uint4(0, 0, 0, 0);
                }
            }
        }
    };

    auto store_tiles = [&](uint32_t k0) {
        if constexpr (ALIGNED) {
#pragma unroll
            for (int i = 0; i < A_LOADS; ++i) {
                const int c = t + 256 * i, row = c / KCH, kc = c % KCH;
                *reinterpret_cast<uint4 *>(&As[row * LDK + kc * 8]) = ra[i];
            }
            if constexpr (W4) {
#pragma unroll
                for (int i = 0; i < W4_LOADS; ++i) {
                    const int c = t + 256 * i;
                    constexpr int LPR = BK / CW;
                    const int row = c / LPR, kc = c % LPR;
                    if (row >= BN) continue;
                    constexpr int PW = 16 / bits;       // packed pairs per 32-bit word: 2, 4 or 8
                    uint32_t o[PW];
                    unpack_word16<FMT, F16T>(rw4[i], o);
                    uint16_t *dst = &Ws[row * LDK + kc * CW];
                    if constexpr (PW == 2) {
                        *reinterpret_cast<uint2 *>(dst) = make_uint2(o[0], o[1]);
                    } else {
#pragma unroll
                        for (int v = 0; v < PW / 4; ++v)
                            *reinterpret_cast<uint4 *>(dst + v * 8) = make_uint4(o[4 * v], o[4 * v + 1], o[4 * v + 2], o[4 * v + 3]);
                    }
                }
            }
#pragma unroll
            for (int i = 0; i < (W4 ? 0 : W_LOADS); ++i) {
                const int c = t + 256 * i;
                constexpr int LPR = BK / EPL;
                const int row = c / LPR, kc = c % LPR;
                if (row >= BN) continue;
                uint16_t *dst = &Ws[row * LDK + kc * EPL];
                if constexpr (FMT == BF16 || FMT == F16) {
                    *reinterpret_cast<uint4 *>(dst) = rw[i];
                } else {
                    const uint32_t w[4] = {rw[i].x, rw[i].y, rw[i].z, rw[i].w};
                    constexpr int PW = 16 / bits;       // packed pairs per 32-bit word
                    uint32_t o[4 * PW];
#pragma unroll
                    for (int q = 0; q < 4; ++q) unpack_word16<FMT, F16T>(w[q], o + q * PW);
#pragma unroll
                    for (int v = 0; v < PW; ++v)
                        *reinterpret_cast<uint4 *>(dst + v * 8) = make_uint4(o[4 * v], o[4 * v + 1], o[4 * v + 2], o[4 * v + 3]);
                }
            }
        } else {
            // element-wise, fully bounds-checked
            for (int e = t; e < BM * BK; e += 256) {
                const int row = e / BK, kk = e % BK;
                const uint32_t m = m0 + row, k = k0 + kk;
                As[row * LDK + kk] = (m < M && k < K) ? A[(size_t)m * K + k] : (uint16_t)0;
            }
            for (int e = t; e < BN * BK; e += 256) {
                const int row = e / BK, kk = e % BK;
                const uint32_t n = n0 + row, k = k0 + kk;
                uint16_t v = 0;
                if (n < N && k < K) {
                    const uint64_t idx = (uint64_t)n * K + k;
                    if constexpr (FMT == BF16 || FMT == F16) v = reinterpret_cast<const uint16_t *>(g.L.w)[idx];
                    else if constexpr (FMT == F32) v = f32_to_t16<F16T>(reinterpret_cast<const float *>(g.L.w)[idx]);
                    else v = (uint16_t)int_to_t16<F16T>(int_code<FMT>(g.L.w, idx));
                }
                Ws[row * LDK + kk] = v;
            }
        }
    };

    const uint32_t ktiles = (kend - kbeg + BK - 1) / BK;
    load_tiles(kbeg);
    for (uint32_t kt = 0; kt < ktiles; ++kt) {
        __syncthreads();                              // previous tile fully consumed
        store_tiles(kbeg + kt * BK);
        __syncthreads();
        if (kt + 1 < ktiles) load_tiles(kbeg + (kt + 1) * BK);

#pragma unroll
        for (int ks = 0; ks < BK; ks += 16) {
            const int koff = ks + 8 * (lane >> 5);
            uint4 fa[TM], fb[TN];
#pragma unroll
            for (int i = 0; i < TM; ++i)
                fa[i] = *reinterpret_cast<const uint4 *>(&As[(wm * TM * 32 + i * 32 + (lane & 31)) * LDK + koff]);
#pragma unroll
            for (int j = 0; j < TN; ++j)
                fb[j] = *reinterpret_cast<const uint4 *>(&Ws[(wn * TN * 32 + j * 32 + (lane & 31)) * LDK + koff]);
#pragma unroll
            for (int i = 0; i < TM; ++i)
#pragma unroll
                for (int j = 0; j < TN; ++j) {
                    if constexpr (F16T) {
                        f16x8 a, b;
                        __builtin_memcpy(&a, &fa[i], 16);
                        __builtin_memcpy(&b, &fb[j], 16);
                        acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, acc[i][j], 0, 0, 0);
                    } else {
                        bf16x8 a, b;
                        __builtin_memcpy(&a, &fa[i], 16);
                        __builtin_memcpy(&b, &fb[j], 16);
                        acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, acc[i][j], 0, 0, 0);
                    }
                }
        }
    }

    if (g.ws) {                                        // partial sums of one activation matrix: a second launch adds them
#pragma unroll
        for (int j = 0; j < TN; ++j) {
            const uint32_t col = n0 + wn * TN * 32 + j * 32 + (lane & 31);
            if (col >= N) continue;
#pragma unroll
            for (int i = 0; i < TM; ++i)
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    const uint32_t row = m0 + wm * TM * 32 + i * 32 + 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3);
                    if (row < M) g.ws[((size_t)blockIdx.y * M + row) * N + col] = acc[i][j][r];
                }
        }
        return;
    }
    // epilogue: scale, bias, activation, store.  Sigmoid and tanh have a copy of the loops to themselves: a switch
    // over all activations behind every one of a lane's outputs is mostly their code, fetched for nothing.
    const float wscale = g.L.wscale;
    // 16-bit outputs in rows of whole 16-byte units: a wave turns each 32 x 32 block around in LDS (the tiles' memory,
    // free once every wave has read its last fragments) and stores 16 bytes per lane, two store instructions per
    // block instead of sixteen two-byte ones
    const bool rows16 = !g.out_f32 && N % 8u == 0 && (reinterpret_cast<uintptr_t>(g.C) & 15u) == 0;     // (uniform)
    if (rows16) __syncthreads();
    constexpr int SP = 40;                                   // row pitch of a wave's 32 x 32 staging block, elements
    uint16_t *const stage = (wave < 2 ? As : Ws) + (wave & 1) * (32 * SP);
    auto emit = [&](auto slow_c) __attribute__((always_inline)) {
        constexpr bool SLOW = decltype(slow_c)::value;
        if (rows16) {
#pragma unroll
            for (int j = 0; j < TN; ++j) {
                const uint32_t col = n0 + wn * TN * 32 + j * 32 + (lane & 31);
                const float bias = elem_value_rt(g.L.bias_fmt, g.L.bias, col < N ? col : N - 1) * g.L.bscale;
#pragma unroll
                for (int i = 0; i < TM; ++i) {
#pragma unroll
                    for (int r = 0; r < 16; ++r) {
                        const float pre = fmaf(acc[i][j][r], wscale, bias);
                        const float v = SLOW ? apply_act(pre, g.L.act) : apply_act_cheap(pre, g.L.act);
                        stage[(8 * (r >> 2) + 4 * (lane >> 5) + (r & 3)) * SP + (lane & 31)] = f32_to_t16<F16T>(v);
                    }
                    __builtin_amdgcn_wave_barrier();
#pragma unroll
                    for (int p = 0; p < 2; ++p) {
                        const int rr = (lane >> 2) + 16 * p, ch = lane & 3;
                        const uint4 d = *reinterpret_cast<const uint4 *>(&stage[rr * SP + ch * 8]);
                        const uint32_t row = m0 + wm * TM * 32 + i * 32 + rr, c0 = n0 + wn * TN * 32 + j * 32 + ch * 8;
                        if (row < M && c0 < N) *reinterpret_cast<uint4 *>(reinterpret_cast<uint16_t *>(g.C) + (size_t)row * N + c0) = d;
                    }
                    __builtin_amdgcn_wave_barrier();
                }
            }
            return;
        }
#pragma unroll
        for (int j = 0; j < TN; ++j) {
            const uint32_t col = n0 + wn * TN * 32 + j * 32 + (lane & 31);
            if (col >= N) continue;
            const float bias = elem_value_rt(g.L.bias_fmt, g.L.bias, col) * g.L.bscale;
#pragma unroll
            for (int i = 0; i < TM; ++i) {
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    const uint32_t row = m0 + wm * TM * 32 + i * 32 + 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3);
                    if (row >= M) continue;
                    const float pre = fmaf(acc[i][j][r], wscale, bias);
                    const float v = SLOW ? apply_act(pre, g.L.act) : apply_act_cheap(pre, g.L.act);
                    const size_t o = (size_t)row * N + col;
                    if (g.out_f32) reinterpret_cast<float *>(g.C)[o] = v;
                    else reinterpret_cast<uint16_t *>(g.C)[o] = f32_to_t16<F16T>(v);
                }
            }
        }
    };
    if (g.L.act == A_SIGMOID || g.L.act == A_TANH) emit(std::true_type{});
    else emit(std::false_type{});
}

// Small layers in one launch: a workgroup owns a 32 x 32 tile of the output, its eight waves split K in whole steps of
// 32, and their sums meet in LDS.  No operand staging: in step s lane (r, h) loads the sixteen consecutive elements
// k = 32 s + 16 h .. + 15 of row r of both operands straight into registers, as two pieces of eight (K % 8 == 0: a piece
// is inside its row or beyond it), and feeds a piece of each operand to one MFMA (a sum over k in any order).  For
// outputs of a few hundred tiles, where the streaming and the tiled kernels need a K split over the grid and a second
// launch to fill the chip.  XF32: the activations are still the caller's FP32 input, rounded here as sp_cvt16 (or, with
// split activations, sp_cvt16_split) would (g.A then points at floats).  HALVES == 2: split activations, two FP16
// matrices hi and lo = (a - hi) 2^11, M K elements apart; a second accumulator takes the lo products, a wave adds it,
// times 2^-11, to its hi sum, and 16-bit outputs leave as the two matrices of the next layer's input.
template <int FMT, bool F16T, bool XF32, int HALVES = 1>
__global__ __launch_bounds__(512) void sp_gemm16_small(const GemmArgs g)
{
    static_assert(HALVES == 1 || F16T, "split activations are FP16");
    constexpr int NW = 8, U = 2;
    constexpr int bits = fmt_bits(FMT);
    constexpr int PB = bits;                           // bytes of a piece of eight weights
    __shared__ float part[NW][32 * 33];
    const uint32_t M = g.M, N = g.L.N, K = g.L.K;
    const int t = threadIdx.x, lane = t & 63, wave = t >> 6, q = lane & 31, h = lane >> 5;
    const uint32_t tiles_n = (N + 31u) / 32u;
    const uint32_t m0 = (blockIdx.x / tiles_n) * 32u, n0 = (blockIdx.x % tiles_n) * 32u;
    const uint32_t steps = (K + 31u) / 32u, per = (steps + NW - 1) / NW;
    const uint32_t s0 = wave * per, s1 = s0 + per < steps ? s0 + per : steps;
    const uint32_t am = m0 + q < M ? m0 + q : M - 1, wn = n0 + q < N ? n0 + q : N - 1;
    const uint16_t *ap16 = g.A + (size_t)am * K + 16 * h;
    const float *ap32 = reinterpret_cast<const float *>(g.A) + (size_t)am * K + 16 * h;
    const uint8_t *wp = g.L.w + (size_t)wn * ((size_t)K * bits / 8u) + (size_t)(2 * h) * PB;

    struct Frag { uint4 a[2], al[HALVES == 2 ? 2 : 1], w[2]; };
    auto ld = [&](uint32_t s) -> Frag {
        Frag f;
#pragma unroll
        for (int p = 0; p < 2; ++p) {
            const bool ok = 32u * s + 16u * h + 8u * p < K;
            if constexpr (XF32) {
                const float4 lo = ok ? *reinterpret_cast<const float4 *>(ap32 + 32u * s + 8 * p) : make_float4(0.0f, 0.0f, 0.0f, 0.0f);
                const float4 hi = ok ? *reinterpret_cast<const float4 *>(ap32 + 32u * s + 8 * p + 4) : make_float4(0.0f, 0.0f, 0.0f, 0.0f);
                if constexpr (HALVES == 2) {
                    const float v[8] = {lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
                    uint16_t eh[8], el[8];
#pragma unroll
                    for (int e = 0; e < 8; ++e) split_f16(v[e], eh[e], el[e]);
                    f.a[p] = make_uint4((uint32_t)eh[0] | ((uint32_t)eh[1] << 16), (uint32_t)eh[2] | ((uint32_t)eh[3] << 16),
                                        (uint32_t)eh[4] | ((uint32_t)eh[5] << 16), (uint32_t)eh[6] | ((uint32_t)eh[7] << 16));
                    f.al[p] = make_uint4((uint32_t)el[0] | ((uint32_t)el[1] << 16), (uint32_t)el[2] | ((uint32_t)el[3] << 16),
                                         (uint32_t)el[4] | ((uint32_t)el[5] << 16), (uint32_t)el[6] | ((uint32_t)el[7] << 16));
                } else {
                    f.a[p].x = (uint32_t)f32_to_t16<F16T>(lo.x) | ((uint32_t)f32_to_t16<F16T>(lo.y) << 16);
                    f.a[p].y = (uint32_t)f32_to_t16<F16T>(lo.z) | ((uint32_t)f32_to_t16<F16T>(lo.w) << 16);
                    f.a[p].z = (uint32_t)f32_to_t16<F16T>(hi.x) | ((uint32_t)f32_to_t16<F16T>(hi.y) << 16);
                    f.a[p].w = (uint32_t)f32_to_t16<F16T>(hi.z) | ((uint32_t)f32_to_t16<F16T>(hi.w) << 16);
                }
            } else {
                f.a[p] = ok ? *reinterpret_cast<const uint4 *>(ap16 + 32u * s + 8 * p) : make_uint4(0, 0, 0, 0);
                if constexpr (HALVES == 2)
                    f.al[p] = ok ? *reinterpret_cast<const uint4 *>(ap16 + (size_t)M * K + 32u * s + 8 * p) : make_uint4(0, 0, 0, 0);
            }
            const uint8_t *src = wp + (size_t)s * (4 * PB) + p * PB;
            if constexpr (FMT == F16 || FMT == BF16) {
                f.w[p] = ok ? *reinterpret_cast<const uint4 *>(src) : make_uint4(0, 0, 0, 0);
            } else if constexpr (FMT == I8) {
                const uint2 c = ok ? *reinterpret_cast<const uint2 *>(src) : make_uint2(0, 0);
                f.w[p].x = c.x; f.w[p].y = c.y;
            } else if constexpr (FMT == I4) {
                f.w[p].x = ok ? *reinterpret_cast<const uint32_t *>(src) : 0u;
            } else {
                f.w[p].x = ok ? (uint32_t)*reinterpret_cast<const uint16_t *>(src) : 0u;
            }
        }
        return f;
    };
    f32x16 acc, accl;
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[r] = accl[r] = 0.0f;
    auto fma2 = [&](const Frag &f) {
#pragma unroll
        for (int p = 0; p < 2; ++p) {
            uint4 wv = f.w[p];
            if constexpr (FMT == I8) {
                uint32_t o[4];
                unpack_word16<I8, F16T>(f.w[p].x, o);
                unpack_word16<I8, F16T>(f.w[p].y, o + 2);
                wv = make_uint4(o[0], o[1], o[2], o[3]);
            } else if constexpr (FMT == I4) {
                uint32_t o[4];
                unpack_word16<I4, F16T>(f.w[p].x, o);
                wv = make_uint4(o[0], o[1], o[2], o[3]);
            } else if constexpr (FMT == I2) {
                uint32_t o[8];                          // (the upper eight codes of the word are not there: zeros)
                unpack_word16<I2, F16T>(f.w[p].x, o);
                wv = make_uint4(o[0], o[1], o[2], o[3]);
            }
            if constexpr (F16T) {
                f16x8 a, b;
                __builtin_memcpy(&a, &f.a[p], 16);
                __builtin_memcpy(&b, &wv, 16);
                acc = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, acc, 0, 0, 0);
                if constexpr (HALVES == 2) {
                    __builtin_memcpy(&a, &f.al[p], 16);
                    accl = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, accl, 0, 0, 0);
                }
            } else {
                bf16x8 a, b;
                __builtin_memcpy(&a, &f.a[p], 16);
                __builtin_memcpy(&b, &wv, 16);
                acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, acc, 0, 0, 0);
            }
        }
    };
    uint32_t s = s0;
    for (; s + U <= s1; s += U) {
        Frag f[U];
#pragma unroll
        for (int u = 0; u < U; ++u) f[u] = ld(s + u);
#pragma unroll
        for (int u = 0; u < U; ++u) fma2(f[u]);
    }
    for (; s < s1; ++s) fma2(ld(s));
#pragma unroll
    for (int r = 0; r < 16; ++r)
        part[wave][(8 * (r >> 2) + 4 * h + (r & 3)) * 33 + q] = HALVES == 2 ? fmaf(accl[r], kLoScale, acc[r]) : acc[r];
    __syncthreads();
    // the waves' sums in wave order, scale, bias, activation; 512 threads, two outputs each
    const float wscale = g.L.wscale;
#pragma unroll
    for (int i = 0; i < 2; ++i) {
        const int e = t + 512 * i, row = e >> 5, col = e & 31;
        float v = 0.0f;
#pragma unroll
        for (int w = 0; w < NW; ++w) v += part[w][row * 33 + col];
        if (m0 + row >= M || n0 + col >= N) continue;
        v = apply_act(fmaf(v, wscale, elem_value_rt(g.L.bias_fmt, g.L.bias, n0 + col) * g.L.bscale), g.L.act);
        const size_t o = (size_t)(m0 + row) * N + n0 + col;
        if (g.out_f32) reinterpret_cast<float *>(g.C)[o] = v;
        else if constexpr (HALVES == 2) {
            uint16_t eh, el;
            split_f16(v, eh, el);
            reinterpret_cast<uint16_t *>(g.C)[o] = eh;
            reinterpret_cast<uint16_t *>(g.C)[(size_t)M * N + o] = el;
        } else reinterpret_cast<uint16_t *>(g.C)[o] = f32_to_t16<F16T>(v);
    }
}

template <int OFF>
__device__ __forceinline__ void ds_read128(u32x4 &dst, uint32_t addr);

// 16 bytes per lane from global memory straight into LDS (wave-contiguous 1 KiB at lds_addr):
// scalar base + 32-bit lane offset, so issuing it costs no vector-ALU instruction.  The compiler
// does not track these loads: the caller waits with s_waitcnt vmcnt before the data is read.
__device__ __forceinline__ void lds_dma16(uint32_t lds_addr, uint32_t voff, const void *sbase)
{
    // Both are uniform by construction; saying so keeps them in scalar registers where the compiler's own analysis
    // gives up (it folds the intrinsic away where it does not).
    lds_addr = (uint32_t)__builtin_amdgcn_readfirstlane((int)lds_addr);
    const uint64_t b = reinterpret_cast<uint64_t>(sbase);
    sbase = reinterpret_cast<const void *>(((uint64_t)(uint32_t)__builtin_amdgcn_readfirstlane((int)(b >> 32)) << 32) |
                                           (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)b));
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(lds_addr), "v"(voff), "s"(sbase) : "memory");
}

template <int OFF>
__device__ __forceinline__ void ds_read128(u32x4 &dst, uint32_t addr)
{
    asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(dst) : "v"(addr), "n"(OFF));
}

// reads CNT fragments 4 KiB apart (32 tile rows of 128 bytes) starting at addr + BASE
template <int BASE, int CNT, int I = 0>
__device__ __forceinline__ void frag_reads(u32x4 *dst, uint32_t addr)
{
    if constexpr (I < CNT) {
        ds_read128<BASE + I * 4096>(dst[I], addr);
        frag_reads<BASE, CNT, I + 1>(dst, addr);
    }
}

// ---------------------------------------------------------------------------
// Large-tile variant of the 16-bit MFMA GEMM (rows 16-byte aligned).  WM x WN waves,
// each TM x TN tiles of 32x32; BK = 64.  A K that is not a multiple of 64 leaves a
// partial K tile, which is processed first: its lanes past the end of a row fetch the
// row's element k0 instead (always inside the array) and overwrite what they fetched
// with zeros once it has landed.
//   * LDS rows hold 64 elements = eight 16-byte chunks, unpadded; chunk c of row
//     r sits at position c ^ ((r >> 1) & 7).  A 128-bit fragment read is served 16
//     lanes (16 consecutive rows, 256 bytes = all 64 banks) per cycle: rows of equal
//     parity share a 128-byte half, and r >> 1 gives those eight rows eight
//     different chunk positions.
//   * 16-bit operands (activations always, BF16/FP16 weights) go from global
//     memory straight into LDS (global_load_lds_dwordx4: each wave fills 1 KiB =
//     8 tile rows per instruction); which global chunk a lane fetches carries the
//     swizzle.  Integer weights pass through registers to be unpacked.
//   * two LDS stages: tile kt+1 is in flight while tile kt feeds the MFMAs; one
//     barrier per K tile.
template <int FMT, bool F16T, int WM, int WN, int TM, int TN>
__global__ __launch_bounds__(64 * WM * WN) void sp_gemm16_big(const GemmArgs g)
{
    constexpr int NT = 64 * WM * WN, NWAVES = WM * WN;
    constexpr int BM = WM * TM * 32, BN = WN * TN * 32, BK = 64;
    constexpr int bits = fmt_bits(FMT);
    constexpr bool W_DIRECT = (FMT == BF16 || FMT == F16);
    constexpr int A_ISSUES = BM * 8 / NT;               // 16-byte chunks per thread and tile
    constexpr int W_ISSUES = BN * 8 / NT;
    constexpr int EPL = 128 / bits;                     // weight elements per 16-byte global load
    constexpr int CPL = EPL / 8;                        // LDS chunks produced per global load
    constexpr int W_LOADS = W_DIRECT ? 1 : (BN * BK / EPL + NT - 1) / NT;

    extern __shared__ __attribute__((aligned(16))) uint16_t smem[];
    uint16_t *As = smem;                                // [2][BM][64]
    uint16_t *Ws = smem + 2 * BM * BK;                  // [2][BN][64]

    const uint32_t M = g.M, N = g.L.N, K = g.L.K;
    const int t = threadIdx.x, lane = t & 63, wave = t >> 6;
    const int wm = wave / WN, wn = wave % WN;

    // Tile order: each XCD (workgroup id mod 8) gets a contiguous run of tiles; inside the run, 8 row tiles x 4
    // column tiles are consecutive so that the 32 workgroups an XCD runs at once share A rows and W rows in its L2.
    // (A workgroup that walks over several tiles instead, one workgroup per compute unit, was measured: no faster,
    // and the longer live ranges cost the integer formats register spills.)
    const uint32_t tiles_n = (N + BN - 1) / BN, tiles_m = (M + BM - 1) / BM;
    const uint32_t ntiles = tiles_m * tiles_n;
    uint32_t m0 = 0, n0 = 0;
    auto place = [&](uint32_t bid) {
        const uint32_t per = ntiles / 8u;
        if (bid < per * 8u) bid = (bid & 7u) * per + (bid >> 3);
        constexpr uint32_t GM = 8;
        const uint32_t group = bid / (GM * tiles_n);
        const uint32_t first = group * GM;
        const uint32_t rows = tiles_m - first < GM ? tiles_m - first : GM;
        const uint32_t in = bid - group * GM * tiles_n;
        m0 = (first + in % rows) * BM;
        n0 = (in / rows) * BN;
    };

    f32x16 acc[TM][TN];

    // LDS-DMA sources: a uniform base (advanced per K tile on the scalar unit) plus a fixed 32-bit
    // byte offset per lane and issue, and LDS destinations derived from a scalar wave index: the main
    // loop then issues its loads without any vector-ALU instruction, which would otherwise queue
    // behind the other wave's MFMAs
    const int wave_s = __builtin_amdgcn_readfirstlane(wave);
    // Only the first wave of each SIMD (waves 0 .. NWAVES/2-1, which the issue arbiter serves first)
    // issues the loads, for itself and for wave + NWAVES/2: a wave stalls while the address unit takes
    // its load, and the other wave of the SIMD keeps the MFMA pipe fed meanwhile.
    // (four-wave workgroups have one wave per SIMD: every wave loads its own share)
    constexpr int HALF = NWAVES > 4 ? NWAVES / 2 : NWAVES;      // loader waves
    constexpr int PER = NWAVES / HALF;                            // shares a loader wave issues
    constexpr int A_DUTY = PER * A_ISSUES, W_DUTY = W_DIRECT ? PER * W_ISSUES : 1;
    uint32_t a_voff[A_DUTY], w_voff[W_DUTY];
    auto lane_offsets = [&]() {
#pragma unroll
        for (int d = 0; d < A_DUTY; ++d) {
            const int i = d / PER, wv = (wave & (HALF - 1)) + (d % PER) * HALF;
            const int ci = (i * NWAVES + wv) * 64 + lane, row = ci >> 3, pos = ci & 7;
            const uint32_t m = m0 + row < M ? m0 + row : M - 1;
            a_voff[d] = (uint32_t)(((size_t)m * K + ((pos ^ ((row >> 1) & 7)) << 3)) * 2u);
        }
        if constexpr (W_DIRECT) {
#pragma unroll
            for (int d = 0; d < W_DUTY; ++d) {
                const int i = d / PER, wv = (wave & (HALF - 1)) + (d % PER) * HALF;
                const int ci = (i * NWAVES + wv) * 64 + lane, row = ci >> 3, pos = ci & 7;
                const uint32_t n = n0 + row < N ? n0 + row : N - 1;
                w_voff[d] = (uint32_t)(((size_t)n * K + ((pos ^ ((row >> 1) & 7)) << 3)) * 2u);
            }
        }
    };
    // which 8 elements of a 64-element tile row this lane fetches: the same for every load it issues, because
    // the rows of two of its loads are a multiple of 16 apart
    static_assert(NWAVES % 2 == 0 && HALF % 2 == 0, "the swizzle of a lane's loads must not depend on the load");
    const uint32_t kchunk = (uint32_t)((lane & 7) ^ ((((wave & (HALF - 1)) * 8 + (lane >> 3)) >> 1) & 7)) << 3;
    const char *a_base = reinterpret_cast<const char *>(g.A + (size_t)(blockIdx.y / g.ksplits) * g.M * g.L.K);
    const char *w_base = reinterpret_cast<const char *>(g.L.w);
    const size_t w_row_bytes = (size_t)K * bits / 8u;
    uint4 rw[W_LOADS];
    const uint32_t lds_a = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) uint16_t *)As + (uint32_t)(wave_s & (HALF - 1)) * 1024u;
    const uint32_t lds_w = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) uint16_t *)Ws + (uint32_t)(wave_s & (HALF - 1)) * 1024u;
    const bool loader = wave_s < HALF;
    // the idx-th load instruction of a loader wave's tile (A first, then W); idx is a constant once
    // the caller's loops are unrolled
    constexpr int DMA_TOTAL = A_DUTY + (W_DIRECT ? W_DUTY : 0);
    auto issue_one = [&](int buf, uint32_t k0, int idx) {
        if (!loader) return;
#pragma unroll
        for (int d = 0; d < A_DUTY; ++d)
            if (d == idx)
                lds_dma16(lds_a + (uint32_t)(buf * BM * BK * 2 + ((d / PER) * NWAVES + (d % PER) * HALF) * 1024), a_voff[d],
                          a_base + (size_t)k0 * 2u);
        if constexpr (W_DIRECT) {
#pragma unroll
            for (int d = 0; d < W_DUTY; ++d)
                if (A_DUTY + d == idx)
                    lds_dma16(lds_w + (uint32_t)(buf * BN * BK * 2 + ((d / PER) * NWAVES + (d % PER) * HALF) * 1024), w_voff[d],
                              w_base + (size_t)k0 * 2u);
        }
    };
    auto issue_direct = [&](int buf, uint32_t k0) {            // the whole tile at once (prologue)
#pragma unroll
        for (int idx = 0; idx < DMA_TOTAL; ++idx) issue_one(buf, k0, idx);
    };
    auto load_w_regs = [&](uint32_t k0) {
        if constexpr (!W_DIRECT) {
            constexpr int LPR = BK / EPL;
#pragma unroll
            for (int i = 0; i < W_LOADS; ++i) {
                const int c = t + NT * i, row = c / LPR, kc = c % LPR;
                const uint32_t n = n0 + row < N ? n0 + row : N - 1;
                if (row < BN)
                    rw[i] = *reinterpret_cast<const uint4 *>(g.L.w + (size_t)n * w_row_bytes + (size_t)(k0 + kc * EPL) * bits / 8u);
            }
        }
    };
    // The partial K tile at k0 (prologue only).  Rows are whole 16-byte units, so a 16-byte piece lies entirely
    // inside a row or entirely past its end; code 0 decodes to 0.
    auto load_w_regs_tail = [&](uint32_t k0) {
        if constexpr (!W_DIRECT) {
            constexpr int LPR = BK / EPL;
#pragma unroll
            for (int i = 0; i < W_LOADS; ++i) {
                const int c = t + NT * i, row = c / LPR, kc = c % LPR;
                const uint32_t n = n0 + row < N ? n0 + row : N - 1;
                if (row >= BN) continue;
                if (k0 + kc * EPL < K)
                    rw[i] = *reinterpret_cast<const uint4 *>(g.L.w + (size_t)n * w_row_bytes + (size_t)(k0 + kc * EPL) * bits / 8u);
                else
                    rw[i] = make_uint4(0u, 0u, 0u, 0u);
            }
        }
    };
    auto issue_tail = [&](uint32_t k0) {                       // into stage 0
        if (!loader) return;
        const uint32_t back = k0 + kchunk < K ? 0u : kchunk * 2u;
#pragma unroll
        for (int d = 0; d < A_DUTY; ++d)
            lds_dma16(lds_a + (uint32_t)(((d / PER) * NWAVES + (d % PER) * HALF) * 1024), a_voff[d] - back, a_base + (size_t)k0 * 2u);
        if constexpr (W_DIRECT) {
#pragma unroll
            for (int d = 0; d < W_DUTY; ++d)
                lds_dma16(lds_w + (uint32_t)(((d / PER) * NWAVES + (d % PER) * HALF) * 1024), w_voff[d] - back, w_base + (size_t)k0 * 2u);
        }
    };
    auto zero_tail = [&](uint32_t k0) {                        // after the loads of issue_tail have landed
        if (!loader || k0 + kchunk < K) return;
        const uint32_t mine = (uint32_t)(wave & (HALF - 1)) * 1024u + (uint32_t)lane * 16u;
#pragma unroll
        for (int d = 0; d < A_DUTY; ++d)
            *reinterpret_cast<uint4 *>(reinterpret_cast<char *>(As) + mine + ((d / PER) * NWAVES + (d % PER) * HALF) * 1024) =
                make_uint4(0u, 0u, 0u, 0u);
        if constexpr (W_DIRECT) {
#pragma unroll
            for (int d = 0; d < W_DUTY; ++d)
                *reinterpret_cast<uint4 *>(reinterpret_cast<char *>(Ws) + mine + ((d / PER) * NWAVES + (d % PER) * HALF) * 1024) =
                    make_uint4(0u, 0u, 0u, 0u);
        }
    };
    auto store_w_regs = [&](int buf) {
        if constexpr (!W_DIRECT) {
            constexpr int LPR = BK / EPL;
            constexpr int PW = 16 / bits;
#pragma unroll
            for (int i = 0; i < W_LOADS; ++i) {
                const int c = t + NT * i, row = c / LPR, kc = c % LPR;
                if (row >= BN) continue;
                const uint32_t w[4] = {rw[i].x, rw[i].y, rw[i].z, rw[i].w};
                uint32_t o[4 * PW];
#pragma unroll
                for (int q = 0; q < 4; ++q) unpack_word16<FMT, F16T>(w[q], o + q * PW);
                uint16_t *rowp = Ws + buf * BN * BK + row * BK;
#pragma unroll
                for (int v = 0; v < CPL; ++v) {
                    const int chunk = kc * CPL + v;
                    *reinterpret_cast<uint4 *>(rowp + ((chunk ^ ((row >> 1) & 7)) << 3)) =
                        make_uint4(o[4 * v], o[4 * v + 1], o[4 * v + 2], o[4 * v + 3]);
                }
            }
        }
    };

    // ---- main loop -----------------------------------------------------------
    // Fragment reads are issued as explicit ds_read_b128 with manual lgkmcnt waits:
    // the compiler would otherwise drain every pending LDS-DMA load before the first
    // LDS read of an iteration and serialise load and compute.  Reads of k-step s+1
    // are in flight while the MFMAs of k-step s run.
    const uint32_t lds0 = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) uint16_t *)smem;
    const int h = lane >> 5, l7 = (lane >> 1) & 7;
    uint32_t va[4], vw[4];
#pragma unroll
    for (int ks = 0; ks < 4; ++ks) {
        const uint32_t xo = (uint32_t)(((2 * ks + h) ^ l7) << 4);
        va[ks] = lds0 + (uint32_t)((wm * TM * 32 + (lane & 31)) * 128) + xo;
        vw[ks] = lds0 + (uint32_t)(2 * BM * BK * 2) + (uint32_t)((wn * TN * 32 + (lane & 31)) * 128) + xo;
    }
    u32x4 fa[2][TM], fb[2][TN];

    // A loader wave slips one load instruction behind each of the first MFMAs of k-steps 0..2: the
    // matrix pipe is busy for eight passes after every issue, and the address unit takes the load meanwhile.
    constexpr int DPS = (DMA_TOTAL + 2) / 3;              // load instructions per k-step
    auto stage = [&](auto cur_c, bool more, uint32_t knext) {
        constexpr int CUR = decltype(cur_c)::value;
        if (more) load_w_regs(knext);
        frag_reads<CUR * BM * BK * 2, TM>(fa[0], va[0]);
        frag_reads<CUR * BN * BK * 2, TN>(fb[0], vw[0]);
#pragma unroll
        for (int ks = 0; ks < 4; ++ks) {
            const int cs = ks & 1;
            if (ks < 3) {
                frag_reads<CUR * BM * BK * 2, TM>(fa[cs ^ 1], va[ks + 1]);
                frag_reads<CUR * BN * BK * 2, TN>(fb[cs ^ 1], vw[ks + 1]);
                asm volatile("s_waitcnt lgkmcnt(%0)" ::"n"(TM + TN));
            } else {
                asm volatile("s_waitcnt lgkmcnt(0)");
            }
#pragma unroll
            for (int i = 0; i < TM; ++i) asm volatile("" : "+v"(fa[cs][i]));
#pragma unroll
            for (int j = 0; j < TN; ++j) asm volatile("" : "+v"(fb[cs][j]));
            __builtin_amdgcn_sched_barrier(0);          // keep the MFMA group between its wait and the next reads
#pragma unroll
            for (int i = 0; i < TM; ++i)
#pragma unroll
                for (int j = 0; j < TN; ++j) {
                    if constexpr (F16T) {
                        f16x8 a, b;
                        __builtin_memcpy(&a, &fa[cs][i], 16);
                        __builtin_memcpy(&b, &fb[cs][j], 16);
                        acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, acc[i][j], 0, 0, 0);
                    } else {
                        bf16x8 a, b;
                        __builtin_memcpy(&a, &fa[cs][i], 16);
                        __builtin_memcpy(&b, &fb[cs][j], 16);
                        acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, acc[i][j], 0, 0, 0);
                    }
                    if (more && ks < 3 && i * TN + j < DPS) {
                        __builtin_amdgcn_sched_barrier(0);
                        issue_one(CUR ^ 1, knext, ks * DPS + i * TN + j);
                        __builtin_amdgcn_sched_barrier(0);
                    }
                }
            __builtin_amdgcn_sched_barrier(0);
        }
        if (more) store_w_regs(CUR ^ 1);
        asm volatile("s_waitcnt vmcnt(0)");         // this wave's share of the next stage has landed
        __syncthreads();                             // ... and everybody's; the current stage is free again
    };

    // grid y splits K for problems with too few tiles to fill the chip
    const uint32_t kbeg = g.kper ? (blockIdx.y % g.ksplits) * g.kper : 0u;
    const uint32_t kend = g.kper && kbeg + g.kper < K ? kbeg + g.kper : K;
    const uint32_t ktiles = (kend - kbeg + BK - 1) / BK;
    const uint32_t tail = (kend - kbeg) % BK;              // only the last K split can have one
    // tile 0 is the partial tile if there is one; tile s >= 1 then starts at kbeg + (s - 1) * BK
    const uint32_t kshift = tail ? (uint32_t)BK : 0u;
    place(blockIdx.x);
    lane_offsets();
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.0f;
    if (tail) {
        const uint32_t kt0 = kend - tail;
        issue_tail(kt0);
        load_w_regs_tail(kt0);
        store_w_regs(0);
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        zero_tail(kt0);
    } else {
        issue_direct(0, kbeg);
        load_w_regs(kbeg);
        store_w_regs(0);
        asm volatile("s_waitcnt vmcnt(0)");
    }
    __syncthreads();
    for (uint32_t kt = 0; kt < ktiles; kt += 2) {
        stage(std::integral_constant<int, 0>{}, kt + 1 < ktiles, kbeg + (kt + 1) * BK - kshift);
        if (kt + 1 < ktiles) stage(std::integral_constant<int, 1>{}, kt + 2 < ktiles, kbeg + (kt + 2) * BK - kshift);
    }
    // partial sums of a K split whose rows are not whole 16-byte units: one element per lane and store
    if (g.ws && (N % 4u != 0 || (reinterpret_cast<uintptr_t>(g.ws) & 15u) != 0)) {
#pragma unroll
        for (int j = 0; j < TN; ++j) {
            const uint32_t col = n0 + (wn * TN + j) * 32 + (lane & 31);
            if (col >= N) continue;
#pragma unroll
            for (int i = 0; i < TM; ++i)
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    const uint32_t row = m0 + (wm * TM + i) * 32 + 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3);
                    if (row < M) g.ws[((size_t)blockIdx.y * M + row) * N + col] = acc[i][j][r];
                }
        }
        return;
    }
    const float wscale = g.L.wscale;
    // Output rows that are whole 16-byte units: a wave turns its 32 x (32 TN) block of each row tile around in LDS
    // (the stages are free after the loop's last barrier; every wave has a region of its own, so no barrier is
    // needed) and writes whole rows of the block, 16 bytes per lane, instead of one element per lane.
    // The partial sums of a K split go the same way into the workspace, unscaled, as FP32.
    const uint32_t esz = g.out_f32 ? 4u : 2u;
    if (g.ws || (((size_t)N * esz) % 16u == 0 && (reinterpret_cast<uintptr_t>(g.C) & 15u) == 0)) {
        constexpr int BW = 32 * TN;                                  // columns of a wave's block
        float bias[TN];
#pragma unroll
        for (int j = 0; j < TN; ++j) {
            const uint32_t col = n0 + (wn * TN + j) * 32 + (lane & 31);
            bias[j] = (col < N && !g.ws) ? elem_value_rt(g.L.bias_fmt, g.L.bias, col) * g.L.bscale : 0.0f;
        }
        char *const out = g.ws ? reinterpret_cast<char *>(g.ws + (size_t)blockIdx.y * M * N) : reinterpret_cast<char *>(g.C);
        // Sigmoid and tanh are kept out of the common path: a run-time switch over all activations inside the
        // unrolled loops puts a copy of their code behind each of a lane's 16 TM TN outputs, and fetching that code
        // took longer than the stores (a tenth of an 8192-cubed launch).  The lambda is forced inline: called, it
        // would take the accumulators through memory.
        // Long K: the outputs bypass the caches' usual retention (they would displace the A and W panels the other
        // tiles of the die are re-reading: 8192 cubed 0.908 against 0.934 ms); short K: the next layer reads them
        // back soon and they are most of the traffic (8192 x 8192 x 1024: 0.162 against 0.175 ms the other way round).
        const bool stream_out = K >= 2048u && !g.ws;
        auto turn = [&](auto es_c, auto mode_c) __attribute__((always_inline)) {
            constexpr int ES = decltype(es_c)::value;
            constexpr int MODE = decltype(mode_c)::value;            // 0: cheap activations, 1: sigmoid / tanh, 2: partial sums
            constexpr int PITCH = BW * ES + 16;                      // lanes 0-31 and 32-63 (four rows apart) on different banks
            constexpr int LPR = BW * ES / 16;                        // lanes that write one row
            constexpr int RPP = 64 / LPR;                            // rows per store instruction
            char *mine = reinterpret_cast<char *>(smem) + wave * (32 * PITCH);
#pragma unroll
            for (int i = 0; i < TM; ++i) {
#pragma unroll
                for (int j = 0; j < TN; ++j)
#pragma unroll
                    for (int r = 0; r < 16; ++r) {
                        const int rl = 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3);
                        const float pre = MODE == 2 ? acc[i][j][r] : fmaf(acc[i][j][r], wscale, bias[j]);
                        const float v = MODE == 2 ? pre : MODE == 1 ? apply_act(pre, g.L.act) : apply_act_cheap(pre, g.L.act);
                        char *dst = mine + rl * PITCH + (j * 32 + (lane & 31)) * ES;
                        if constexpr (ES == 4) *reinterpret_cast<float *>(dst) = v;
                        else *reinterpret_cast<uint16_t *>(dst) = f32_to_t16<F16T>(v);
                    }
#pragma unroll
                for (int p = 0; p < 32 / RPP; ++p) {
                    const int rl = p * RPP + lane / LPR, seg = lane % LPR;
                    const uint4 v = *reinterpret_cast<const uint4 *>(mine + rl * PITCH + seg * 16);
                    const uint32_t row = m0 + (wm * TM + i) * 32 + rl;
                    const uint32_t col = n0 + wn * BW + seg * (16 / ES);
                    if (row < M && col < N) {                        // N is a multiple of 16 / ES: a unit is all in or all out
                        u32x4 *dstp = reinterpret_cast<u32x4 *>(out + ((size_t)row * N + col) * ES);
                        const u32x4 vv{v.x, v.y, v.z, v.w};
                        if (stream_out) __builtin_nontemporal_store(vv, dstp);
                        else *dstp = vv;
                    }
                }
            }
        };
        const bool slow = g.L.act == A_SIGMOID || g.L.act == A_TANH;
        using E4 = std::integral_constant<int, 4>;
        using E2 = std::integral_constant<int, 2>;
        if (g.ws) {
            turn(E4{}, std::integral_constant<int, 2>{});
        } else if (g.out_f32) {
            if (slow) turn(E4{}, std::integral_constant<int, 1>{});
            else turn(E4{}, std::integral_constant<int, 0>{});
        } else {
            if (slow) turn(E2{}, std::integral_constant<int, 1>{});
            else turn(E2{}, std::integral_constant<int, 0>{});
        }
        return;
    }
#pragma unroll
    for (int j = 0; j < TN; ++j) {
        const uint32_t col = n0 + (wn * TN + j) * 32 + (lane & 31);
        if (col >= N) continue;
        const float bias = elem_value_rt(g.L.bias_fmt, g.L.bias, col) * g.L.bscale;
#pragma unroll
        for (int i = 0; i < TM; ++i) {
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const uint32_t row = m0 + (wm * TM + i) * 32 + 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3);
                if (row >= M) continue;
                const float v = apply_act(fmaf(acc[i][j][r], wscale, bias), g.L.act);
                const size_t o = (size_t)row * N + col;
                if (g.out_f32) reinterpret_cast<float *>(g.C)[o] = v;
                else reinterpret_cast<uint16_t *>(g.C)[o] = f32_to_t16<F16T>(v);
            }
        }
    }
}

// adds the partial sums of a split launch (K splits in split order; with split activations the sums of the second
// matrix, scaled by 2^-11, after those of the first) and applies scale, bias and activation; a thread takes four
// neighbouring columns (VEC: N a multiple of four, workspace and C 16-byte aligned) or one.  16-bit outputs of a
// split-activation forward are written as the two matrices of the next layer's input (g.halves == 2).
template <bool F16T, bool VEC>
__global__ __launch_bounds__(256) void sp_gemm16_reduce(const GemmArgs g, uint32_t splits)
{
    const uint64_t total = (uint64_t)g.M * g.L.N;
    const uint32_t parts = splits * g.halves;
    if constexpr (VEC) {
        const uint64_t idx = ((uint64_t)blockIdx.x * 256u + threadIdx.x) * 4u;
        if (idx >= total) return;
        float4 sum = make_float4(0.0f, 0.0f, 0.0f, 0.0f), low = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
        for (uint32_t sp = 0; sp < parts; ++sp) {
            const float4 v = *reinterpret_cast<const float4 *>(g.ws + (uint64_t)sp * total + idx);
            if (sp < splits) { sum.x += v.x; sum.y += v.y; sum.z += v.z; sum.w += v.w; }
            else { low.x += v.x; low.y += v.y; low.z += v.z; low.w += v.w; }
        }
        const uint32_t col = (uint32_t)(idx % g.L.N);
        const float in[4] = {fmaf(low.x, kLoScale, sum.x), fmaf(low.y, kLoScale, sum.y), fmaf(low.z, kLoScale, sum.z),
                             fmaf(low.w, kLoScale, sum.w)};
        float v[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const float bias = elem_value_rt(g.L.bias_fmt, g.L.bias, col + i) * g.L.bscale;
            v[i] = apply_act(fmaf(in[i], g.L.wscale, bias), g.L.act);
        }
        if (g.out_f32) {
            *reinterpret_cast<float4 *>(reinterpret_cast<float *>(g.C) + idx) = make_float4(v[0], v[1], v[2], v[3]);
        } else if (g.halves == 2) {
            uint16_t hi[4], lo[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) split_f16(v[i], hi[i], lo[i]);
            uint16_t *c = reinterpret_cast<uint16_t *>(g.C);
            *reinterpret_cast<uint2 *>(c + idx) = make_uint2((uint32_t)hi[0] | ((uint32_t)hi[1] << 16), (uint32_t)hi[2] | ((uint32_t)hi[3] << 16));
            *reinterpret_cast<uint2 *>(c + total + idx) = make_uint2((uint32_t)lo[0] | ((uint32_t)lo[1] << 16), (uint32_t)lo[2] | ((uint32_t)lo[3] << 16));
        } else {
            const uint32_t lo = (uint32_t)f32_to_t16<F16T>(v[0]) | ((uint32_t)f32_to_t16<F16T>(v[1]) << 16);
            const uint32_t hi = (uint32_t)f32_to_t16<F16T>(v[2]) | ((uint32_t)f32_to_t16<F16T>(v[3]) << 16);
            *reinterpret_cast<uint2 *>(reinterpret_cast<uint16_t *>(g.C) + idx) = make_uint2(lo, hi);
        }
    } else {
        const uint64_t idx = (uint64_t)blockIdx.x * 256u + threadIdx.x;
        if (idx >= total) return;
        float sum = 0.0f, low = 0.0f;
        for (uint32_t sp = 0; sp < parts; ++sp) {
            const float v = g.ws[(uint64_t)sp * total + idx];
            if (sp < splits) sum += v; else low += v;
        }
        const uint32_t col = (uint32_t)(idx % g.L.N);
        const float bias = elem_value_rt(g.L.bias_fmt, g.L.bias, col) * g.L.bscale;
        const float v = apply_act(fmaf(fmaf(low, kLoScale, sum), g.L.wscale, bias), g.L.act);
        if (g.out_f32) reinterpret_cast<float *>(g.C)[idx] = v;
        else if (g.halves == 2) {
            uint16_t hi, lo;
            split_f16(v, hi, lo);
            reinterpret_cast<uint16_t *>(g.C)[idx] = hi;
            reinterpret_cast<uint16_t *>(g.C)[total + idx] = lo;
        } else reinterpret_cast<uint16_t *>(g.C)[idx] = f32_to_t16<F16T>(v);
    }
}
