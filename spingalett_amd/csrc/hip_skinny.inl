// hip_skinny.inl — the streaming MFMA kernels for layers with one thin side (sp_skinny16,
// sp_skinny16_kw, sp_skinny_reduce, sp_codes16).  Part of hip_forward.hip's translation unit (included
// there, inside its unnamed namespace); not compiled on its own.

// ---------------------------------------------------------------------------
// Streaming MFMA kernel for layers with one thin side
// ---------------------------------------------------------------------------
// Few samples (5 .. 256) or few outputs (<= 64): one operand is a tall matrix that is
// read exactly once (the weights, or the 16-bit activations when the layer has few
// outputs), the other a thin 16-bit matrix of at most 64 rows per workgroup.  The tall
// operand never touches LDS: a workgroup has NWV waves (4 or 8), a wave owns RT tiles of 32 streamed rows and loads them
// straight into registers, 16 bytes per lane, one chunk ahead; lanes 0-31 and 32-63 take
// adjacent 16-byte pieces of a row.  The integer codes become FP16 pairs with the
// 0x6400 | code trick (1024 + code, minus the constant, exact), which delivers the codes
// of a step in a format-specific order; the thin operand is written to LDS in that same
// order, so both MFMA operands agree on which k sits where.
// Workgroups split K (grid y) to fill the chip; partial tiles go to a workspace and a
// second launch adds them, otherwise the epilogue is applied here.
struct SkinnyArgs {
    LayerArgs L;
    const uint8_t *stream;   // streamed rows, K codes each
    const uint16_t *thin;    // [NC][K] 16-bit
    void *C;                 // [M][N]
    float *ws;               // [S][NC][R] partial sums when the grid splits K
    uint32_t R, NC;          // streamed rows, thin rows
    uint32_t row_blocks, cblocks;   // workgroups along the streamed rows / blocks of thin rows (grid x covers both)
    uint32_t kper;           // codes per K split (whole chunks)
    int out_f32;
    int mode_b;              // 0: streamed rows are outputs, thin rows samples; 1: the reverse
    void *soft_out;          // sp_skinny16_kw, mode_b, no K split: softmax over a sample's outputs goes here instead of C
    int soft_kind;           // its element type: 0 FP32, 1 BF16, 2 FP16
    // Split activations (GemmArgs has the layout): grid y = halves x ksplits, y / ksplits picks the activation matrix
    // (the thin operand, or the streamed one in mode b), y % ksplits the K range.
    uint32_t ksplits;        // K splits (>= 1)
    uint32_t halves;         // 1, or 2 with split activations
    uint64_t half_elems;     // elements between the two activation matrices (samples x K)
};

template <int FMT>
struct SkinnyFmt {
    static constexpr int bits = fmt_bits(FMT);
    static constexpr int EPL = 128 / bits;                                  // codes per 16-byte lane load
    static constexpr int LPC = (FMT == I2) ? 2 : 4;                         // lane loads per chunk and tile
    static constexpr int BKC = 2 * LPC * EPL;                               // codes per chunk: 64 (16-bit), 128, 256, 256
    static constexpr int STEPS = EPL / 8;                                   // MFMA k-steps per lane load
    static constexpr int PITCH = BKC * 2 + 16;                              // LDS row pitch: 16 rows hit 16 different slots
};

// position p of a 16-code group holds code skinny_perm(p) of the group
template <int FMT>
__host__ __device__ constexpr int skinny_perm(int p)
{
    if (FMT == I8) { constexpr int t[8] = {0, 2, 1, 3, 4, 6, 5, 7}; return t[p & 7] + (p & 8); }
    if (FMT == I4) { constexpr int t[8] = {0, 4, 1, 5, 2, 6, 3, 7}; return t[p & 7] + (p & 8); }
    if (FMT == I2) { constexpr int t[16] = {0, 8, 1, 9, 2, 10, 3, 11, 4, 12, 5, 13, 6, 14, 7, 15}; return t[p]; }
    return p;
}

// the 16 codes of a unit of the thin operand (eight 16-bit pairs) in the order skinny_perm gives
template <int FMT>
__device__ __forceinline__ void skinny_permute_unit(const uint32_t (&in)[8], uint32_t (&o)[8])
{
#pragma unroll
    for (int w = 0; w < 8; ++w) {
        const int ea = skinny_perm<FMT>(2 * w), eb = skinny_perm<FMT>(2 * w + 1);
        const uint32_t sel = (uint32_t)(2 * (ea & 1)) | ((uint32_t)(2 * (ea & 1) + 1) << 8) |
                             ((uint32_t)(4 + 2 * (eb & 1)) << 16) | ((uint32_t)(4 + 2 * (eb & 1) + 1) << 24);
        o[w] = __builtin_amdgcn_perm(in[eb >> 1], in[ea >> 1], sel);
    }
}

typedef _Float16 h16x2 __attribute__((ext_vector_type(2)));

__device__ __forceinline__ uint32_t magic_sub(uint32_t v, uint32_t c)
{
    h16x2 a, b;
    __builtin_memcpy(&a, &v, 4);
    __builtin_memcpy(&b, &c, 4);
    a = a - b;
    uint32_t r;
    __builtin_memcpy(&r, &a, 4);
    return r;
}

// The 8 values of k-step j of one lane load, as four FP16 pairs.  A field of the word is
// masked in place and XORed onto an FP16 constant whose last mantissa bit has the weight of
// the field's lowest bit (1024 for bit 0, 256 for bit 2, 64 for bit 4, ...), the same XOR flips
// the field's sign bit (two's complement -> offset binary); subtracting the constant plus the
// offset leaves the code, exactly.  Only fields above the 10 mantissa bits need a shift first.
template <int FMT>
__device__ __forceinline__ void skinny_frag(const uint4 &v, int j, uint32_t (&f)[4])
{
    const uint32_t w[4] = {v.x, v.y, v.z, v.w};
    if constexpr (FMT == I8) {
        // word = codes b0 b1 b2 b3: pairs (b0, b2) and (b1, b3)
#pragma unroll
        for (int q = 0; q < 2; ++q) {
            const uint32_t x = w[2 * j + q];
            f[2 * q]     = magic_sub((x & 0x00FF00FFu) ^ 0x64806480u, 0x64806480u);          // 1024 + 128 + q
            f[2 * q + 1] = magic_sub(((x >> 8) & 0x00FF00FFu) ^ 0x64806480u, 0x64806480u);
        }
    } else if constexpr (FMT == I4) {
        // word = nibbles c0 .. c7: pairs (c0, c4), (c1, c5), (c2, c6), (c3, c7)
        const uint32_t x = w[j], y = x >> 8;
        f[0] = magic_sub((x & 0x000F000Fu) ^ 0x64086408u, 0x64086408u);                      // 1024 + 8 + q
        f[1] = magic_sub((x & 0x00F000F0u) ^ 0x54805480u, 0x54805480u);                      // 64 + 8 + q
        f[2] = magic_sub((y & 0x000F000Fu) ^ 0x64086408u, 0x64086408u);
        f[3] = magic_sub((y & 0x00F000F0u) ^ 0x54805480u, 0x54805480u);
    } else if constexpr (FMT == I2) {
        // word = fields c0 .. c15: step 0 pairs (c0, c8) .. (c3, c11), step 1 pairs (c4, c12) .. (c7, c15)
        const uint32_t x = w[j >> 1];
        if ((j & 1) == 0) {
            f[0] = magic_sub((x & 0x00030003u) ^ 0x64026402u, 0x64026402u);                  // 1024 + 2 + q
            f[1] = magic_sub((x & 0x000C000Cu) ^ 0x5C085C08u, 0x5C085C08u);                  // 256 + 2 + q
            f[2] = magic_sub((x & 0x00300030u) ^ 0x54205420u, 0x54205420u);                  // 64 + 2 + q
            f[3] = magic_sub((x & 0x00C000C0u) ^ 0x4C804C80u, 0x4C804C80u);                  // 16 + 2 + q
        } else {
            const uint32_t y = x >> 10;
            f[0] = magic_sub((x & 0x03000300u) ^ 0x46004600u, 0x46004600u);                  // 4 + 2 + q
            f[1] = magic_sub((y & 0x00030003u) ^ 0x64026402u, 0x64026402u);
            f[2] = magic_sub((y & 0x000C000Cu) ^ 0x5C085C08u, 0x5C085C08u);
            f[3] = magic_sub((y & 0x00300030u) ^ 0x54205420u, 0x54205420u);
        }
    } else {
        f[0] = w[0]; f[1] = w[1]; f[2] = w[2]; f[3] = w[3];
    }
}

// SLOW: the activation may be sigmoid or tanh.  Callers with many outputs per lane keep a copy of their loops for
// those two: a switch over all activations behind every output is mostly their code, fetched for nothing.
template <bool F16T, bool SLOW = true>
__device__ __forceinline__ void skinny_emit_biased(const SkinnyArgs &a, uint32_t c, uint32_t r, float accv, float bias)
{
    const uint32_t m = a.mode_b ? r : c, n = a.mode_b ? c : r;
    const float pre = fmaf(accv, a.L.wscale, bias);
    const float v = SLOW ? apply_act(pre, a.L.act) : apply_act_cheap(pre, a.L.act);
    const size_t o = (size_t)m * a.L.N + n;
    if (a.out_f32) reinterpret_cast<float *>(a.C)[o] = v;
    else reinterpret_cast<uint16_t *>(a.C)[o] = f32_to_t16<F16T>(v);
}

template <bool F16T>
__device__ __forceinline__ void skinny_emit(const SkinnyArgs &a, uint32_t c, uint32_t r, float accv)
{
    const float bias = elem_value_rt(a.L.bias_fmt, a.L.bias, a.mode_b ? c : r) * a.L.bscale;
    skinny_emit_biased<F16T>(a, c, r, accv, bias);
}

// 16 bytes per lane from scalar base + 32-bit lane offset + immediate.  Inline assembly: the compiler's
// wait-count bookkeeping does not see the load, the caller waits with s_waitcnt vmcnt before using dst.
template <int OFF>
__device__ __forceinline__ void load16_async(u32x4 &dst, uint32_t voff, const void *sbase)
{
    asm volatile("global_load_dwordx4 %0, %1, %2 offset:%3" : "=v"(dst) : "v"(voff), "s"(sbase), "n"(OFF) : "memory");
}

template <int FMT, bool F16T, int RT, int CT, int NWV>
__global__ __launch_bounds__(64 * NWV) void sp_skinny16(const SkinnyArgs a)
{
    using F = SkinnyFmt<FMT>;
    constexpr int EPL = F::EPL, LPC = F::LPC, BKC = F::BKC, STEPS = F::STEPS, PITCH = F::PITCH;
    constexpr int UNITS = 32 * CT * (BKC / 16);            // 16-code units of a thin chunk
    constexpr int NT = 64 * NWV;                           // threads of a workgroup
    constexpr int UPT = (UNITS + NT - 1) / NT;
    constexpr int STAGE = 32 * CT * PITCH;
    extern __shared__ __attribute__((aligned(16))) uint8_t sk_lds[];

    const int t = threadIdx.x, lane = t & 63, wave = t >> 6;
    const uint32_t n31 = lane & 31, h = lane >> 5;
    const uint32_t K = a.L.K;
    // Grid x enumerates (row block, thin block).  Consecutive workgroup ids go to consecutive dies (eight of them,
    // each with its own L2): the thin blocks of one row block get ids eight apart, so they run on the same die at
    // about the same time and the second and later ones find the streamed rows in its L2.
    uint32_t rblk = blockIdx.x, cblk = 0;
    if (a.cblocks > 1) {
        const uint32_t per = 8u * a.cblocks, group = blockIdx.x / per, rem = blockIdx.x % per;
        rblk = group * 8u + (rem & 7u);
        cblk = rem >> 3;
        if (rblk >= a.row_blocks) return;                 // padding of the last group
    }
    const uint32_t row0 = (rblk * (uint32_t)NWV + (uint32_t)wave) * (32u * RT);
    const uint32_t cbase = cblk * (32u * CT);
    const uint32_t half = blockIdx.y / a.ksplits;
    const uint8_t *const stream = a.mode_b ? a.stream + (size_t)half * a.half_elems * 2u : a.stream;
    const uint16_t *const thin = a.mode_b ? a.thin : a.thin + (size_t)half * a.half_elems;
    const uint32_t kbeg = (blockIdx.y % a.ksplits) * a.kper;
    const uint32_t kend = kbeg + a.kper < K ? kbeg + a.kper : K;
    const uint32_t nchunks = (kend - kbeg + BKC - 1) / BKC;
    const size_t row_bytes = (size_t)K * F::bits / 8u;

    // per-lane byte offsets (32-bit: the host checks that both operands span less than 4 GiB)
    uint32_t svoff[RT];
#pragma unroll
    for (int rt = 0; rt < RT; ++rt) {
        const uint32_t r = row0 + rt * 32u + n31;
        svoff[rt] = (uint32_t)((size_t)(r < a.R ? r : a.R - 1) * row_bytes) + h * 16u;
    }
    uint32_t tvoff[UPT][2];
    bool trow_ok[UPT];
#pragma unroll
    for (int q = 0; q < UPT; ++q) {
        const uint32_t u = (uint32_t)t + (uint32_t)NT * q;
        const uint32_t row = u / (BKC / 16), uc = u % (BKC / 16);
        const uint32_t c = cbase + row;
        trow_ok[q] = u < (uint32_t)UNITS && c < a.NC;
#pragma unroll
        for (int e = 0; e < 2; ++e) tvoff[q][e] = trow_ok[q] ? (uint32_t)(((size_t)c * K + uc * 16u + 8u * e) * 2u) : 0u;
    }

    f32x16 acc[RT][CT];
#pragma unroll
    for (int rt = 0; rt < RT; ++rt)
#pragma unroll
        for (int ct = 0; ct < CT; ++ct)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[rt][ct][r] = 0.0f;

    // Loads are issued two chunks ahead for the streamed rows and one ahead for the thin block.  A chunk past
    // the end is clamped to the last one (a redundant load) so that the number of loads in flight is always the
    // same.  In the last chunk a lane load that would start past the end of its row reads the row's start
    // instead; what it fetched is masked (16-bit values) or meets zeros of the thin operand (integer codes).
    constexpr int S_LOADS = RT * LPC, T_LOADS = UPT * 2;
    const uint32_t last_chunk = nchunks - 1;
    auto issue_stream = [&](uint32_t ch, u32x4 (&dst)[RT][LPC]) {
        if (ch < last_chunk) {
            const uint8_t *sb = stream + (size_t)(kbeg + ch * BKC) * F::bits / 8u;
#pragma unroll
            for (int i = 0; i < LPC; ++i)
#pragma unroll
                for (int rt = 0; rt < RT; ++rt) {
                    if (i == 0) load16_async<0>(dst[rt][i], svoff[rt], sb);
                    else if (i == 1) load16_async<32>(dst[rt][i], svoff[rt], sb);
                    else if (i == 2) load16_async<64>(dst[rt][i], svoff[rt], sb);
                    else load16_async<96>(dst[rt][i], svoff[rt], sb);
                }
        } else {
            const uint32_t kc0 = kbeg + last_chunk * BKC;
#pragma unroll
            for (int i = 0; i < LPC; ++i) {
                const uint32_t k = kc0 + 2u * i * EPL;                 // first code of the h = 0 lane load
                const uint32_t add = k + h * EPL < K ? k * F::bits / 8u : 0u - h * 16u;
#pragma unroll
                for (int rt = 0; rt < RT; ++rt) load16_async<0>(dst[rt][i], svoff[rt] + add, stream);
            }
        }
    };
    u32x4 thin_regs[UPT][2];
    auto issue_thin = [&](uint32_t ch) {
        if (ch < last_chunk) {
            const uint16_t *tb = thin + (kbeg + ch * BKC);
#pragma unroll
            for (int q = 0; q < UPT; ++q)
#pragma unroll
                for (int e = 0; e < 2; ++e) load16_async<0>(thin_regs[q][e], tvoff[q][e], tb);
        } else {
            const uint32_t kc0 = kbeg + last_chunk * BKC;
#pragma unroll
            for (int q = 0; q < UPT; ++q) {
                const uint32_t uc = ((uint32_t)t + (uint32_t)NT * q) % (BKC / 16);
#pragma unroll
                for (int e = 0; e < 2; ++e) {
                    const bool valid = trow_ok[q] && kc0 + uc * 16u + 8u * e + 8u <= kend;
                    load16_async<0>(thin_regs[q][e], valid ? tvoff[q][e] + kc0 * 2u : 0u, thin);
                }
            }
        }
    };
    // ties the registers to the preceding wait: nothing that reads them is scheduled above it
    auto pin_stream = [&](u32x4 (&r)[RT][LPC]) {
#pragma unroll
        for (int rt = 0; rt < RT; ++rt)
#pragma unroll
            for (int i = 0; i < LPC; ++i) asm volatile("" : "+v"(r[rt][i]));
    };
    auto pin_thin = [&]() {
#pragma unroll
        for (int q = 0; q < UPT; ++q)
#pragma unroll
            for (int e = 0; e < 2; ++e) asm volatile("" : "+v"(thin_regs[q][e]));
    };
    auto store_thin = [&](int stage, uint32_t ch) {
        const uint32_t kc0 = kbeg + (ch < last_chunk ? ch : last_chunk) * BKC;
#pragma unroll
        for (int q = 0; q < UPT; ++q) {
            const uint32_t u = (uint32_t)t + (uint32_t)NT * q;
            if (u >= (uint32_t)UNITS) continue;
            const uint32_t row = u / (BKC / 16), uc = u % (BKC / 16);
            const uint32_t k = kc0 + uc * 16u;
            const uint32_t keep0 = (trow_ok[q] && k + 8u <= kend) ? 0xFFFFFFFFu : 0u;
            const uint32_t keep1 = (trow_ok[q] && k + 16u <= kend) ? 0xFFFFFFFFu : 0u;
            const uint32_t in[8] = {thin_regs[q][0].x & keep0, thin_regs[q][0].y & keep0, thin_regs[q][0].z & keep0,
                                    thin_regs[q][0].w & keep0, thin_regs[q][1].x & keep1, thin_regs[q][1].y & keep1,
                                    thin_regs[q][1].z & keep1, thin_regs[q][1].w & keep1};
            uint32_t o[8];
            skinny_permute_unit<FMT>(in, o);
            uint8_t *dst = sk_lds + stage * STAGE + row * PITCH + uc * 32u;
            *reinterpret_cast<uint4 *>(dst) = make_uint4(o[0], o[1], o[2], o[3]);
            *reinterpret_cast<uint4 *>(dst + 16) = make_uint4(o[4], o[5], o[6], o[7]);
        }
    };

    auto compute = [&](int stage, uint32_t ch, const u32x4 (&cur)[RT][LPC]) {
        const uint8_t *sbase = sk_lds + stage * STAGE + n31 * PITCH + h * (EPL * 2);
        const uint32_t kc0 = kbeg + ch * BKC;
#pragma unroll
        for (int i = 0; i < LPC; ++i) {
            // 16-bit values past the end of the row could be NaN or infinite: masked (integer codes need not be)
            const uint32_t keep = (F::bits == 16 && kc0 + (2u * i + h) * EPL >= K) ? 0u : 0xFFFFFFFFu;
#pragma unroll
            for (int j = 0; j < STEPS; ++j) {
                const int koff = (2 * i * EPL + 8 * j) * 2;
                uint4 tf[CT];
#pragma unroll
                for (int ct = 0; ct < CT; ++ct) tf[ct] = *reinterpret_cast<const uint4 *>(sbase + ct * 32 * PITCH + koff);
#pragma unroll
                for (int rt = 0; rt < RT; ++rt) {
                    uint4 v = make_uint4(cur[rt][i].x, cur[rt][i].y, cur[rt][i].z, cur[rt][i].w);
                    if constexpr (F::bits == 16) { v.x &= keep; v.y &= keep; v.z &= keep; v.w &= keep; }
                    uint32_t sf[4];
                    skinny_frag<FMT>(v, j, sf);
#pragma unroll
                    for (int ct = 0; ct < CT; ++ct) {
                        if constexpr (F16T) {
                            f16x8 af, bf;
                            __builtin_memcpy(&af, &tf[ct], 16);
                            __builtin_memcpy(&bf, sf, 16);
                            acc[rt][ct] = __builtin_amdgcn_mfma_f32_32x32x16_f16(af, bf, acc[rt][ct], 0, 0, 0);
                        } else {
                            bf16x8 af, bf;
                            __builtin_memcpy(&af, &tf[ct], 16);
                            __builtin_memcpy(&bf, sf, 16);
                            acc[rt][ct] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(af, bf, acc[rt][ct], 0, 0, 0);
                        }
                    }
                }
            }
        }
    };
    // One chunk.  In flight on entry: streamed chunks ch (in `cur`) and ch + 1; issued here: the thin block of
    // ch + 1, then streamed chunk ch + 2 into `far`.  Loads complete in order, so waiting until only the S_LOADS
    // youngest are outstanding means the thin block (and everything older) has arrived.
    auto step = [&](uint32_t ch, u32x4 (&cur)[RT][LPC], u32x4 (&far)[RT][LPC]) {
        const int stage = (int)(ch & 1u);
        issue_thin(ch + 1);
        issue_stream(ch + 2, far);
        asm volatile("s_waitcnt vmcnt(%0)" ::"n"(2 * S_LOADS + T_LOADS) : "memory");    // chunk ch is here
        pin_stream(cur);
        compute(stage, ch, cur);
        asm volatile("s_waitcnt vmcnt(%0)" ::"n"(S_LOADS) : "memory");
        pin_thin();
        store_thin(stage ^ 1, ch + 1);
        __syncthreads();
    };

    u32x4 ra[RT][LPC], rb[RT][LPC], rc[RT][LPC];
    issue_thin(0);
    issue_stream(0, ra);
    issue_stream(1, rb);
    asm volatile("s_waitcnt vmcnt(%0)" ::"n"(2 * S_LOADS) : "memory");
    pin_thin();
    store_thin(0, 0);
    __syncthreads();
    for (uint32_t ch = 0; ch < nchunks; ch += 3) {
        step(ch, ra, rc);
        if (ch + 1 < nchunks) step(ch + 1, rb, ra);
        if (ch + 2 < nchunks) step(ch + 2, rc, rb);
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");       // the redundant tail loads

    // accumulator register r of lane (n31, h): thin row 8 (r / 4) + 4 h + r % 4, streamed row n31
    if (a.ws) {
#pragma unroll
        for (int rt = 0; rt < RT; ++rt) {
            const uint32_t r = row0 + rt * 32u + n31;
            if (r >= a.R) continue;
#pragma unroll
            for (int ct = 0; ct < CT; ++ct)
#pragma unroll
                for (int q = 0; q < 16; ++q) {
                    const uint32_t c = cbase + ct * 32u + 8u * (q >> 2) + 4u * h + (q & 3);
                    if (c < a.NC) a.ws[((size_t)blockIdx.y * a.NC + c) * a.R + r] = acc[rt][ct][q];
                }
        }
        return;
    }
    auto emit = [&](auto slow_c) __attribute__((always_inline)) {
        constexpr bool SLOW = decltype(slow_c)::value;
#pragma unroll
        for (int rt = 0; rt < RT; ++rt) {
            const uint32_t r = row0 + rt * 32u + n31;
            if (r >= a.R) continue;
            // streamed rows that are outputs have one bias per lane and row tile
            const float bias_r = a.mode_b ? 0.0f : elem_value_rt(a.L.bias_fmt, a.L.bias, r) * a.L.bscale;
#pragma unroll
            for (int ct = 0; ct < CT; ++ct)
#pragma unroll
                for (int q = 0; q < 16; ++q) {
                    const uint32_t c = cbase + ct * 32u + 8u * (q >> 2) + 4u * h + (q & 3);
                    if (c >= a.NC) continue;
                    const float bias = a.mode_b ? elem_value_rt(a.L.bias_fmt, a.L.bias, c) * a.L.bscale : bias_r;
                    skinny_emit_biased<F16T, SLOW>(a, c, r, acc[rt][ct][q], bias);
                }
        }
    };
    if (a.L.act == A_SIGMOID || a.L.act == A_TANH) emit(std::true_type{});
    else emit(std::false_type{});
}

// Variant for a thin operand of at most NCP (8 or 16; the host uses 8) rows: the NW waves of a workgroup share one tile of 32
// streamed rows and split K among themselves (wave w takes chunks w, w + NW, ...), so that a layer with many streamed
// rows needs no K split across workgroups, no partial sums in memory and no second launch.  Each wave stages its own
// thin chunks in its own LDS region (no workgroup barrier in the loop); the NW accumulator tiles meet in LDS at the
// end and are added in wave order.  Loads and their bookkeeping are those of sp_skinny16.
template <int FMT, bool F16T, int NCP, int NW>
__global__ __launch_bounds__(64 * NW) void sp_skinny16_kw(const SkinnyArgs a)
{
    using F = SkinnyFmt<FMT>;
    constexpr int EPL = F::EPL, LPC = F::LPC, BKC = F::BKC, STEPS = F::STEPS, PITCH = F::PITCH;
    constexpr int UNITS = NCP * (BKC / 16);                // 16-code units of one thin chunk
    constexpr int UPL = (UNITS + 63) / 64;                 // units per lane
    constexpr int STAGE = NCP * PITCH;
    constexpr int NQ = NCP / 2;                            // accumulator registers per lane that belong to thin rows < NCP
    extern __shared__ __attribute__((aligned(16))) uint8_t sk_lds[];

    const int t = threadIdx.x, lane = t & 63;
    const int wave = __builtin_amdgcn_readfirstlane(t >> 6);   // uniform: chunk addresses stay in scalar registers
    const uint32_t n31 = lane & 31, h = lane >> 5;
    const uint32_t K = a.L.K;
    const uint32_t r_out = blockIdx.x * 32u + n31;
    const uint32_t half = blockIdx.y / a.ksplits;
    const uint8_t *const stream = a.mode_b ? a.stream + (size_t)half * a.half_elems * 2u : a.stream;
    const uint16_t *const thin = a.mode_b ? a.thin : a.thin + (size_t)half * a.half_elems;
    const uint32_t kbeg = (blockIdx.y % a.ksplits) * a.kper;
    const uint32_t kend = kbeg + a.kper < K ? kbeg + a.kper : K;
    const uint32_t nchunks = (kend - kbeg + BKC - 1) / BKC;
    const size_t row_bytes = (size_t)K * F::bits / 8u;
    uint8_t *my_lds = sk_lds + wave * (2 * STAGE);

    const uint32_t svoff = (uint32_t)((size_t)(r_out < a.R ? r_out : a.R - 1) * row_bytes) + h * 16u;
    uint32_t tvoff[UPL][2];
    bool trow_ok[UPL];
#pragma unroll
    for (int q = 0; q < UPL; ++q) {
        const uint32_t u = (uint32_t)lane + 64u * q;
        const uint32_t row = u / (BKC / 16), uc = u % (BKC / 16);
        trow_ok[q] = u < (uint32_t)UNITS && row < a.NC;
#pragma unroll
        for (int e = 0; e < 2; ++e) tvoff[q][e] = trow_ok[q] ? (uint32_t)(((size_t)row * K + uc * 16u + 8u * e) * 2u) : 0u;
    }

    f32x16 acc;
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[r] = 0.0f;

    // this wave's chunks: w, w + NW, ...; index i of that sequence past the end is clamped to the last one
    const uint32_t my_n = nchunks > (uint32_t)wave ? (nchunks - (uint32_t)wave + NW - 1) / NW : 0u;
    const uint32_t last_chunk = nchunks - 1;
    auto chunk_of = [&](uint32_t i) { return (uint32_t)wave + (i < my_n ? i : my_n - 1) * NW; };
    constexpr int S_LOADS = LPC, T_LOADS = UPL * 2;
    auto issue_stream = [&](uint32_t i, u32x4 (&dst)[LPC]) {
        const uint32_t ch = chunk_of(i);
        if (ch < last_chunk) {
            const uint8_t *sb = stream + (size_t)(kbeg + ch * BKC) * F::bits / 8u;
#pragma unroll
            for (int j = 0; j < LPC; ++j) {
                if (j == 0) load16_async<0>(dst[j], svoff, sb);
                else if (j == 1) load16_async<32>(dst[j], svoff, sb);
                else if (j == 2) load16_async<64>(dst[j], svoff, sb);
                else load16_async<96>(dst[j], svoff, sb);
            }
        } else {
            const uint32_t kc0 = kbeg + last_chunk * BKC;
#pragma unroll
            for (int j = 0; j < LPC; ++j) {
                const uint32_t k = kc0 + 2u * j * EPL;                 // first code of the h = 0 lane load
                const uint32_t add = k + h * EPL < K ? k * F::bits / 8u : 0u - h * 16u;
                load16_async<0>(dst[j], svoff + add, stream);
            }
        }
    };
    u32x4 thin_regs[UPL][2];
    auto issue_thin = [&](uint32_t i) {
        const uint32_t ch = chunk_of(i);
        if (ch < last_chunk) {
            const uint16_t *tb = thin + (kbeg + ch * BKC);
#pragma unroll
            for (int q = 0; q < UPL; ++q)
#pragma unroll
                for (int e = 0; e < 2; ++e) load16_async<0>(thin_regs[q][e], tvoff[q][e], tb);
        } else {
            const uint32_t kc0 = kbeg + last_chunk * BKC;
#pragma unroll
            for (int q = 0; q < UPL; ++q) {
                const uint32_t uc = ((uint32_t)lane + 64u * q) % (BKC / 16);
#pragma unroll
                for (int e = 0; e < 2; ++e) {
                    const bool valid = trow_ok[q] && kc0 + uc * 16u + 8u * e + 8u <= kend;
                    load16_async<0>(thin_regs[q][e], valid ? tvoff[q][e] + kc0 * 2u : 0u, thin);
                }
            }
        }
    };
    auto store_thin = [&](int stage, uint32_t i) {
        const uint32_t kc0 = kbeg + chunk_of(i) * BKC;
#pragma unroll
        for (int q = 0; q < UPL; ++q) {
            const uint32_t u = (uint32_t)lane + 64u * q;
            if (u >= (uint32_t)UNITS) continue;
            const uint32_t row = u / (BKC / 16), uc = u % (BKC / 16);
            const uint32_t k = kc0 + uc * 16u;
            const uint32_t keep0 = (trow_ok[q] && k + 8u <= kend) ? 0xFFFFFFFFu : 0u;
            const uint32_t keep1 = (trow_ok[q] && k + 16u <= kend) ? 0xFFFFFFFFu : 0u;
            const uint32_t in[8] = {thin_regs[q][0].x & keep0, thin_regs[q][0].y & keep0, thin_regs[q][0].z & keep0,
                                    thin_regs[q][0].w & keep0, thin_regs[q][1].x & keep1, thin_regs[q][1].y & keep1,
                                    thin_regs[q][1].z & keep1, thin_regs[q][1].w & keep1};
            uint32_t o[8];
            skinny_permute_unit<FMT>(in, o);
            uint8_t *dst = my_lds + stage * STAGE + row * PITCH + uc * 32u;
            *reinterpret_cast<uint4 *>(dst) = make_uint4(o[0], o[1], o[2], o[3]);
            *reinterpret_cast<uint4 *>(dst + 16) = make_uint4(o[4], o[5], o[6], o[7]);
        }
    };
    auto compute = [&](int stage, uint32_t i, const u32x4 (&cur)[LPC]) {
        // lanes of thin rows >= NCP read a row below NCP again: their accumulator rows are never stored
        const uint8_t *sbase = my_lds + stage * STAGE + (n31 & (NCP - 1)) * PITCH + h * (EPL * 2);
        const uint32_t kc0 = kbeg + chunk_of(i) * BKC;
#pragma unroll
        for (int j = 0; j < LPC; ++j) {
            const uint32_t keep = (F::bits == 16 && kc0 + (2u * j + h) * EPL >= K) ? 0u : 0xFFFFFFFFu;
#pragma unroll
            for (int st = 0; st < STEPS; ++st) {
                const uint4 tf = *reinterpret_cast<const uint4 *>(sbase + (2 * j * EPL + 8 * st) * 2);
                uint4 v = make_uint4(cur[j].x, cur[j].y, cur[j].z, cur[j].w);
                if constexpr (F::bits == 16) { v.x &= keep; v.y &= keep; v.z &= keep; v.w &= keep; }
                uint32_t sf[4];
                skinny_frag<FMT>(v, st, sf);
                if constexpr (F16T) {
                    f16x8 af, bf;
                    __builtin_memcpy(&af, &tf, 16);
                    __builtin_memcpy(&bf, sf, 16);
                    acc = __builtin_amdgcn_mfma_f32_32x32x16_f16(af, bf, acc, 0, 0, 0);
                } else {
                    bf16x8 af, bf;
                    __builtin_memcpy(&af, &tf, 16);
                    __builtin_memcpy(&bf, sf, 16);
                    acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(af, bf, acc, 0, 0, 0);
                }
            }
        }
    };
    auto pin_stream = [&](u32x4 (&r)[LPC]) {
#pragma unroll
        for (int j = 0; j < LPC; ++j) asm volatile("" : "+v"(r[j]));
    };
    auto pin_thin = [&]() {
#pragma unroll
        for (int q = 0; q < UPL; ++q)
#pragma unroll
            for (int e = 0; e < 2; ++e) asm volatile("" : "+v"(thin_regs[q][e]));
    };
    // in flight on entry: streamed chunks i (in `cur`) and i + 1; issued here: thin block i + 1, streamed chunk i + 2
    auto step = [&](uint32_t i, u32x4 (&cur)[LPC], u32x4 (&far)[LPC]) {
        const int stage = (int)(i & 1u);
        issue_thin(i + 1);
        issue_stream(i + 2, far);
        asm volatile("s_waitcnt vmcnt(%0)" ::"n"(2 * S_LOADS + T_LOADS) : "memory");
        pin_stream(cur);
        compute(stage, i, cur);
        asm volatile("s_waitcnt vmcnt(%0)" ::"n"(S_LOADS) : "memory");
        pin_thin();
        store_thin(stage ^ 1, i + 1);
    };
    if (my_n) {
        u32x4 ra[LPC], rb[LPC], rc[LPC];
        issue_thin(0);
        issue_stream(0, ra);
        issue_stream(1, rb);
        asm volatile("s_waitcnt vmcnt(%0)" ::"n"(2 * S_LOADS) : "memory");
        pin_thin();
        store_thin(0, 0);
        for (uint32_t i = 0; i < my_n; i += 3) {
            step(i, ra, rc);
            if (i + 1 < my_n) step(i + 1, rb, ra);
            if (i + 2 < my_n) step(i + 2, rc, rb);
        }
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");   // the redundant tail loads
    }

    // accumulator register q of lane (n31, h): thin row 8 (q / 4) + 4 h + q % 4, streamed row n31
    float *red = reinterpret_cast<float *>(sk_lds + NW * 2 * STAGE);
#pragma unroll
    for (int q = 0; q < NQ; ++q) red[(wave * NQ + q) * 64 + lane] = acc[q];
    __syncthreads();
    if (wave != 0 || r_out >= a.R) return;
    if (a.soft_out) {
        // the thin rows are all the outputs of sample r_out, half of them in lane n31 and half in lane n31 + 32:
        // softmax as Activation.c:5-21 (largest logit subtracted, exponentials, one division by their sum)
        float v[NQ];
        float m = -3.402823466e+38f;
#pragma unroll
        for (int q = 0; q < NQ; ++q) {
            const uint32_t c = 8u * (q >> 2) + 4u * h + (q & 3);
            float sum = 0.0f;
#pragma unroll
            for (int w = 0; w < NW; ++w) sum += red[(w * NQ + q) * 64 + lane];
            const float bias = elem_value_rt(a.L.bias_fmt, a.L.bias, c < a.NC ? c : 0u) * a.L.bscale;
            v[q] = c < a.NC ? fmaf(sum, a.L.wscale, bias) : -3.402823466e+38f;
            m = fmaxf(m, v[q]);
        }
        m = fmaxf(m, __shfl_xor(m, 32));
        float s = 0.0f;
#pragma unroll
        for (int q = 0; q < NQ; ++q) {
            const uint32_t c = 8u * (q >> 2) + 4u * h + (q & 3);
            v[q] = c < a.NC ? expf(v[q] - m) : 0.0f;
            s += v[q];
        }
        s += __shfl_xor(s, 32);
        const float inv = s > 0.0f ? 1.0f / s : 1.0f;
#pragma unroll
        for (int q = 0; q < NQ; ++q) {
            const uint32_t c = 8u * (q >> 2) + 4u * h + (q & 3);
            if (c >= a.NC) continue;
            const size_t o = (size_t)r_out * a.L.N + c;
            const float y = v[q] * inv;
            if (a.soft_kind == 0) reinterpret_cast<float *>(a.soft_out)[o] = y;
            else if (a.soft_kind == 1) reinterpret_cast<uint16_t *>(a.soft_out)[o] = f32_to_bf16_rne(y);
            else reinterpret_cast<uint16_t *>(a.soft_out)[o] = f32_to_f16_sat(y);
        }
        return;
    }
#pragma unroll
    for (int q = 0; q < NQ; ++q) {
        const uint32_t c = 8u * (q >> 2) + 4u * h + (q & 3);
        if (c >= a.NC) continue;
        float sum = 0.0f;
#pragma unroll
        for (int w = 0; w < NW; ++w) sum += red[(w * NQ + q) * 64 + lane];
        if (a.ws) a.ws[((size_t)blockIdx.y * a.NC + c) * a.R + r_out] = sum;
        else skinny_emit<F16T>(a, c, r_out, sum);
    }
}

// adds the partial sums of sp_skinny16 (K splits in split order; with split activations the sums of the second matrix,
// scaled by 2^-11, after those of the first) and applies bias and activation; a thread takes four neighbouring
// streamed rows (VEC: R is a multiple of four and the rows are outputs, so they are neighbours in C as well) or one
template <bool F16T>
__device__ __forceinline__ void skinny_store(const SkinnyArgs &a, size_t o, float v)
{
    if (a.out_f32) reinterpret_cast<float *>(a.C)[o] = v;
    else if (a.halves == 2) {
        uint16_t hi, lo;
        split_f16(v, hi, lo);
        uint16_t *c = reinterpret_cast<uint16_t *>(a.C);
        c[o] = hi;
        c[(size_t)a.NC * a.R + o] = lo;               // samples x outputs elements further on
    } else reinterpret_cast<uint16_t *>(a.C)[o] = f32_to_t16<F16T>(v);
}

template <bool F16T, bool VEC>
__global__ __launch_bounds__(256) void sp_skinny_reduce(const SkinnyArgs a, uint32_t splits)
{
    const uint64_t total = (uint64_t)a.NC * a.R;
    const uint32_t parts = splits * a.halves;
    if constexpr (VEC) {
        const uint64_t idx = ((uint64_t)blockIdx.x * 256u + threadIdx.x) * 4u;
        if (idx >= total) return;
        float4 sum = make_float4(0.0f, 0.0f, 0.0f, 0.0f), low = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
        for (uint32_t sp = 0; sp < parts; ++sp) {
            const float4 v = *reinterpret_cast<const float4 *>(a.ws + (uint64_t)sp * total + idx);
            if (sp < splits) { sum.x += v.x; sum.y += v.y; sum.z += v.z; sum.w += v.w; }
            else { low.x += v.x; low.y += v.y; low.z += v.z; low.w += v.w; }
        }
        const uint32_t c = (uint32_t)(idx / a.R), r = (uint32_t)(idx % a.R);
        const float in[4] = {fmaf(low.x, kLoScale, sum.x), fmaf(low.y, kLoScale, sum.y), fmaf(low.z, kLoScale, sum.z),
                             fmaf(low.w, kLoScale, sum.w)};
        float v[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const float bias = elem_value_rt(a.L.bias_fmt, a.L.bias, r + i) * a.L.bscale;
            v[i] = apply_act(fmaf(in[i], a.L.wscale, bias), a.L.act);
        }
        const size_t o = (size_t)c * a.L.N + r;
        if (a.out_f32) {
            *reinterpret_cast<float4 *>(reinterpret_cast<float *>(a.C) + o) = make_float4(v[0], v[1], v[2], v[3]);
        } else if (a.halves == 2) {
            uint16_t hi[4], lo[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) split_f16(v[i], hi[i], lo[i]);
            uint16_t *cc = reinterpret_cast<uint16_t *>(a.C);
            *reinterpret_cast<uint2 *>(cc + o) = make_uint2((uint32_t)hi[0] | ((uint32_t)hi[1] << 16), (uint32_t)hi[2] | ((uint32_t)hi[3] << 16));
            *reinterpret_cast<uint2 *>(cc + total + o) = make_uint2((uint32_t)lo[0] | ((uint32_t)lo[1] << 16), (uint32_t)lo[2] | ((uint32_t)lo[3] << 16));
        } else {
            const uint32_t lo = (uint32_t)f32_to_t16<F16T>(v[0]) | ((uint32_t)f32_to_t16<F16T>(v[1]) << 16);
            const uint32_t hi = (uint32_t)f32_to_t16<F16T>(v[2]) | ((uint32_t)f32_to_t16<F16T>(v[3]) << 16);
            *reinterpret_cast<uint2 *>(reinterpret_cast<uint16_t *>(a.C) + o) = make_uint2(lo, hi);
        }
    } else {
        const uint64_t idx = (uint64_t)blockIdx.x * 256u + threadIdx.x;
        if (idx >= total) return;
        float sum = 0.0f, low = 0.0f;
        for (uint32_t sp = 0; sp < parts; ++sp) {
            const float v = a.ws[(uint64_t)sp * total + idx];
            if (sp < splits) sum += v; else low += v;
        }
        const uint32_t c = (uint32_t)(idx / a.R), r = (uint32_t)(idx % a.R);
        const uint32_t m = a.mode_b ? r : c, n = a.mode_b ? c : r;
        const float bias = elem_value_rt(a.L.bias_fmt, a.L.bias, n) * a.L.bscale;
        skinny_store<F16T>(a, (size_t)m * a.L.N + n, apply_act(fmaf(fmaf(low, kLoScale, sum), a.L.wscale, bias), a.L.act));
    }
}

// unscaled integer codes of a small weight array as FP16 (the thin operand of a layer with few outputs)
template <int FMT>
__global__ __launch_bounds__(256) void sp_codes16(const uint8_t *__restrict__ codes, uint16_t *__restrict__ out, uint64_t n)
{
    const uint64_t i = (uint64_t)blockIdx.x * 256u + threadIdx.x;
    if (i < n) out[i] = f32_to_f16_sat(elem_value<FMT>(codes, i));
}
