// hip_forward.hip — gfx950 kernels and the C ABI of spingalett_hip.h.
//
// One translation unit holds every HIP runtime call and every kernel:
//   sp_decode         element decoders (bit-exact with Serialize.c:45-85,195-297)
//   sp_gemv*          1..4 samples (FP32 weights: up to 64): vector kernels, FP32-grade arithmetic; integer weights
//                     as exact integer dot products on the INT8 matrix cores (sp_gemv_i8mfma)
//   sp_skinny16[_kw]  5..256 samples, or layers with <= 64 outputs: one operand streamed once through registers
//                     into 16-bit MFMAs, the thin one in LDS (_kw: thin side of <= 8 rows, K split inside the workgroup)
//   sp_gemm16_big / sp_gemm16   larger batches: LDS-tiled dequant-to-16-bit MFMA GEMM, fused epilogue
//   sp_gemm32_f32     FP32 weights beyond 64 samples: FP32 MFMA GEMM
//   sp_softmax_rows   per-sample softmax (Activation.c:5-21)
//   sp_eval_*         loss and argmax of a labelled batch (SIMD.c:522-552, Training.c:421-435)
//   hip_train.inl     the batched training step (included at the end)
// Weights stay in their serialized form on the device; row-major [out][in]
// (Private.h:16), element i of an INT4 array in nibble i&1 of byte i/2, element
// i of an INT2 array at bits 2(i%4) of byte i/4 (Serialize.c:148-152,181-183).

#include <hip/hip_runtime.h>

#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <mutex>
#include <new>
#include <type_traits>
#include <vector>

#include "spingalett_hip.h"

namespace {

// ---------------------------------------------------------------------------
// formats and small helpers
// ---------------------------------------------------------------------------
enum : int { F32 = 0, F16 = 1, BF16 = 2, I8 = 3, I4 = 4, I2 = 5, NFMT = 6 };
enum : int { A_SIGMOID = 0, A_RELU, A_TANH, A_LEAKY, A_FOO52, A_SOFTMAX, A_NONE, A_COUNT };

constexpr int kWave = 64;

__host__ __device__ constexpr int fmt_bits(int f)
{
    return f == F32 ? 32 : (f == F16 || f == BF16) ? 16 : f == I8 ? 8 : f == I4 ? 4 : 2;
}

size_t fmt_bytes(int f, uint64_t n)
{
    return (size_t)((n * (uint64_t)fmt_bits(f) + 7u) / 8u);
}

// divisor d of the integer formats: w = (q / d) * max   (Serialize.c:233,258,285)
float fmt_divisor(int f) { return f == I8 ? 127.0f : f == I4 ? 7.0f : 1.0f; }

// folded scale used by the arithmetic kernels: w = q * scale
float fmt_scale(int f, float max_val)
{
    if (f == F32 || f == F16 || f == BF16) return 1.0f;
    if (!(max_val > 0.0f)) return 0.0f;            // Serialize.c:231-236: zeros
    return (float)((double)max_val / (double)fmt_divisor(f));
}

thread_local char g_err[512] = "";

int fail_msg(const char *msg)
{
    snprintf(g_err, sizeof g_err, "%s", msg);
    return 1;
}

int fail_hip(const char *what, hipError_t e)
{
    snprintf(g_err, sizeof g_err, "%s: %s", what, hipGetErrorString(e));
    return 1;
}

#define HCHECK(expr)                                              \
    do {                                                          \
        hipError_t e_ = (expr);                                   \
        if (e_ != hipSuccess) return fail_hip(#expr, e_);         \
    } while (0)

hipStream_t g_stream = nullptr;
const char *g_last_kernel = "";   // main kernel of the most recent layer launch
constexpr uint32_t kGemvStageBytes = 64u * 1024u;   // LDS budget of one stage of the integer GEMV

std::mutex g_init_mutex;

// One stream per process (default priority), created at first use; safe to call from several threads.
int ensure_stream()
{
    std::lock_guard<std::mutex> lock(g_init_mutex);
    if (g_stream) return 0;
    int cnt = 0;
    HCHECK(hipGetDeviceCount(&cnt));
    if (cnt <= 0) return fail_msg("no HIP device");
    HCHECK(hipSetDevice(0));
    HCHECK(hipStreamCreateWithFlags(&g_stream, hipStreamNonBlocking));
    return 0;
}

// ---------------------------------------------------------------------------
// device-side element access
// ---------------------------------------------------------------------------
__device__ __forceinline__ float bits_to_float(uint32_t u) { return __uint_as_float(u); }

// binary16 -> binary32, integer arithmetic only; any NaN becomes the quiet NaN
// of the same sign (Serialize.c:45-72).
__device__ __forceinline__ float half_bits_to_float_exact(uint32_t h)
{
    uint32_t s = (h & 0x8000u) << 16;
    uint32_t e = (h >> 10) & 31u;
    uint32_t m = h & 1023u;
    uint32_t f;
    if (e == 31u) {
        f = s | (m ? 0x7FC00000u : 0x7F800000u);
    } else if (e != 0u) {
        f = s | ((e + 112u) << 23) | (m << 13);
    } else if (m == 0u) {
        f = s;
    } else {
        int lz = __clz((int)m) - 21;               // shifts until bit 10 is set
        m = (m << lz) & 1023u;
        f = s | ((uint32_t)(113 - lz) << 23) | (m << 13);
    }
    return bits_to_float(f);
}

// integer code of element i of a packed INT array
template <int FMT>
__device__ __forceinline__ int int_code(const uint8_t *codes, uint64_t i)
{
    if constexpr (FMT == I8) {
        return (int)(int8_t)codes[i];
    } else if constexpr (FMT == I4) {
        uint32_t byte = codes[i >> 1];
        uint32_t nib = (i & 1u) ? (byte >> 4) : (byte & 15u);
        return (int)nib - (int)((nib & 8u) << 1);
    } else {
        uint32_t c = (codes[i >> 2] >> ((i & 3u) * 2u)) & 3u;
        return (int)c - (int)((c & 2u) << 1);
    }
}

// unscaled value of element i: the float itself for FP formats, (float)q for INT
template <int FMT>
__device__ __forceinline__ float elem_value(const uint8_t *codes, uint64_t i)
{
    if constexpr (FMT == F32) {
        return reinterpret_cast<const float *>(codes)[i];
    } else if constexpr (FMT == F16) {
        return half_bits_to_float_exact(reinterpret_cast<const uint16_t *>(codes)[i]);
    } else if constexpr (FMT == BF16) {
        return bits_to_float((uint32_t)reinterpret_cast<const uint16_t *>(codes)[i] << 16);
    } else {
        return (float)int_code<FMT>(codes, i);
    }
}

__device__ __forceinline__ float elem_value_rt(int fmt, const uint8_t *codes, uint64_t i)
{
    switch (fmt) {
    case F32:  return elem_value<F32>(codes, i);
    case F16:  return elem_value<F16>(codes, i);
    case BF16: return elem_value<BF16>(codes, i);
    case I8:   return elem_value<I8>(codes, i);
    case I4:   return elem_value<I4>(codes, i);
    default:   return elem_value<I2>(codes, i);
    }
}

// Activation.c:23-38 (leak factor fixed at 0.01f).  Softmax is a row operation
// and handled by sp_softmax_rows.
__device__ __forceinline__ float apply_act(float x, int act)
{
    switch (act) {
    case A_SIGMOID: return 1.0f / (1.0f + expf(-x));
    case A_RELU:    return x > 0.0f ? x : 0.0f;
    case A_TANH:    return tanhf(x);
    case A_LEAKY:   return x > 0.0f ? x : 0.01f * x;
    case A_FOO52:   return x > 1.0f ? 1.0f + 0.01f * (x - 1.0f) : (x < 0.0f ? 0.01f * x : x);
    default:        return x;
    }
}

__device__ __forceinline__ uint16_t f32_to_bf16_rne(float x)
{
    uint32_t u = __float_as_uint(x);
    if ((u & 0x7FFFFFFFu) > 0x7F800000u) return (uint16_t)((u >> 16) | 0x40u);   // NaN
    u += 0x7FFFu + ((u >> 16) & 1u);
    return (uint16_t)(u >> 16);
}

__device__ __forceinline__ uint16_t f32_to_f16_sat(float x)
{
    if (x != x) return (uint16_t)0x7E00u;
    x = fminf(fmaxf(x, -65504.0f), 65504.0f);
    _Float16 h = (_Float16)x;
    uint16_t r;
    __builtin_memcpy(&r, &h, 2);
    return r;
}

template <bool F16T>
__device__ __forceinline__ uint16_t f32_to_t16(float x)
{
    if constexpr (F16T) return f32_to_f16_sat(x);
    else return f32_to_bf16_rne(x);
}

__device__ __forceinline__ float wave_sum(float v)
{
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, kWave);
    return v;
}

__device__ __forceinline__ int wave_sum_i(int v)
{
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, kWave);
    return v;
}

__device__ __forceinline__ float wave_max(float v)
{
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, kWave));
    return v;
}

// ---------------------------------------------------------------------------
// decode kernel — the device form of read_array_compressed
// ---------------------------------------------------------------------------
// lut[q + bias] = fl((float)q / d) computed on the host in IEEE arithmetic, so the
// strict result fl(lut * max) does not depend on the device's division.
struct DecodeParams {
    const uint8_t *codes;
    float *out;
    uint64_t n;
    float max_val;       // scale from the file
    float rel_scale;     // fl(max * fl(1/d))  (mode 1)
    int mode;            // 0 strict, 1 release
    float lut[256];
};

template <int FMT>
__global__ __launch_bounds__(256) void sp_decode(const DecodeParams p)
{
    uint64_t i = (uint64_t)blockIdx.x * 256u + threadIdx.x;
    if (i >= p.n) return;
    float v;
    if constexpr (FMT == F32 || FMT == F16 || FMT == BF16) {
        v = elem_value<FMT>(p.codes, i);
    } else {
        if (!(p.max_val > 0.0f)) {
            v = 0.0f;
        } else {
            int q = int_code<FMT>(p.codes, i);
            if (FMT == I2) v = __fmul_rn((float)q, p.max_val);                    // Serialize.c:285
            else if (p.mode == 1) v = __fmul_rn((float)q, p.rel_scale);
            else v = __fmul_rn(p.lut[q + (FMT == I8 ? 128 : 8)], p.max_val);      // Serialize.c:233,258
        }
    }
    p.out[i] = v;
}

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
#pragma unroll
        for (int b = 0; b < BT; ++b) {
            const int bb = b < nb ? b : nb - 1;
            const float4 *xp = reinterpret_cast<const float4 *>(x + (size_t)bb * L.K + (size_t)c * EPC);
#pragma unroll
            for (int e = 0; e < EPC / 4; ++e) {
                float4 xv = xp[e];
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
    uint32_t rw, ks;       // waves of a workgroup: row groups x K shares
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

// One wave quantises one scale chunk (kc <= 2048 codes starting at code kbase) of up to NS
// samples (rows xr, xr + K, ...; ns of them are real): every lane fetches its words'
// activations in one batch of loads (quant_load), the wave agrees on the largest magnitude per
// sample, and each lane converts what it holds (quant_finish).
// A 64-byte weight segment (block) is spread over 4 lane groups g of 16 bytes = 4 words w;
// word w holds WK codes; after unpacking, MFMA u of that block takes byte i of word w from code
//   INT8: 4w+i (u = 0)      INT4: 8w + 2i + u      INT2: 16w + 4i + u
// of the lane group.  store(sample, block in chunk, u, g, w, d0, d1, d2) receives the operand
// words; done(sample, {bits of 2^-p, sum d0, sum d1, sum d2}) the scale record (same in every lane).
template <int FMT, int NS>
struct QuantRegs {
    static constexpr int MAXIT = 2048 / (64 * I8Fmt<FMT>::WK);
    static constexpr int F4 = I8Fmt<FMT>::WK / 4;
    float4 v[NS][MAXIT][F4];
    float m[NS];
};

template <int FMT, int NS>
__device__ __forceinline__ void quant_load(QuantRegs<FMT, NS> &q, const float *xr, uint32_t K, uint32_t kbase,
                                           uint32_t kc, int ns, int lane)
{
    using F = I8Fmt<FMT>;
    constexpr int KL = F::KL, WK = F::WK, F4 = WK / 4, MAXIT = QuantRegs<FMT, NS>::MAXIT;
    constexpr uint32_t WPB = KL / WK;                            // words per block (16)
    const uint32_t iters = kc / (64u * WK);
#pragma unroll
    for (int s = 0; s < NS; ++s) {
        q.m[s] = 0.0f;
        const float *xs = xr + (size_t)(s < ns ? s : 0) * K;
#pragma unroll
        for (int it = 0; it < MAXIT; ++it) {
            const uint32_t wl = (uint32_t)it * 64u + (uint32_t)lane;
            const uint32_t blk = wl / WPB, r = wl % WPB, gg = r >> 2, w = r & 3u;
            const uint32_t kw = kbase + blk * KL + gg * (KL / 4) + w * WK;     // first code of the word
            const bool valid = (uint32_t)it < iters && kw < K;                  // rows are whole numbers of words
            const float4 *src = reinterpret_cast<const float4 *>(xs + (valid ? kw : 0u));
#pragma unroll
            for (int c = 0; c < F4; ++c) {
                float4 t = src[c];
                if (!valid) t = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
                q.v[s][it][c] = t;
                q.m[s] = fmaxf(q.m[s], fmaxf(fmaxf(fabsf(t.x), fabsf(t.y)), fmaxf(fabsf(t.z), fabsf(t.w))));
            }
        }
    }
}

template <int FMT, int NS, class Store, class Done>
__device__ __forceinline__ void quant_finish(const QuantRegs<FMT, NS> &q, uint32_t kc, int ns, int lane, Store store, Done done)
{
    using F = I8Fmt<FMT>;
    constexpr int KL = F::KL, NMF = F::NMF, WK = F::WK, MAXIT = QuantRegs<FMT, NS>::MAXIT;
    constexpr uint32_t WPB = KL / WK;
    const uint32_t iters = kc / (64u * WK);
#pragma unroll
    for (int s = 0; s < NS; ++s) {
        if (s >= ns) break;
        const float amax = wave_max(q.m[s]);
        int e = (int)((__float_as_uint(amax) >> 23) & 255u) - 127;
        if (e < -126) e = -126;
        int p = 21 - e;                                          // |X| < 2^22: the top digit stays inside INT8
        p = p > 126 ? 126 : p;
        const bool live = amax > 0.0f && amax < 3.0e38f;         // zero, inf and NaN chunks contribute nothing
        const float scale = live ? __uint_as_float((uint32_t)(p + 127) << 23) : 0.0f;
        int ds0 = 0, ds1 = 0, ds2 = 0;
#pragma unroll
        for (int it = 0; it < MAXIT; ++it) {
            if ((uint32_t)it < iters) {
                const uint32_t wl = (uint32_t)it * 64u + (uint32_t)lane;
                const uint32_t blk = wl / WPB, r = wl % WPB, gg = r >> 2, w = r & 3u;
                uint32_t d0[NMF], d1[NMF], d2[NMF];
                quant_word<FMT>(q.v[s][it], scale, d0, d1, d2, ds0, ds1, ds2);
#pragma unroll
                for (int u = 0; u < NMF; ++u) store((uint32_t)s, blk, (uint32_t)u, gg, w, d0[u], d1[u], d2[u]);
            }
        }
        ds0 = wave_sum_i(ds0);
        ds1 = wave_sum_i(ds1);
        ds2 = wave_sum_i(ds2);
        done((uint32_t)s, make_int4(live ? (int)((uint32_t)(127 - p) << 23) : 0, ds0, ds1, ds2));
    }
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
    QuantRegs<FMT, 1> qr;
    quant_load<FMT, 1>(qr, a.x + (size_t)s0 * a.L.K, a.L.K, ch * a.kc, a.kc, 1, lane);
    quant_finish<FMT, 1>(qr, a.kc, 1, lane,
        [&](uint32_t, uint32_t blk, uint32_t u, uint32_t g, uint32_t w, uint32_t d0, uint32_t d1, uint32_t d2) {
            uint8_t *dst = a.aq + (((((size_t)ch * nblk + blk) * NMF + u) * 4 + g) * (size_t)a.nb + s0) * 48 + w * 4;
            *reinterpret_cast<uint32_t *>(dst) = d0;
            *reinterpret_cast<uint32_t *>(dst + 16) = d1;
            *reinterpret_cast<uint32_t *>(dst + 32) = d2;
        },
        [&](uint32_t, int4 md) {
            if (lane == 0) {
                a.inv[rec] = __int_as_float(md.x);
                int *d = a.dsum + (size_t)rec * 4;
                d[0] = md.y; d[1] = md.z; d[2] = md.w; d[3] = 0;
            }
        });
}

// MT = 16-row A tiles (four samples each).  Rows of D that belong to no sample
// (fourth row of a slot, slots beyond nb) are never read, so their lanes may load
// anything: they are pointed at the start of the block.
// The waves of a workgroup are rw row groups x ks K shares (wave = ks_id * rw +
// rw_id); share ks_id takes the 64-byte blocks ks_id, ks_id + ks, ... of its rows.
// Weights are fetched in groups of four blocks, the next group in flight while
// the current one is multiplied; scale chunks are whole numbers of groups.
//
// FQ > 0 (n <= FQ <= 4): the workgroup (at most 8 waves) quantises the activations itself,
// straight into LDS, instead of copying planes a separate launch prepared: every workgroup
// repeats the (small) job, and the layer costs one launch instead of two.
template <int FMT, int MT, int FQ>
__global__ __launch_bounds__(FQ ? 512 : MT <= 4 ? 1024 : 256) void sp_gemv_i8mfma(const GemvI8Args a)
{
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

    // The self-quantising variant requests the activations of its first scale chunk before the
    // weights: loads complete in order, and the quantiser should not wait behind the weight stream.
    constexpr int QN = FQ ? FQ : 1;
    QuantRegs<FMT, QN> qr;
    const uint32_t spc = ((uint32_t)nb + QN - 1) / QN;         // sample groups per chunk
    const uint32_t nch_first = chunks_per_stage <= a.nchunks ? chunks_per_stage : a.nchunks;
    auto unit_load = [&](uint32_t ch0, uint32_t ui) {
        const uint32_t chl = ui / spc, sbase = (ui % spc) * QN;
        const int ns = nb - (int)sbase < QN ? nb - (int)sbase : QN;
        quant_load<FMT, QN>(qr, a.x + (size_t)sbase * K, K, (ch0 + chl) * a.kc, a.kc, ns, lane);
    };
    if constexpr (FQ != 0) {
        if ((uint32_t)wave < nch_first * spc) unit_load(0u, (uint32_t)wave);
    }
    // then the first weight group (PD groups in flight; two measured slower than one)
    constexpr int PD = 1;
    uint4 nxt[PD][G];
#pragma unroll
    for (int d = 0; d < PD; ++d)
#pragma unroll
        for (int u = 0; u < G; ++u) nxt[d][u] = load_blk((uint32_t)(d * G + u));

    // scale records of all chunks
    if constexpr (!FQ) {
        for (uint32_t i = t; i < a.nchunks * (uint32_t)nb; i += nthreads) {
            const int *d = a.dsum + (size_t)i * 4;
            meta[i] = make_int4(__float_as_int(a.inv[i]), d[0], d[1], d[2]);
        }
    }

    uint32_t q = 0;                                            // this wave's block counter
    for (uint32_t ch0 = 0; ch0 < a.nchunks; ch0 += chunks_per_stage) {
        const uint32_t nch = ch0 + chunks_per_stage <= a.nchunks ? chunks_per_stage : a.nchunks - ch0;
        if (ch0) __syncthreads();                             // previous stage fully consumed
        if constexpr (!FQ) {
            const uint4 *src = reinterpret_cast<const uint4 *>(a.aq + (size_t)ch0 * kcb * blk_bytes);
            const uint32_t pieces = nch * kcb * (blk_bytes / 16u);
            for (uint32_t i = t; i < pieces; i += nthreads) reinterpret_cast<uint4 *>(A_lds)[i] = src[i];
        } else {
            // every wave takes whole scale chunks of this stage, FQ samples at once
            for (uint32_t ui = (uint32_t)wave; ui < nch * spc; ui += nthreads / 64u) {
                if (ch0 != 0 || ui != (uint32_t)wave) unit_load(ch0, ui);      // the first one is on its way
                const uint32_t chl = ui / spc, sbase = (ui % spc) * QN;
                const int ns = nb - (int)sbase < QN ? nb - (int)sbase : QN;
                quant_finish<FMT, QN>(qr, a.kc, ns, lane,
                    [&](uint32_t s, uint32_t blk, uint32_t u, uint32_t gg, uint32_t w, uint32_t d0, uint32_t d1, uint32_t d2) {
                        uint8_t *dst = A_lds + (((((size_t)chl * kcb + blk) * NMF + u) * 4 + gg) * (size_t)nb + sbase + s) * 48 + w * 4;
                        *reinterpret_cast<uint32_t *>(dst) = d0;
                        *reinterpret_cast<uint32_t *>(dst + 16) = d1;
                        *reinterpret_cast<uint32_t *>(dst + 32) = d2;
                    },
                    [&](uint32_t s, int4 md) {
                        if (lane == 0) meta[(size_t)(ch0 + chl) * nb + sbase + s] = md;
                    });
            }
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
            if (s0 < nb) a.y[(size_t)s0 * N + nrow] = apply_act(fmaf(yacc[mt], a.L.wscale, bias), a.L.act);
        }
    }
}

// ---------------------------------------------------------------------------
// softmax over rows (Activation.c:5-21); one wave per row
// ---------------------------------------------------------------------------
// out_kind: 0 FP32, 1 BF16, 2 FP16
__global__ __launch_bounds__(256) void sp_softmax_rows(const float *__restrict__ in, void *__restrict__ out,
                                                       int out_kind, uint32_t rows, uint32_t width)
{
    const int lane = threadIdx.x & 63;
    const uint32_t row = blockIdx.x * 4u + (threadIdx.x >> 6);
    if (row >= rows) return;
    const float *p = in + (size_t)row * width;
    auto put = [&](uint32_t i, float v) {
        const size_t o = (size_t)row * width + i;
        if (out_kind == 0) reinterpret_cast<float *>(out)[o] = v;
        else if (out_kind == 1) reinterpret_cast<uint16_t *>(out)[o] = f32_to_bf16_rne(v);
        else reinterpret_cast<uint16_t *>(out)[o] = f32_to_f16_sat(v);
    };
    constexpr int R = 16;                       // rows up to 1024 wide stay in registers: one batch of loads
    if (width <= (uint32_t)R * kWave) {
        float v[R];
#pragma unroll
        for (int j = 0; j < R; ++j) {
            const uint32_t i = (uint32_t)j * kWave + (uint32_t)lane;
            const float t = p[i < width ? i : 0u];
            v[j] = i < width ? t : -3.402823466e+38f;
        }
        float m = v[0];
#pragma unroll
        for (int j = 1; j < R; ++j) m = fmaxf(m, v[j]);
        m = wave_max(m);
        float s = 0.0f;
#pragma unroll
        for (int j = 0; j < R; ++j) {
            const uint32_t i = (uint32_t)j * kWave + (uint32_t)lane;
            v[j] = i < width ? expf(v[j] - m) : 0.0f;
            s += v[j];
        }
        s = wave_sum(s);
        const float inv = s > 0.0f ? 1.0f / s : 1.0f;
#pragma unroll
        for (int j = 0; j < R; ++j) {
            const uint32_t i = (uint32_t)j * kWave + (uint32_t)lane;
            if (i < width) put(i, v[j] * inv);
        }
        return;
    }
    float m = -3.402823466e+38f;
    for (uint32_t i = lane; i < width; i += kWave) m = fmaxf(m, p[i]);
    m = wave_max(m);
    float s = 0.0f;
    for (uint32_t i = lane; i < width; i += kWave) s += expf(p[i] - m);
    s = wave_sum(s);
    const float inv = s > 0.0f ? 1.0f / s : 1.0f;
    for (uint32_t i = lane; i < width; i += kWave) put(i, expf(p[i] - m) * inv);
}

// FP32 -> 16-bit activations for the first GEMM layer
template <bool F16T>
__global__ __launch_bounds__(256) void sp_cvt16(const float *__restrict__ in, uint16_t *__restrict__ out, uint64_t n)
{
    uint64_t i = ((uint64_t)blockIdx.x * 256u + threadIdx.x) * 4u;
    if (i + 4 <= n) {
        float4 v = *reinterpret_cast<const float4 *>(in + i);
        uint2 o;
        o.x = (uint32_t)f32_to_t16<F16T>(v.x) | ((uint32_t)f32_to_t16<F16T>(v.y) << 16);
        o.y = (uint32_t)f32_to_t16<F16T>(v.z) | ((uint32_t)f32_to_t16<F16T>(v.w) << 16);
        *reinterpret_cast<uint2 *>(out + i) = o;
    } else {
        for (; i < n; ++i) out[i] = f32_to_t16<F16T>(in[i]);
    }
}

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
    float *ws;             // [splits][M][N] partial sums when the grid splits K (sp_gemm16_big only), else nullptr
    uint32_t kper;         // k range of one split, a multiple of 64 (0: all of K)
};

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

// Tile: BM x BN x 64, 256 threads = 2 x 2 waves, each wave TM x TN tiles of 32x32.
// LDS rows are padded by 8 elements so that 128-bit fragment reads of 32
// consecutive rows spread over the banks.
template <int FMT, bool F16T, int TM, int TN, bool ALIGNED>
__global__ __launch_bounds__(256) void sp_gemm16(const GemmArgs g)
{
    constexpr int BM = 64 * TM, BN = 64 * TN, BK = 64, LDK = BK + 8;
    constexpr int bits = fmt_bits(FMT);
    constexpr int EPL = 128 / bits;                 // weight elements per 16-byte load
    constexpr int W_LOADS = (BN * BK / EPL + 255) / 256;
    constexpr int A_LOADS = BM * BK / 8 / 256;

    __shared__ __attribute__((aligned(16))) uint16_t As[BM * LDK];
    __shared__ __attribute__((aligned(16))) uint16_t Ws[BN * LDK];

    const uint32_t M = g.M, N = g.L.N, K = g.L.K;
    const int t = threadIdx.x, lane = t & 63, wave = t >> 6;
    const int wm = wave >> 1, wn = wave & 1;

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

    uint4 ra[A_LOADS], rw[W_LOADS];
    const size_t w_row_bytes = (size_t)K * bits / 8u;

    auto load_tiles = [&](uint32_t k0) {
        if constexpr (ALIGNED) {
#pragma unroll
            for (int i = 0; i < A_LOADS; ++i) {
                const int c = t + 256 * i, row = c >> 3, kc = c & 7;
                const uint32_t m = m0 + row < M ? m0 + row : M - 1;
                const uint32_t k = k0 + kc * 8;
                ra[i] = k < K ? *reinterpret_cast<const uint4 *>(g.A + (size_t)m * K + k) : make_uint4(0, 0, 0, 0);
            }
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
    };

    auto store_tiles = [&](uint32_t k0) {
        if constexpr (ALIGNED) {
#pragma unroll
            for (int i = 0; i < A_LOADS; ++i) {
                const int c = t + 256 * i, row = c >> 3, kc = c & 7;
                *reinterpret_cast<uint4 *>(&As[row * LDK + kc * 8]) = ra[i];
            }
#pragma unroll
            for (int i = 0; i < W_LOADS; ++i) {
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
                As[row * LDK + kk] = (m < M && k < K) ? g.A[(size_t)m * K + k] : (uint16_t)0;
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

    const uint32_t ktiles = (K + BK - 1) / BK;
    load_tiles(0);
    for (uint32_t kt = 0; kt < ktiles; ++kt) {
        __syncthreads();                              // previous tile fully consumed
        store_tiles(kt * BK);
        __syncthreads();
        if (kt + 1 < ktiles) load_tiles((kt + 1) * BK);

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

    // epilogue: scale, bias, activation, store
    const float wscale = g.L.wscale;
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
                const float v = apply_act(fmaf(acc[i][j][r], wscale, bias), g.L.act);
                const size_t o = (size_t)row * N + col;
                if (g.out_f32) reinterpret_cast<float *>(g.C)[o] = v;
                else reinterpret_cast<uint16_t *>(g.C)[o] = f32_to_t16<F16T>(v);
            }
        }
    }
}

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

// f(integral_constant<int, 0>) ... f(integral_constant<int, N - 1>)
template <int N, int I = 0, class F>
__device__ __forceinline__ void static_for(F &&f)
{
    if constexpr (I < N) {
        f(std::integral_constant<int, I>{});
        static_for<N, I + 1>(f);
    }
}

template <int OFF>
__device__ __forceinline__ void ds_read128(u32x4 &dst, uint32_t addr);

// 16 bytes per lane from global memory straight into LDS (wave-contiguous 1 KiB at lds_addr):
// scalar base + 32-bit lane offset, so issuing it costs no vector-ALU instruction.  The compiler
// does not track these loads: the caller waits with s_waitcnt vmcnt before the data is read.
__device__ __forceinline__ void lds_dma16(uint32_t lds_addr, uint32_t voff, const void *sbase)
{
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
// Large-tile variant of the 16-bit MFMA GEMM (K a multiple of 64, rows 16-byte
// aligned).  WM x WN waves, each TM x TN tiles of 32x32; BK = 64.
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

    // tile order: each XCD (workgroup id mod 8) gets a contiguous run of tiles; inside
    // the run, 8 row tiles x 4 column tiles are consecutive so that the 32 workgroups
    // an XCD runs at once share A rows and W rows in its L2
    const uint32_t tiles_n = (N + BN - 1) / BN, tiles_m = (M + BM - 1) / BM;
    const uint32_t ntiles = tiles_m * tiles_n;
    uint32_t bid = blockIdx.x;
    {
        const uint32_t per = ntiles / 8u;
        if (bid < per * 8u) bid = (bid & 7u) * per + (bid >> 3);
    }
    uint32_t tm, tn;
    {
        constexpr uint32_t GM = 8;
        const uint32_t group = bid / (GM * tiles_n);
        const uint32_t first = group * GM;
        const uint32_t rows = tiles_m - first < GM ? tiles_m - first : GM;
        const uint32_t in = bid - group * GM * tiles_n;
        tm = first + in % rows;
        tn = in / rows;
    }
    const uint32_t m0 = tm * BM, n0 = tn * BN;

    f32x16 acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.0f;

    // LDS-DMA sources: a uniform base (advanced per K tile on the scalar unit) plus a fixed 32-bit
    // byte offset per lane and issue, and LDS destinations derived from a scalar wave index: the main
    // loop then issues its loads without any vector-ALU instruction, which would otherwise queue
    // behind the other wave's MFMAs
    const int wave_s = __builtin_amdgcn_readfirstlane(wave);
    // Only the first wave of each SIMD (waves 0 .. NWAVES/2-1, which the issue arbiter serves first)
    // issues the loads, for itself and for wave + NWAVES/2: a wave stalls while the address unit takes
    // its load, and the other wave of the SIMD keeps the MFMA pipe fed meanwhile.
    constexpr int HALF = NWAVES / 2;
    constexpr int A_DUTY = 2 * A_ISSUES, W_DUTY = W_DIRECT ? 2 * W_ISSUES : 1;
    uint32_t a_voff[A_DUTY], w_voff[W_DUTY];
#pragma unroll
    for (int d = 0; d < A_DUTY; ++d) {
        const int i = d >> 1, wv = (wave & (HALF - 1)) + (d & 1) * HALF;
        const int ci = (i * NWAVES + wv) * 64 + lane, row = ci >> 3, pos = ci & 7;
        const uint32_t m = m0 + row < M ? m0 + row : M - 1;
        a_voff[d] = (uint32_t)(((size_t)m * K + ((pos ^ ((row >> 1) & 7)) << 3)) * 2u);
    }
    if constexpr (W_DIRECT) {
#pragma unroll
        for (int d = 0; d < W_DUTY; ++d) {
            const int i = d >> 1, wv = (wave & (HALF - 1)) + (d & 1) * HALF;
            const int ci = (i * NWAVES + wv) * 64 + lane, row = ci >> 3, pos = ci & 7;
            const uint32_t n = n0 + row < N ? n0 + row : N - 1;
            w_voff[d] = (uint32_t)(((size_t)n * K + ((pos ^ ((row >> 1) & 7)) << 3)) * 2u);
        }
    }
    const char *a_base = reinterpret_cast<const char *>(g.A);
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
                lds_dma16(lds_a + (uint32_t)(buf * BM * BK * 2 + ((d >> 1) * NWAVES + (d & 1) * HALF) * 1024), a_voff[d],
                          a_base + (size_t)k0 * 2u);
        if constexpr (W_DIRECT) {
#pragma unroll
            for (int d = 0; d < W_DUTY; ++d)
                if (A_DUTY + d == idx)
                    lds_dma16(lds_w + (uint32_t)(buf * BN * BK * 2 + ((d >> 1) * NWAVES + (d & 1) * HALF) * 1024), w_voff[d],
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
    const uint32_t kbeg = g.kper ? blockIdx.y * g.kper : 0u;
    const uint32_t kend = g.kper && kbeg + g.kper < K ? kbeg + g.kper : K;
    const uint32_t ktiles = (kend - kbeg) / BK;
    issue_direct(0, kbeg);
    load_w_regs(kbeg);
    store_w_regs(0);
    asm volatile("s_waitcnt vmcnt(0)");
    __syncthreads();
    for (uint32_t kt = 0; kt < ktiles; kt += 2) {
        stage(std::integral_constant<int, 0>{}, kt + 1 < ktiles, kbeg + (kt + 1) * BK);
        if (kt + 1 < ktiles) stage(std::integral_constant<int, 1>{}, kt + 2 < ktiles, kbeg + (kt + 2) * BK);
    }
    if (g.ws) {
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

// adds the K splits of sp_gemm16_big (in split order) and applies scale, bias and activation
template <bool F16T>
__global__ __launch_bounds__(256) void sp_gemm16_reduce(const GemmArgs g, uint32_t splits)
{
    const uint64_t idx = (uint64_t)blockIdx.x * 256u + threadIdx.x;
    const uint64_t total = (uint64_t)g.M * g.L.N;
    if (idx >= total) return;
    float sum = 0.0f;
    for (uint32_t sp = 0; sp < splits; ++sp) sum += g.ws[(uint64_t)sp * total + idx];
    const uint32_t col = (uint32_t)(idx % g.L.N);
    const float bias = elem_value_rt(g.L.bias_fmt, g.L.bias, col) * g.L.bscale;
    const float v = apply_act(fmaf(sum, g.L.wscale, bias), g.L.act);
    if (g.out_f32) reinterpret_cast<float *>(g.C)[idx] = v;
    else reinterpret_cast<uint16_t *>(g.C)[idx] = f32_to_t16<F16T>(v);
}

// ---------------------------------------------------------------------------
// Streaming MFMA kernel for layers with one thin side
// ---------------------------------------------------------------------------
// Few samples (5 .. 256) or few outputs (<= 64): one operand is a tall matrix that is
// read exactly once (the weights, or the 16-bit activations when the layer has few
// outputs), the other a thin 16-bit matrix of at most 64 rows per workgroup.  The tall
// operand never touches LDS: a wave owns RT tiles of 32 streamed rows and loads them
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

template <bool F16T>
__device__ __forceinline__ void skinny_emit(const SkinnyArgs &a, uint32_t c, uint32_t r, float accv)
{
    const uint32_t m = a.mode_b ? r : c, n = a.mode_b ? c : r;
    const float bias = elem_value_rt(a.L.bias_fmt, a.L.bias, n) * a.L.bscale;
    const float v = apply_act(fmaf(accv, a.L.wscale, bias), a.L.act);
    const size_t o = (size_t)m * a.L.N + n;
    if (a.out_f32) reinterpret_cast<float *>(a.C)[o] = v;
    else reinterpret_cast<uint16_t *>(a.C)[o] = f32_to_t16<F16T>(v);
}

// 16 bytes per lane from scalar base + 32-bit lane offset + immediate.  Inline assembly: the compiler's
// wait-count bookkeeping does not see the load, the caller waits with s_waitcnt vmcnt before using dst.
template <int OFF>
__device__ __forceinline__ void load16_async(u32x4 &dst, uint32_t voff, const void *sbase)
{
    asm volatile("global_load_dwordx4 %0, %1, %2 offset:%3" : "=v"(dst) : "v"(voff), "s"(sbase), "n"(OFF) : "memory");
}

template <int FMT, bool F16T, int RT, int CT>
__global__ __launch_bounds__(256) void sp_skinny16(const SkinnyArgs a)
{
    using F = SkinnyFmt<FMT>;
    constexpr int EPL = F::EPL, LPC = F::LPC, BKC = F::BKC, STEPS = F::STEPS, PITCH = F::PITCH;
    constexpr int UNITS = 32 * CT * (BKC / 16);            // 16-code units of a thin chunk
    constexpr int UPT = (UNITS + 255) / 256;
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
    const uint32_t row0 = (rblk * 4u + (uint32_t)wave) * (32u * RT);
    const uint32_t cbase = cblk * (32u * CT);
    const uint32_t kbeg = blockIdx.y * a.kper;
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
        const uint32_t u = (uint32_t)t + 256u * q;
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
            const uint8_t *sb = a.stream + (size_t)(kbeg + ch * BKC) * F::bits / 8u;
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
                for (int rt = 0; rt < RT; ++rt) load16_async<0>(dst[rt][i], svoff[rt] + add, a.stream);
            }
        }
    };
    u32x4 thin_regs[UPT][2];
    auto issue_thin = [&](uint32_t ch) {
        if (ch < last_chunk) {
            const uint16_t *tb = a.thin + (kbeg + ch * BKC);
#pragma unroll
            for (int q = 0; q < UPT; ++q)
#pragma unroll
                for (int e = 0; e < 2; ++e) load16_async<0>(thin_regs[q][e], tvoff[q][e], tb);
        } else {
            const uint32_t kc0 = kbeg + last_chunk * BKC;
#pragma unroll
            for (int q = 0; q < UPT; ++q) {
                const uint32_t uc = ((uint32_t)t + 256u * q) % (BKC / 16);
#pragma unroll
                for (int e = 0; e < 2; ++e) {
                    const bool valid = trow_ok[q] && kc0 + uc * 16u + 8u * e + 8u <= kend;
                    load16_async<0>(thin_regs[q][e], valid ? tvoff[q][e] + kc0 * 2u : 0u, a.thin);
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
            const uint32_t u = (uint32_t)t + 256u * q;
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
#pragma unroll
    for (int rt = 0; rt < RT; ++rt) {
        const uint32_t r = row0 + rt * 32u + n31;
        if (r >= a.R) continue;
#pragma unroll
        for (int ct = 0; ct < CT; ++ct)
#pragma unroll
            for (int q = 0; q < 16; ++q) {
                const uint32_t c = cbase + ct * 32u + 8u * (q >> 2) + 4u * h + (q & 3);
                if (c >= a.NC) continue;
                if (a.ws) a.ws[((size_t)blockIdx.y * a.NC + c) * a.R + r] = acc[rt][ct][q];
                else skinny_emit<F16T>(a, c, r, acc[rt][ct][q]);
            }
    }
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
    const uint32_t kbeg = blockIdx.y * a.kper;
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
            const uint8_t *sb = a.stream + (size_t)(kbeg + ch * BKC) * F::bits / 8u;
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
                load16_async<0>(dst[j], svoff + add, a.stream);
            }
        }
    };
    u32x4 thin_regs[UPL][2];
    auto issue_thin = [&](uint32_t i) {
        const uint32_t ch = chunk_of(i);
        if (ch < last_chunk) {
            const uint16_t *tb = a.thin + (kbeg + ch * BKC);
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
                    load16_async<0>(thin_regs[q][e], valid ? tvoff[q][e] + kc0 * 2u : 0u, a.thin);
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

// adds the K splits of sp_skinny16 and applies bias and activation
template <bool F16T>
__global__ __launch_bounds__(256) void sp_skinny_reduce(const SkinnyArgs a, uint32_t splits)
{
    const uint64_t idx = (uint64_t)blockIdx.x * 256u + threadIdx.x;
    const uint64_t total = (uint64_t)a.NC * a.R;
    if (idx >= total) return;
    float sum = 0.0f;
    for (uint32_t sp = 0; sp < splits; ++sp) sum += a.ws[(uint64_t)sp * total + idx];
    skinny_emit<F16T>(a, (uint32_t)(idx / a.R), (uint32_t)(idx % a.R), sum);
}

// unscaled integer codes of a small weight array as FP16 (the thin operand of a layer with few outputs)
template <int FMT>
__global__ __launch_bounds__(256) void sp_codes16(const uint8_t *__restrict__ codes, uint16_t *__restrict__ out, uint64_t n)
{
    const uint64_t i = (uint64_t)blockIdx.x * 256u + threadIdx.x;
    if (i < n) out[i] = f32_to_f16_sat(elem_value<FMT>(codes, i));
}

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
    const uint32_t m0 = (blockIdx.x / tiles_n) * BM, n0 = (blockIdx.x % tiles_n) * BN;
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

// ---------------------------------------------------------------------------
// small copies (host staging of single-sample forwards)
// ---------------------------------------------------------------------------
__global__ __launch_bounds__(256) void sp_copy32(const float *__restrict__ src, float *__restrict__ dst, uint64_t n)
{
    const uint64_t i = (uint64_t)blockIdx.x * 256u + threadIdx.x;
    if (i < n) dst[i] = src[i];
}

// gathers up to 16 layer slots (16-byte aligned starts) into the dense neurons layout
struct PackArgs {
    const float *src;
    float *dst;
    uint32_t count;
    uint32_t src_off[16], dst_off[16], len[16];
};

__global__ __launch_bounds__(256) void sp_pack_layers(const PackArgs a)
{
    const uint32_t s = blockIdx.y;
    if (s >= a.count) return;
    for (uint32_t i = blockIdx.x * 256u + threadIdx.x; i < a.len[s]; i += gridDim.x * 256u)
        a.dst[a.dst_off[s] + i] = a.src[a.src_off[s] + i];
}

// ---------------------------------------------------------------------------
// evaluation of a batch of outputs (compute_sample_loss, SIMD.c:522-552;
// batch_compute_loss, Training.c:421-435): one wave per sample
// ---------------------------------------------------------------------------
struct EvalArgs {
    const float *y;        // [n][width] outputs
    const float *target;   // [n][width]
    float *loss;           // [n] per-sample loss
    uint32_t *pred;        // [n] index of the first largest output
    uint32_t *hit;         // [n] 1 when the target's first largest entry has the same index
    uint32_t n, width;
    int loss_func;         // 0 sum of squared differences, 1 cross-entropy
    int sigmoid_out;       // cross-entropy in its binary form (output layer is a sigmoid)
};

__global__ __launch_bounds__(256) void sp_eval_rows(const EvalArgs a)
{
    const int lane = threadIdx.x & 63;
    const uint32_t row = blockIdx.x * 4u + (threadIdx.x >> 6);
    if (row >= a.n) return;
    const float *o = a.y + (size_t)row * a.width, *tg = a.target + (size_t)row * a.width;
    const float eps = 1e-9f;
    float acc = 0.0f;
    float bo = -__builtin_inff(), bt = -__builtin_inff();
    uint32_t io = 0xFFFFFFFFu, it = 0xFFFFFFFFu;
    for (uint32_t k = lane; k < a.width; k += kWave) {
        const float ov = o[k], tv = tg[k];
        if (a.loss_func == 0) {
            const float d = ov - tv;
            acc += d * d;
        } else if (a.sigmoid_out) {
            float c = ov < eps ? eps : ov;
            c = c > 1.0f - eps ? 1.0f - eps : c;
            acc -= tv * logf(c) + (1.0f - tv) * logf(1.0f - c);
        } else {
            const float c = ov < eps ? eps : ov;
            acc -= tv * logf(c);
        }
        if (ov > bo || io == 0xFFFFFFFFu) { bo = ov; io = k; }
        if (tv > bt || it == 0xFFFFFFFFu) { bt = tv; it = k; }
    }
    acc = wave_sum(acc);
    // first largest element: larger value wins, equal values keep the lower index
#pragma unroll
    for (int s = 32; s > 0; s >>= 1) {
        const float vo = __shfl_xor(bo, s, kWave), vt = __shfl_xor(bt, s, kWave);
        const uint32_t jo = __shfl_xor(io, s, kWave), jt = __shfl_xor(it, s, kWave);
        if (jo != 0xFFFFFFFFu && (io == 0xFFFFFFFFu || vo > bo || (vo == bo && jo < io))) { bo = vo; io = jo; }
        if (jt != 0xFFFFFFFFu && (it == 0xFFFFFFFFu || vt > bt || (vt == bt && jt < it))) { bt = vt; it = jt; }
    }
    if (lane == 0) {
        a.loss[row] = acc;
        a.pred[row] = io;
        a.hit[row] = io == it ? 1u : 0u;
    }
}

// one workgroup: total loss (added in FP64) and number of hits
__global__ __launch_bounds__(1024) void sp_eval_total(const float *loss, const uint32_t *hit, uint32_t n, double *out_loss,
                                                      uint32_t *out_hits)
{
    __shared__ double s_l[16];
    __shared__ uint32_t s_h[16];
    double l = 0.0;
    uint32_t h = 0;
    for (uint32_t i = threadIdx.x; i < n; i += 1024u) { l += (double)loss[i]; h += hit[i]; }
#pragma unroll
    for (int s = 32; s > 0; s >>= 1) { l += __shfl_xor(l, s, kWave); h += __shfl_xor(h, s, kWave); }
    if ((threadIdx.x & 63) == 0) { s_l[threadIdx.x >> 6] = l; s_h[threadIdx.x >> 6] = h; }
    __syncthreads();
    if (threadIdx.x == 0) {
        double tl = 0.0;
        uint32_t th = 0;
        for (int w = 0; w < 16; ++w) { tl += s_l[w]; th += s_h[w]; }
        *out_loss = tl;
        *out_hits = th;
    }
}

}  // namespace

// ---------------------------------------------------------------------------
// host side
// ---------------------------------------------------------------------------
struct DevArray {
    uint8_t *base = nullptr;       // allocation (256-byte aligned by hipMalloc)
    size_t bytes = 0;
    uint64_t count = 0;
    float max_val = 0.0f;
    bool uploaded = false;
    uint16_t *codes16 = nullptr;   // weights of a layer with few outputs: unscaled codes as FP16 (made on demand)
    bool codes16_valid = false;
};

struct sphip_train_state;

struct sphip_net {
    uint32_t layers = 0;
    std::vector<uint32_t> topo;
    std::vector<uint8_t> act;
    int prec = 0;
    std::vector<DevArray> W, B;    // [layers-1]
    // workspace, grown on demand
    uint64_t cap_elems = 0;        // capacity of each ping-pong buffer in FP32 elements
    void *buf[2] = {nullptr, nullptr};
    uint8_t *aq = nullptr;         // digit planes of the current layer input (integer GEMV)
    float *aq_inv = nullptr;
    int *aq_dsum = nullptr;
    uint32_t aq_valid_layer = 0, aq_valid_n = 0;   // which layer input the planes describe (layer-only timing)
    uint32_t aq_cap_n = 0;
    float *soft_tmp = nullptr;     // FP32 logits of a softmax layer
    uint64_t soft_cap = 0;
    float *layers_buf = nullptr;   // all activations of a single-sample forward, each layer at a 16-byte aligned slot
    std::vector<uint32_t> slot_off;  // start of each layer's slot (floats)
    uint64_t slots_total = 0;
    float *pin_in = nullptr, *pin_out = nullptr;   // pinned host staging of small inputs / outputs
    uint64_t pin_in_cap = 0, pin_out_cap = 0;
    float *stage_x = nullptr;      // device staging of host inputs / outputs
    float *stage_y = nullptr;
    uint64_t stage_x_cap = 0, stage_y_cap = 0;
    uint32_t max_width = 0;
    uint64_t total_neurons = 0;
    float *split_ws = nullptr;     // partial sums of the K splits of the thin-operand kernel
    uint64_t split_cap = 0;
    float *eval_buf = nullptr;     // evaluation: outputs, staged targets, per-sample loss / prediction / hit, totals
    uint64_t eval_cap = 0;
    sphip_train_state *train = nullptr;   // gradients, optimizer moments, kept activations (training only)
};

namespace {

void train_free(sphip_net *net);

enum Regime { R_GEMV, R_GEMM16, R_GEMM32 };

Regime pick_regime(const sphip_net *net, uint32_t n, uint32_t flags)
{
    if ((flags & SPHIP_FORCE_GEMV) && n <= 64) return R_GEMV;
    if (flags & SPHIP_FORCE_GEMM) return net->prec == F32 ? R_GEMM32 : R_GEMM16;
    if (net->prec == F32) return n <= 64 ? R_GEMV : R_GEMM32;
    return n <= 4 ? R_GEMV : R_GEMM16;
}

LayerArgs make_layer_args(const sphip_net *net, uint32_t l /*1-based layer*/)
{
    LayerArgs L{};
    const DevArray &w = net->W[l - 1], &b = net->B[l - 1];
    L.w = w.base;
    L.bias = b.base;
    L.wscale = fmt_scale(net->prec, w.max_val);
    L.bscale = fmt_scale(net->prec, b.max_val);
    L.bias_fmt = net->prec;
    L.act = net->act[l - 1] == A_SOFTMAX ? A_NONE : net->act[l - 1];
    L.N = net->topo[l];
    L.K = net->topo[l - 1];
    return L;
}

bool rows_aligned(int fmt, uint32_t K) { return ((uint64_t)K * (uint64_t)fmt_bits(fmt)) % 128u == 0; }

template <int FMT>
void launch_gemv_fmt(const LayerArgs &L, const float *x, float *y, uint32_t n)
{
    const bool aligned = rows_aligned(FMT, L.K) && (L.K % 4u == 0);
    for (uint32_t b0 = 0; b0 < n; b0 += 8) {
        const int nb = (int)(n - b0 < 8 ? n - b0 : 8);
        const float *xb = x + (size_t)b0 * L.K;
        float *yb = y + (size_t)b0 * L.N;
        g_last_kernel = aligned ? "sp_gemv" : "sp_gemv_generic";
        if (aligned) {
            constexpr int R = 2;
            const uint32_t waves = (L.N + R - 1) / R, grid = (waves + 3) / 4;
            if (nb == 1) sp_gemv<FMT, 1, R><<<grid, 256, 0, g_stream>>>(L, xb, yb, nb);
            else if (nb == 2) sp_gemv<FMT, 2, R><<<grid, 256, 0, g_stream>>>(L, xb, yb, nb);
            else if (nb <= 4) sp_gemv<FMT, 4, R><<<grid, 256, 0, g_stream>>>(L, xb, yb, nb);
            else sp_gemv<FMT, 8, R><<<grid, 256, 0, g_stream>>>(L, xb, yb, nb);
        } else {
            const uint32_t grid = (L.N + 3) / 4;
            if (nb == 1) sp_gemv_generic<FMT, 1><<<grid, 256, 0, g_stream>>>(L, xb, yb, nb);
            else if (nb <= 4) sp_gemv_generic<FMT, 4><<<grid, 256, 0, g_stream>>>(L, xb, yb, nb);
            else sp_gemv_generic<FMT, 8><<<grid, 256, 0, g_stream>>>(L, xb, yb, nb);
        }
    }
}

template <int FMT, int MT, int FQ = 0>
void launch_gemv_i8_mt(const GemvI8Args &a, uint32_t grid_x, uint32_t threads, size_t lds)
{
    auto kern = sp_gemv_i8mfma<FMT, MT, FQ>;
    static bool once = ((void)hipFuncSetAttribute((const void *)kern, hipFuncAttributeMaxDynamicSharedMemorySize, 156 * 1024), true);
    (void)once;
    kern<<<grid_x, threads, lds, g_stream>>>(a);
}

// Integer formats with 16-byte aligned rows go to the INT8 matrix cores:
// one quantise launch for the layer's input, then the GEMV proper.
template <int FMT>
bool launch_gemv_i8(const sphip_net *net, const LayerArgs &L, const float *x, float *y, uint32_t n, bool main_only)
{
    constexpr int KL = I8Fmt<FMT>::KL;
    if (!rows_aligned(FMT, L.K) || L.K < (uint32_t)KL || !net->aq) return false;
    if (reinterpret_cast<uintptr_t>(x) & 15u) return false;   // the quantiser reads float4
    const int need = (int)(n + 3) / 4;
    const int MT = need <= 1 ? 1 : need <= 2 ? 2 : need <= 3 ? 3 : need <= 4 ? 4 : need <= 6 ? 6 : need <= 8 ? 8 : need <= 12 ? 12 : 16;
    GemvI8Args a{};
    a.L = L; a.x = x; a.y = y; a.nb = (int)n;
    a.aq = net->aq; a.inv = net->aq_inv; a.dsum = net->aq_dsum;
    // waves of a workgroup: rw row groups (sharing the digit planes) x ks K shares
    const uint32_t wave_rows = (L.N + 15) / 16;
    const uint32_t kblocks = (L.K + KL - 1) / KL;
    const uint32_t blk_bytes = (uint32_t)I8Fmt<FMT>::NMF * 4u * n * 48u;
    const uint32_t budget = kGemvStageBytes;
    const uint32_t max_waves = MT > 4 ? 4u : 16u;             // register budget of the wide tiles
    // up to four samples: the GEMV workgroups quantise the activations themselves
    const bool fused = MT == 1;
    const uint32_t ks_cap = 2048u / (4u * KL);                 // a scale chunk is a whole number of fetch groups
                                                               // and at most 2048 codes (one wave's batch of loads)
    uint32_t rw, ks;
    if (fused) {
        // about eight waves per compute unit in all; eight-wave workgroups unless that leaves fewer
        // workgroups than compute units
        ks = 2048u / wave_rows;
        ks = ks >= 8u ? 8u : ks >= 4u ? 4u : ks >= 2u ? 2u : 1u;
        if (ks > ks_cap) ks = ks_cap;
        rw = 8u / ks;
        while (rw > 1 && wave_rows / rw < 256u) rw >>= 1;
    } else {
        // the planes cost 3 n bytes per column and workgroup, the weights 2 bits-per-code bytes per
        // column and row group: more row groups per workgroup as n grows or the codes shrink
        rw = (3u * n + (uint32_t)I8Fmt<FMT>::bits - 1) / (uint32_t)I8Fmt<FMT>::bits;
        rw = rw >= 4 ? 4u : rw >= 2 ? 2u : 1u;
        while (rw > 1 && wave_rows / rw < 512u) rw >>= 1;      // keep the grid at least twice the chip
        ks = max_waves / rw > 8u ? 8u : max_waves / rw;
        if (ks > ks_cap) ks = ks_cap;
    }
    // one fetch group (4 blocks of every K share) must fit the row, the stage budget and one scale chunk
    while (ks > 1 && (kblocks < 4u * ks || 4u * ks * blk_bytes > budget)) ks >>= 1;
    const uint32_t group_blocks = 4u * ks;
    // scale chunk: about 2048 codes, a whole number of fetch groups, and small enough for one LDS stage
    uint32_t kc_blocks = 2048u / KL;
    if (kc_blocks > budget / blk_bytes) kc_blocks = budget / blk_bytes;
    kc_blocks = kc_blocks / group_blocks * group_blocks;
    if (kc_blocks == 0) kc_blocks = group_blocks;
    a.kc = kc_blocks * KL;
    a.nchunks = (kblocks + kc_blocks - 1) / kc_blocks;
    a.meta_bytes = a.nchunks * n * 16u;
    if ((uint64_t)kc_blocks * blk_bytes + a.meta_bytes > 156u * 1024u) return false;
    const uint32_t nblocks = a.nchunks * kc_blocks;
    // LDS stage: everything if it fits the budget, else whole scale chunks
    uint32_t stage = nblocks;
    if ((uint64_t)nblocks * blk_bytes > budget) {
        stage = (budget / blk_bytes) / kc_blocks * kc_blocks;
        if (stage == 0) stage = kc_blocks;
    }
    a.stage_blocks = stage;
    a.rw = rw;
    a.ks = ks;
    const uint32_t waves = rw * ks;
    const uint32_t grid = (wave_rows + rw - 1) / rw;
    size_t lds = (size_t)stage * blk_bytes;
    const size_t red_bytes = (size_t)waves * MT * 64u * sizeof(float);
    if (lds < red_bytes) lds = red_bytes;
    lds += a.meta_bytes;
    g_last_kernel = "sp_gemv_i8mfma";
    if (fused) {
        // samples one wave quantises at once: as many as still leave every wave a unit of work
        const uint32_t cps = stage / kc_blocks;
        uint32_t ns = 4;
        while (ns > 1 && (ns / 2 >= n || cps * ((n + ns - 1) / ns) < waves)) ns >>= 1;
        if (ns == 1) launch_gemv_i8_mt<FMT, 1, 1>(a, grid, waves * 64, lds);
        else if (ns == 2) launch_gemv_i8_mt<FMT, 1, 2>(a, grid, waves * 64, lds);
        else launch_gemv_i8_mt<FMT, 1, 4>(a, grid, waves * 64, lds);
        return true;
    }
    if (!main_only) sp_quant_x<FMT><<<(a.nchunks * n + 3u) / 4u, 256, 0, g_stream>>>(a);
    switch (MT) {
    case 1:  launch_gemv_i8_mt<FMT, 1>(a, grid, waves * 64, lds); break;
    case 2:  launch_gemv_i8_mt<FMT, 2>(a, grid, waves * 64, lds); break;
    case 3:  launch_gemv_i8_mt<FMT, 3>(a, grid, waves * 64, lds); break;
    case 4:  launch_gemv_i8_mt<FMT, 4>(a, grid, waves * 64, lds); break;
    case 6:  launch_gemv_i8_mt<FMT, 6>(a, grid, waves * 64, lds); break;
    case 8:  launch_gemv_i8_mt<FMT, 8>(a, grid, waves * 64, lds); break;
    case 12: launch_gemv_i8_mt<FMT, 12>(a, grid, waves * 64, lds); break;
    default: launch_gemv_i8_mt<FMT, 16>(a, grid, waves * 64, lds); break;
    }
    return true;
}

void launch_gemv(const sphip_net *net, const LayerArgs &L, const float *x, float *y, uint32_t n, bool main_only)
{
    switch (net->prec) {
    case F32:  launch_gemv_fmt<F32>(L, x, y, n); break;
    case F16:  launch_gemv_fmt<F16>(L, x, y, n); break;
    case BF16: launch_gemv_fmt<BF16>(L, x, y, n); break;
    case I8:   if (!launch_gemv_i8<I8>(net, L, x, y, n, main_only)) launch_gemv_fmt<I8>(L, x, y, n); break;
    case I4:   if (!launch_gemv_i8<I4>(net, L, x, y, n, main_only)) launch_gemv_fmt<I4>(L, x, y, n); break;
    default:   if (!launch_gemv_i8<I2>(net, L, x, y, n, main_only)) launch_gemv_fmt<I2>(L, x, y, n); break;
    }
}

// K splits of the 256 x 256 GEMM when its tiles would leave compute units idle: at least eight K tiles each
// Rows of a tile of the big GEMM: up to 128 samples a single row of 128 x 256 tiles instead of half-empty 256 x 256
// ones; for larger batches the smaller tile was measured and is no faster (256 to 2048 samples, 8192-wide layers).
uint32_t gemm16_tile_rows(uint32_t M)
{
    return M <= 128u ? 128u : 256u;
}

uint32_t gemm16_splits(uint32_t M, uint32_t N, uint32_t K, uint32_t *kper)
{
    const uint32_t bm = gemm16_tile_rows(M);
    const uint32_t tiles = ((M + bm - 1) / bm) * ((N + 255u) / 256u), ktiles = K / 64u;
    *kper = 0;
    if (tiles >= 192u || ktiles < 16u) return 1;
    uint32_t splits = (256u + tiles - 1) / tiles;
    if (splits > 8u) splits = 8u;
    if (splits > ktiles / 8u) splits = ktiles / 8u;
    if (splits <= 1u) return 1;
    const uint32_t per = (ktiles + splits - 1) / splits;
    *kper = per * 64u;
    return (ktiles + per - 1) / per;
}

// What the thin-operand kernel needs beyond the layer itself
struct ThinCtx {
    const uint16_t *w16;   // [N][K] 16-bit weights (raw 16-bit formats, or FP16 codes) when N <= 64, else nullptr
    float *ws;             // split-K workspace
    uint64_t ws_floats;
};

struct ThinPlan {
    bool use;
    bool mode_b;
    bool kw;               // thin operand of <= 8 rows: K split among the waves of a workgroup (sp_skinny16_kw)
    int ncp;               // thin rows held in LDS in that case
    int nw;                // waves per workgroup in that case (4 or 8)
    uint32_t R, NC;        // streamed rows, thin rows
    int rt, ct;
    uint32_t splits, kper, row_blocks, cblocks;
};

// Largest batch the weight-streaming kernel takes before the tiled GEMM does better (which runs from 65 samples up, a
// partly filled row of 256 x 256 tiles).  Measured on whole nets: 8192-wide BF16 layers 417 / 439 / 475 us at 72 / 96 /
// 128 samples through the GEMM against 468 / 486 / 502 us streaming (and 576 against 918 us at 256); 16384-wide INT4
// 281 / 305 us at 192 / 256 against 366 / 369 us, but 257 / 263 us at 96 / 128 against 213 / 233 us; 8192-wide INT2 still
// 8 % better streaming at 256.  The fewer bytes a code has, the longer re-reading the weights per block of 64 samples pays.
// Layers of a few megabytes stay with the streaming kernel up to 256 samples (the 784-512-1000-10 INT8 net: 36 us
// against 57 us at 256 samples).
uint32_t thin_max_samples(int fmt, uint32_t N, uint32_t K)
{
    if ((uint64_t)N * K * (uint64_t)fmt_bits(fmt) / 8u <= (8ull << 20)) return 256u;
    return fmt_bits(fmt) == 16 ? 64u : fmt == I2 ? 256u : 128u;
}

// mode_b streams 16-bit activations (fmt = the activation type), mode a the weights
ThinPlan plan_thin(int fmt, uint32_t M, uint32_t N, uint32_t K)
{
    ThinPlan p{};
    if (N <= 64 && K % 8u == 0 && M >= 1) {
        p.use = true; p.mode_b = true; p.R = M; p.NC = N;
    } else if (M <= thin_max_samples(fmt, N, K) && rows_aligned(fmt, K) && K % 8u == 0) {
        p.use = true; p.mode_b = false; p.R = N; p.NC = M;
    } else {
        return p;
    }
    const int sfmt = p.mode_b ? F16 : fmt;
    // the kernel addresses both operands with 32-bit lane offsets
    if ((uint64_t)p.R * K * (uint64_t)fmt_bits(sfmt) / 8u >= (1ull << 32) || (uint64_t)p.NC * K * 2u >= (1ull << 32)) {
        p.use = false;
        return p;
    }
    const uint32_t bkc = sfmt == I8 ? 128u : (sfmt == I4 || sfmt == I2) ? 256u : 64u;
    // K split inside the workgroup (sp_skinny16_kw) for thin operands of at most 8 rows.  Every wave then fetches its
    // own thin chunks (four times the thin traffic, from L2), which pays where the second launch of the split-K path
    // weighs more: measured faster for INT8 at every size tried, for INT4 / INT2 up to 64 MB and for 16-bit operands
    // up to 32 MB of streamed bytes, slower beyond (16384 x 16384 INT4 at 8 samples: 40 us against 34 us).
    const uint64_t streamed_bytes = (uint64_t)p.R * K * (uint64_t)fmt_bits(sfmt) / 8u;
    const bool kw_pays = sfmt == I8 || streamed_bytes <= ((sfmt == I4 || sfmt == I2) ? (64ull << 20) : (32ull << 20));
    if (p.NC <= 8u && kw_pays) {
        // one workgroup per 32 streamed rows, its four waves share K; K is split across workgroups as well only
        // when the rows alone do not fill the chip
        p.kw = true;
        p.ncp = 8;
        p.rt = p.ct = 1;
        p.cblocks = 1;
        p.row_blocks = (p.R + 31u) / 32u;
        const uint32_t chunks = (K + bkc - 1) / bkc;
        // 6144 to 12287 streamed rows: eight waves per workgroup instead of a K split across two workgroups
        p.nw = (p.row_blocks >= 192u && p.row_blocks < 384u && chunks >= 16u) ? 8 : 4;
        uint32_t splits = p.row_blocks >= 192u ? 1u : (512u + p.row_blocks - 1) / p.row_blocks;
        if (splits > 16u) splits = 16u;
        if (splits > chunks / 4u) splits = chunks / 4u;
        if (splits < 1u) splits = 1u;
        const uint32_t cps = (chunks + splits - 1) / splits;
        p.kper = cps * bkc;
        p.splits = (chunks + cps - 1) / cps;
        return p;
    }
    p.ct = p.NC <= 32 ? 1 : 2;
    p.cblocks = (p.NC + 32u * p.ct - 1) / (32u * p.ct);
    p.rt = (p.R + 255u) / 256u * p.cblocks >= 128u ? 2 : 1;
    p.row_blocks = (p.R + 128u * p.rt - 1) / (128u * p.rt);
    const uint32_t chunks = (K + bkc - 1) / bkc;
    const uint32_t wgs = p.row_blocks * p.cblocks;
    uint32_t splits = (512u + wgs - 1) / wgs;
    if (splits > 16u) splits = 16u;
    if (splits > chunks / 2u) splits = chunks / 2u;
    if (splits < 1u) splits = 1u;
    const uint32_t cps = (chunks + splits - 1) / splits;
    p.kper = cps * bkc;
    p.splits = (chunks + cps - 1) / cps;
    return p;
}

template <int SFMT, bool F16T, int RT, int CT>
void launch_thin_inst(const SkinnyArgs &a, const ThinPlan &p)
{
    constexpr size_t lds = 2 * 32 * CT * SkinnyFmt<SFMT>::PITCH;
    auto kern = sp_skinny16<SFMT, F16T, RT, CT>;
    static bool once = ((void)hipFuncSetAttribute((const void *)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds), true);
    (void)once;
    const uint32_t gx = p.cblocks > 1 ? (p.row_blocks + 7u) / 8u * 8u * p.cblocks : p.row_blocks;
    kern<<<dim3(gx, p.splits, 1), 256, lds, g_stream>>>(a);
}

template <int SFMT, bool F16T, int NCP, int NW>
void launch_thin_kw(const SkinnyArgs &a, const ThinPlan &p)
{
    constexpr size_t lds = (size_t)NW * 2 * NCP * SkinnyFmt<SFMT>::PITCH + (size_t)NW * (NCP / 2) * 64 * sizeof(float);
    auto kern = sp_skinny16_kw<SFMT, F16T, NCP, NW>;
    static bool once = ((void)hipFuncSetAttribute((const void *)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds), true);
    (void)once;
    kern<<<dim3(p.row_blocks, p.splits, 1), 64 * NW, lds, g_stream>>>(a);
}

template <int SFMT, bool F16T>
void launch_thin(SkinnyArgs a, const ThinPlan &p)
{
    if (p.splits == 1) a.ws = nullptr;
    if (p.kw) {
        if (p.nw == 8) launch_thin_kw<SFMT, F16T, 8, 8>(a, p); else launch_thin_kw<SFMT, F16T, 8, 4>(a, p);
    } else if (p.rt == 2) {
        if (p.ct == 2) launch_thin_inst<SFMT, F16T, 2, 2>(a, p); else launch_thin_inst<SFMT, F16T, 2, 1>(a, p);
    } else {
        if (p.ct == 2) launch_thin_inst<SFMT, F16T, 1, 2>(a, p); else launch_thin_inst<SFMT, F16T, 1, 1>(a, p);
    }
    if (p.splits > 1) {
        const uint64_t total = (uint64_t)a.NC * a.R;
        sp_skinny_reduce<F16T><<<(uint32_t)((total + 255) / 256), 256, 0, g_stream>>>(a, p.splits);
    }
}

template <int FMT, bool F16T>
void launch_gemm16_fmt(const LayerArgs &L, const uint16_t *A, void *C, uint32_t M, int out_f32, const ThinCtx &ctx)
{
    const ThinPlan tp = plan_thin(FMT, M, L.N, L.K);
    if (tp.use && (!tp.mode_b || ctx.w16) && (tp.splits == 1 || (uint64_t)tp.splits * tp.NC * tp.R <= ctx.ws_floats)) {
        SkinnyArgs a{};
        a.L = L; a.C = C; a.ws = ctx.ws; a.R = tp.R; a.NC = tp.NC; a.row_blocks = tp.row_blocks; a.cblocks = tp.cblocks; a.kper = tp.kper; a.out_f32 = out_f32; a.mode_b = tp.mode_b ? 1 : 0;
        g_last_kernel = tp.kw ? "sp_skinny16_kw" : "sp_skinny16";
        if (tp.mode_b) {
            a.stream = reinterpret_cast<const uint8_t *>(A);
            a.thin = ctx.w16;
            launch_thin<F16T ? F16 : BF16, F16T>(a, tp);
        } else {
            a.stream = L.w;
            a.thin = A;
            launch_thin<FMT, F16T>(a, tp);
        }
        return;
    }
    GemmArgs g{L, A, C, M, out_f32, nullptr, 0};
    const bool aligned = rows_aligned(FMT, L.K) && (L.K % 8u == 0);
    const bool fits32 = (uint64_t)M * L.K * 2u < (1ull << 32) && (uint64_t)L.N * L.K * 2u < (1ull << 32);   // 32-bit DMA offsets
    // the 256 x 256 tiles need about a tile per compute unit; smaller problems fill the chip better with 128 x 128
    const uint32_t bm = gemm16_tile_rows(M);
    const uint32_t big_tiles = ((M + bm - 1) / bm) * ((L.N + 255u) / 256u);
    const uint32_t splits = gemm16_splits(M, L.N, L.K, &g.kper);
    const bool split_ok = splits > 1 && (uint64_t)splits * M * L.N <= ctx.ws_floats;
    if (aligned && L.K % 64u == 0 && M > 64 && L.N >= 256 && fits32 && (big_tiles >= 192u || split_ok)) {
        if (big_tiles >= 192u || !split_ok) g.kper = 0;
        else g.ws = ctx.ws;
        const dim3 grid(big_tiles, g.ws ? splits : 1u);
        g_last_kernel = "sp_gemm16_big";
        if (bm == 128u) {
            // a single row of tiles: 128 rows instead of 256 half-empty ones
            constexpr size_t lds = 2 * (128 + 256) * 64 * sizeof(uint16_t);
            auto kern = sp_gemm16_big<FMT, F16T, 2, 4, 2, 2>;
            static bool once = ((void)hipFuncSetAttribute((const void *)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds), true);
            (void)once;
            kern<<<grid, 512, lds, g_stream>>>(g);
        } else {
            constexpr size_t lds = 2 * (256 + 256) * 64 * sizeof(uint16_t);
            auto kern = sp_gemm16_big<FMT, F16T, 2, 4, 4, 2>;
            static bool once = ((void)hipFuncSetAttribute((const void *)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds), true);
            (void)once;
            kern<<<grid, 512, lds, g_stream>>>(g);
        }
        if (g.ws) sp_gemm16_reduce<F16T><<<(uint32_t)(((uint64_t)M * L.N + 255) / 256), 256, 0, g_stream>>>(g, splits);
        return;
    }
    g.kper = 0;
    g_last_kernel = "sp_gemm16";
    constexpr int TM = 2, TN = 2, BM = 64 * TM, BN = 64 * TN;
    const uint32_t grid = ((M + BM - 1) / BM) * ((L.N + BN - 1) / BN);
    if (aligned) sp_gemm16<FMT, F16T, TM, TN, true><<<grid, 256, 0, g_stream>>>(g);
    else sp_gemm16<FMT, F16T, TM, TN, false><<<grid, 256, 0, g_stream>>>(g);
}

void launch_gemm16(int fmt, const LayerArgs &L, const uint16_t *A, void *C, uint32_t M, int out_f32, const ThinCtx &ctx)
{
    switch (fmt) {
    case F16:  launch_gemm16_fmt<F16, true>(L, A, C, M, out_f32, ctx); break;
    case BF16: launch_gemm16_fmt<BF16, false>(L, A, C, M, out_f32, ctx); break;
    // integer codes are exact in either 16-bit type; FP16 keeps 11 bits of the activations instead of 8
    case I8:   launch_gemm16_fmt<I8, true>(L, A, C, M, out_f32, ctx); break;
    case I4:   launch_gemm16_fmt<I4, true>(L, A, C, M, out_f32, ctx); break;
    default:   launch_gemm16_fmt<I2, true>(L, A, C, M, out_f32, ctx); break;     // FP32 weights never come here
    }
}

// K splits of the FP32 GEMM: enough workgroups for four per compute unit, at least two K tiles each
uint32_t gemm32_splits(uint32_t M, uint32_t N, uint32_t K, uint32_t *kper)
{
    const uint32_t tiles = ((M + 63) / 64) * ((N + 63) / 64), ktiles = (K + 31) / 32;
    uint32_t splits = (1024u + tiles - 1) / tiles;
    if (splits > 16u) splits = 16u;
    if (splits > ktiles / 2u) splits = ktiles / 2u;
    if (splits < 1u) splits = 1u;
    const uint32_t per = (ktiles + splits - 1) / splits;
    *kper = per * 32u;
    return (ktiles + per - 1) / per;
}

void launch_gemm32(const LayerArgs &L, const float *A, float *C, uint32_t M, float *ws, uint64_t ws_floats)
{
    Gemm32Args g{L, A, C, nullptr, M, 0};
    uint32_t splits = gemm32_splits(M, L.N, L.K, &g.kper);
    if (splits > 1 && (uint64_t)splits * M * L.N > ws_floats) { splits = 1; g.kper = (L.K + 31u) / 32u * 32u; }
    if (splits > 1) g.ws = ws;
    g_last_kernel = "sp_gemm32_f32";
    const dim3 grid(((M + 63) / 64) * ((L.N + 63) / 64), splits);
    const bool vec = L.K % 4u == 0 && (reinterpret_cast<uintptr_t>(A) & 15u) == 0 && (reinterpret_cast<uintptr_t>(L.w) & 15u) == 0;
    if (vec) sp_gemm32_f32<true><<<grid, 256, 0, g_stream>>>(g);
    else sp_gemm32_f32<false><<<grid, 256, 0, g_stream>>>(g);
    if (splits > 1) sp_gemm32_reduce<<<(uint32_t)(((uint64_t)M * L.N + 255) / 256), 256, 0, g_stream>>>(g, splits);
}

int reserve(sphip_net *net, uint32_t n, bool keep_layers)
{
    const uint64_t need = (uint64_t)n * net->max_width;
    if (need > net->cap_elems) {
        for (int i = 0; i < 2; ++i) {
            if (net->buf[i]) { HCHECK(hipFree(net->buf[i])); net->buf[i] = nullptr; }
        }
        net->cap_elems = 0;
        for (int i = 0; i < 2; ++i) HCHECK(hipMalloc(&net->buf[i], need * sizeof(float)));
        net->cap_elems = need;
    }
    uint64_t soft = 0;
    for (uint32_t l = 1; l < net->layers; ++l)
        if (net->act[l - 1] == A_SOFTMAX && (uint64_t)n * net->topo[l] > soft) soft = (uint64_t)n * net->topo[l];
    if (soft > net->soft_cap) {
        if (net->soft_tmp) { HCHECK(hipFree(net->soft_tmp)); net->soft_tmp = nullptr; }
        net->soft_cap = 0;
        HCHECK(hipMalloc((void **)&net->soft_tmp, soft * sizeof(float)));
        net->soft_cap = soft;
    }
    if (n <= 64 && net->prec >= I8 && n > net->aq_cap_n) {
        // digit planes of the integer GEMV: 4 bytes per element (+ padding of the last chunk), one scale per chunk
        if (net->aq) { HCHECK(hipFree(net->aq)); HCHECK(hipFree(net->aq_inv)); HCHECK(hipFree(net->aq_dsum)); net->aq = nullptr; }
        net->aq_cap_n = 0;
        const uint64_t padded = (uint64_t)n * ((uint64_t)net->max_width + 4096u);
        HCHECK(hipMalloc((void **)&net->aq, padded * 4u));
        HCHECK(hipMalloc((void **)&net->aq_inv, (padded / 64u + 64u) * sizeof(float)));
        HCHECK(hipMalloc((void **)&net->aq_dsum, (padded / 64u + 64u) * 4u * sizeof(int)));
        net->aq_cap_n = n;
        net->aq_valid_layer = 0;
    }
    if (keep_layers && !net->layers_buf)
        HCHECK(hipMalloc((void **)&net->layers_buf, net->slots_total * sizeof(float)));
    if (net->prec == F32 && n > 64) {
        uint64_t ws = 0;
        for (uint32_t l = 1; l < net->layers; ++l) {
            uint32_t kper = 0;
            const uint32_t sp = gemm32_splits(n, net->topo[l], net->topo[l - 1], &kper);
            if (sp > 1 && (uint64_t)sp * n * net->topo[l] > ws) ws = (uint64_t)sp * n * net->topo[l];
        }
        if (ws > net->split_cap) {
            if (net->split_ws) { HCHECK(hipFree(net->split_ws)); net->split_ws = nullptr; }
            net->split_cap = 0;
            HCHECK(hipMalloc((void **)&net->split_ws, ws * sizeof(float)));
            net->split_cap = ws;
        }
    }
    if (net->prec != F32) {
        // thin-operand kernel: split-K workspace, and FP16 copies of the codes of layers with few outputs
        uint64_t ws = 0;
        for (uint32_t l = 1; l < net->layers; ++l) {
            const ThinPlan tp = plan_thin(net->prec, n, net->topo[l], net->topo[l - 1]);
            if (!tp.use) {
                uint32_t kper = 0;
                const uint32_t sp = gemm16_splits(n, net->topo[l], net->topo[l - 1], &kper);
                if (sp > 1 && (uint64_t)sp * n * net->topo[l] > ws) ws = (uint64_t)sp * n * net->topo[l];
                continue;
            }
            if (tp.splits > 1 && (uint64_t)tp.splits * tp.NC * tp.R > ws) ws = (uint64_t)tp.splits * tp.NC * tp.R;
            DevArray &wa = net->W[l - 1];
            if (tp.mode_b && net->prec >= I8 && !wa.codes16_valid && wa.uploaded) {
                if (!wa.codes16) HCHECK(hipMalloc((void **)&wa.codes16, wa.count * sizeof(uint16_t)));
                const uint32_t grid = (uint32_t)((wa.count + 255) / 256);
                if (net->prec == I8) sp_codes16<I8><<<grid, 256, 0, g_stream>>>(wa.base, wa.codes16, wa.count);
                else if (net->prec == I4) sp_codes16<I4><<<grid, 256, 0, g_stream>>>(wa.base, wa.codes16, wa.count);
                else sp_codes16<I2><<<grid, 256, 0, g_stream>>>(wa.base, wa.codes16, wa.count);
                HCHECK(hipGetLastError());
                wa.codes16_valid = true;
            }
        }
        if (ws > net->split_cap) {
            if (net->split_ws) { HCHECK(hipFree(net->split_ws)); net->split_ws = nullptr; }
            net->split_cap = 0;
            HCHECK(hipMalloc((void **)&net->split_ws, ws * sizeof(float)));
            net->split_cap = ws;
        }
    }
    return 0;
}

int grow(float **p, uint64_t *cap, uint64_t need)
{
    if (need <= *cap) return 0;
    if (*p) { HCHECK(hipFree(*p)); *p = nullptr; }
    *cap = 0;
    HCHECK(hipMalloc((void **)p, need * sizeof(float)));
    *cap = need;
    return 0;
}

int check_uploaded(const sphip_net *net)
{
    for (uint32_t l = 0; l + 1 < net->layers; ++l)
        if (!net->W[l].uploaded || !net->B[l].uploaded) return fail_msg("sphip: an array of this net was never uploaded");
    return 0;
}

// Enqueues every kernel of one forward.  d_x, d_y are device pointers.
// only_layer != 0 restricts the launch to the main kernel of that layer.
// keep (n == 1): every layer's output goes to its slot of layers_buf, d_x must be slot 0 and d_y the last slot.
int enqueue_forward(sphip_net *net, const float *d_x, uint32_t n, float *d_y, uint32_t flags, uint32_t only_layer,
                    bool keep = false)
{
    const Regime reg = pick_regime(net, n, flags);
    const bool f16t = net->prec != BF16;          // 16-bit activation type of the matrix-core path
    const uint32_t last = net->layers - 1;

    const void *in = d_x;
    if (reg == R_GEMM16 && !only_layer) {
        const uint64_t cnt = (uint64_t)n * net->topo[0];
        const uint32_t grid = (uint32_t)((cnt / 4 + 255) / 256 + 1);
        if (f16t) sp_cvt16<true><<<grid, 256, 0, g_stream>>>(d_x, (uint16_t *)net->buf[1], cnt);
        else sp_cvt16<false><<<grid, 256, 0, g_stream>>>(d_x, (uint16_t *)net->buf[1], cnt);
        in = net->buf[1];
    } else if (reg == R_GEMM16) {
        in = net->buf[1];
    }

    for (uint32_t l = 1; l <= last; ++l) {
        const LayerArgs L = make_layer_args(net, l);
        const bool softmax = net->act[l - 1] == A_SOFTMAX;
        const bool is_last = l == last;
        void *dst = is_last ? (void *)d_y : keep ? (void *)(net->layers_buf + net->slot_off[l]) : net->buf[(l + 1) & 1];
        // logits of a softmax layer go to FP32 scratch first
        void *main_out = softmax ? (void *)net->soft_tmp : dst;
        const int out_f32 = (reg != R_GEMM16) || is_last || softmax;
        const bool run = !only_layer || only_layer == l;
        if (run) {
            if (reg == R_GEMV) launch_gemv(net, L, (const float *)in, (float *)main_out, n, only_layer != 0 && net->aq_valid_layer == l && net->aq_valid_n == n);
            if (reg == R_GEMV) { net->aq_valid_layer = l; net->aq_valid_n = n; }
            else if (reg == R_GEMM32) launch_gemm32(L, (const float *)in, (float *)main_out, n, net->split_ws, net->split_cap);
            else {
                const DevArray &wa = net->W[l - 1];
                ThinCtx ctx{};
                if (net->prec == F16 || net->prec == BF16) ctx.w16 = reinterpret_cast<const uint16_t *>(wa.base);
                else if (wa.codes16_valid) ctx.w16 = wa.codes16;
                ctx.ws = net->split_ws;
                ctx.ws_floats = net->split_cap;
                launch_gemm16(net->prec, L, (const uint16_t *)in, main_out, n, out_f32, ctx);
            }
        }
        if (softmax && !only_layer) {
            const int kind = (reg == R_GEMM16 && !is_last) ? (f16t ? 2 : 1) : 0;
            sp_softmax_rows<<<(n + 3) / 4, 256, 0, g_stream>>>(net->soft_tmp, dst, kind, n, net->topo[l]);
        }
        in = dst;
    }
    HCHECK(hipGetLastError());
    return 0;
}

}  // namespace

extern "C" {

int sphip_device_count(void)
{
    int cnt = 0;
    if (hipGetDeviceCount(&cnt) != hipSuccess) return 0;
    return cnt;
}

const char *sphip_last_error_string(void) { return g_err; }

int sphip_create(const sphip_desc *desc, sphip_net **out)
{
    if (!desc || !out || desc->layers < 2 || !desc->topology || !desc->act) return fail_msg("sphip_create: invalid descriptor");
    if (desc->precision >= NFMT) return fail_msg("sphip_create: invalid precision");
    for (uint32_t l = 0; l < desc->layers; ++l)
        if (desc->topology[l] == 0) return fail_msg("sphip_create: empty layer");
    for (uint32_t l = 0; l + 1 < desc->layers; ++l)
        if (desc->act[l] >= A_COUNT) return fail_msg("sphip_create: invalid activation");
    if (ensure_stream()) return 1;
    sphip_net *net = new (std::nothrow) sphip_net;
    if (!net) return fail_msg("sphip_create: out of host memory");
    net->layers = desc->layers;
    net->topo.assign(desc->topology, desc->topology + desc->layers);
    net->act.assign(desc->act, desc->act + desc->layers - 1);
    net->prec = desc->precision;
    net->W.resize(desc->layers - 1);
    net->B.resize(desc->layers - 1);
    for (uint32_t l = 0; l < desc->layers; ++l) {
        if (net->topo[l] > net->max_width) net->max_width = net->topo[l];
        net->total_neurons += net->topo[l];
        net->slot_off.push_back((uint32_t)net->slots_total);
        net->slots_total += ((uint64_t)net->topo[l] + 3u) & ~3ull;
    }
    for (uint32_t l = 0; l + 1 < desc->layers; ++l) {
        DevArray &w = net->W[l], &b = net->B[l];
        w.count = (uint64_t)net->topo[l] * net->topo[l + 1];
        b.count = net->topo[l + 1];
        w.bytes = fmt_bytes(net->prec, w.count);
        b.bytes = fmt_bytes(net->prec, b.count);
        // 16 bytes of slack: vector loads of the last chunk never leave the allocation
        if (hipMalloc((void **)&w.base, w.bytes + 16) != hipSuccess || hipMalloc((void **)&b.base, b.bytes + 16) != hipSuccess) {
            sphip_destroy(net);
            return fail_msg("sphip_create: device allocation failed");
        }
    }
    *out = net;
    return 0;
}

void sphip_destroy(sphip_net *net)
{
    if (!net) return;
    if (g_stream) (void)hipStreamSynchronize(g_stream);
    train_free(net);
    for (auto &a : net->W) { if (a.base) (void)hipFree(a.base); if (a.codes16) (void)hipFree(a.codes16); }
    for (auto &a : net->B) if (a.base) (void)hipFree(a.base);
    if (net->split_ws) (void)hipFree(net->split_ws);
    if (net->eval_buf) (void)hipFree(net->eval_buf);
    for (int i = 0; i < 2; ++i) if (net->buf[i]) (void)hipFree(net->buf[i]);
    if (net->soft_tmp) (void)hipFree(net->soft_tmp);
    if (net->aq) (void)hipFree(net->aq);
    if (net->aq_inv) (void)hipFree(net->aq_inv);
    if (net->aq_dsum) (void)hipFree(net->aq_dsum);
    if (net->layers_buf) (void)hipFree(net->layers_buf);
    if (net->pin_in) (void)hipHostFree(net->pin_in);
    if (net->pin_out) (void)hipHostFree(net->pin_out);
    if (net->stage_x) (void)hipFree(net->stage_x);
    if (net->stage_y) (void)hipFree(net->stage_y);
    delete net;
}

int sphip_upload_array(sphip_net *net, uint32_t l, int which, const void *codes, size_t bytes, float max_val)
{
    if (!net || l + 1 >= net->layers || (which != 0 && which != 1) || !codes) return fail_msg("sphip_upload_array: invalid argument");
    DevArray &a = which == 0 ? net->W[l] : net->B[l];
    if (bytes != a.bytes) return fail_msg("sphip_upload_array: byte count does not match the array's serialized size");
    HCHECK(hipMemcpyAsync(a.base, codes, bytes, hipMemcpyHostToDevice, g_stream));
    HCHECK(hipStreamSynchronize(g_stream));
    a.max_val = max_val;
    a.uploaded = true;
    a.codes16_valid = false;
    return 0;
}

int sphip_clone(const sphip_net *src, sphip_net **out)
{
    if (!src || !out) return fail_msg("sphip_clone: invalid argument");
    sphip_desc d{src->layers, src->topo.data(), src->act.data(), (uint8_t)src->prec};
    sphip_net *net = nullptr;
    if (sphip_create(&d, &net)) return 1;
    for (uint32_t l = 0; l + 1 < src->layers; ++l) {
        for (int which = 0; which < 2; ++which) {
            const DevArray &s = which == 0 ? src->W[l] : src->B[l];
            DevArray &t = which == 0 ? net->W[l] : net->B[l];
            hipError_t e = hipMemcpyAsync(t.base, s.base, s.bytes, hipMemcpyDeviceToDevice, g_stream);
            if (e != hipSuccess) { sphip_destroy(net); return fail_hip("sphip_clone copy", e); }
            t.max_val = s.max_val;
            t.uploaded = s.uploaded;
        }
    }
    HCHECK(hipStreamSynchronize(g_stream));
    *out = net;
    return 0;
}

// Small host inputs travel through a pinned staging buffer and a copy kernel; small outputs are
// written by the last layer's kernel straight into pinned memory (scattered stores over PCIe do
// not pay beyond a few thousand values), and the call ends with one stream synchronisation.
static const uint64_t kSmallIn = 256u * 1024u, kSmallOut = 4096u;

static int grow_pinned(float **p, uint64_t *cap, uint64_t need)
{
    if (need <= *cap) return 0;
    if (*p) { HCHECK(hipHostFree(*p)); *p = nullptr; }
    *cap = 0;
    HCHECK(hipHostMalloc((void **)p, need * sizeof(float), hipHostMallocDefault));
    *cap = need;
    return 0;
}

int sphip_forward(sphip_net *net, const float *x, uint32_t n, float *y, uint32_t flags)
{
    if (!net || !x || !y || n == 0) return fail_msg("sphip_forward: invalid argument");
    if (check_uploaded(net)) return 1;
    if (reserve(net, n, false)) return 1;
    const uint64_t in_cnt = (uint64_t)n * net->topo[0], out_cnt = (uint64_t)n * net->topo[net->layers - 1];
    const float *d_x = x;
    float *d_y = y;
    bool y_pinned = false;
    if (!(flags & SPHIP_X_ON_DEVICE)) {
        if (grow(&net->stage_x, &net->stage_x_cap, in_cnt)) return 1;
        if (in_cnt <= kSmallIn) {
            if (grow_pinned(&net->pin_in, &net->pin_in_cap, in_cnt)) return 1;
            memcpy(net->pin_in, x, in_cnt * sizeof(float));
            sp_copy32<<<(uint32_t)((in_cnt + 255) / 256), 256, 0, g_stream>>>(net->pin_in, net->stage_x, in_cnt);
        } else {
            HCHECK(hipMemcpyAsync(net->stage_x, x, in_cnt * sizeof(float), hipMemcpyHostToDevice, g_stream));
        }
        d_x = net->stage_x;
    }
    if (!(flags & SPHIP_Y_ON_DEVICE)) {
        if (out_cnt <= kSmallOut) {
            if (grow_pinned(&net->pin_out, &net->pin_out_cap, out_cnt)) return 1;
            d_y = net->pin_out;
            y_pinned = true;
        } else {
            if (grow(&net->stage_y, &net->stage_y_cap, out_cnt)) return 1;
            d_y = net->stage_y;
        }
    }
    if (enqueue_forward(net, d_x, n, d_y, flags, 0)) return 1;
    if (!(flags & SPHIP_Y_ON_DEVICE)) {
        if (!y_pinned) HCHECK(hipMemcpyAsync(y, d_y, out_cnt * sizeof(float), hipMemcpyDeviceToHost, g_stream));
        HCHECK(hipStreamSynchronize(g_stream));
        if (y_pinned) memcpy(y, net->pin_out, out_cnt * sizeof(float));
    }
    return 0;
}

int sphip_forward_layers(sphip_net *net, const float *x, float *host_neurons)
{
    if (!net || !x || !host_neurons) return fail_msg("sphip_forward_layers: invalid argument");
    if (check_uploaded(net)) return 1;
    if (reserve(net, 1, true)) return 1;
    const uint32_t last = net->layers - 1;
    if (grow_pinned(&net->pin_in, &net->pin_in_cap, net->topo[0])) return 1;
    if (grow_pinned(&net->pin_out, &net->pin_out_cap, net->total_neurons)) return 1;
    memcpy(net->pin_in, x, (size_t)net->topo[0] * sizeof(float));
    sp_copy32<<<(net->topo[0] + 255) / 256, 256, 0, g_stream>>>(net->pin_in, net->layers_buf, net->topo[0]);
    if (enqueue_forward(net, net->layers_buf, 1, net->layers_buf + net->slot_off[last], 0, 0, true)) return 1;
    // all slots, densely packed, straight into pinned memory
    uint32_t dense = 0;
    for (uint32_t l0 = 0; l0 < net->layers; l0 += 16) {
        PackArgs pa{};
        pa.src = net->layers_buf;
        pa.dst = net->pin_out;
        pa.count = net->layers - l0 < 16 ? net->layers - l0 : 16;
        uint32_t widest = 1;
        for (uint32_t i = 0; i < pa.count; ++i) {
            pa.src_off[i] = net->slot_off[l0 + i];
            pa.dst_off[i] = dense;
            pa.len[i] = net->topo[l0 + i];
            dense += net->topo[l0 + i];
            if (pa.len[i] > widest) widest = pa.len[i];
        }
        uint32_t gx = (widest + 255) / 256;
        if (gx > 64) gx = 64;
        sp_pack_layers<<<dim3(gx, pa.count), 256, 0, g_stream>>>(pa);
    }
    HCHECK(hipGetLastError());
    HCHECK(hipStreamSynchronize(g_stream));
    memcpy(host_neurons, net->pin_out, net->total_neurons * sizeof(float));
    return 0;
}

int sphip_evaluate(sphip_net *net, const float *x, const float *targets, uint32_t n, int loss_func, uint32_t flags,
                   float *total_loss, uint32_t *predictions, uint32_t *correct)
{
    if (!net || !x || !targets || n == 0 || (loss_func != 0 && loss_func != 1))
        return fail_msg("sphip_evaluate: invalid argument");
    if (check_uploaded(net)) return 1;
    if (reserve(net, n, false)) return 1;
    const uint32_t width = net->topo[net->layers - 1];
    const uint64_t in_cnt = (uint64_t)n * net->topo[0], out_cnt = (uint64_t)n * width;
    const bool on_dev = (flags & SPHIP_X_ON_DEVICE) != 0;
    // layout of the evaluation buffer (4-byte units): outputs | staged targets | loss | pred | hit | totals (16 bytes)
    const uint64_t need = out_cnt * (on_dev ? 1u : 2u) + 3ull * n + 8u;
    if (grow(&net->eval_buf, &net->eval_cap, need)) return 1;
    float *d_y = net->eval_buf;
    float *d_t = on_dev ? nullptr : net->eval_buf + out_cnt;
    float *d_loss = net->eval_buf + out_cnt * (on_dev ? 1u : 2u);
    uint32_t *d_pred = reinterpret_cast<uint32_t *>(d_loss + n);
    uint32_t *d_hit = d_pred + n;
    double *d_tot = reinterpret_cast<double *>((reinterpret_cast<uintptr_t>(d_hit + n) + 7u) & ~(uintptr_t)7u);
    uint32_t *d_hits = reinterpret_cast<uint32_t *>(d_tot + 1);
    const float *d_x = x;
    if (!on_dev) {
        if (grow(&net->stage_x, &net->stage_x_cap, in_cnt)) return 1;
        HCHECK(hipMemcpyAsync(net->stage_x, x, in_cnt * sizeof(float), hipMemcpyHostToDevice, g_stream));
        HCHECK(hipMemcpyAsync(d_t, targets, out_cnt * sizeof(float), hipMemcpyHostToDevice, g_stream));
        d_x = net->stage_x;
    }
    if (enqueue_forward(net, d_x, n, d_y, flags & (SPHIP_FORCE_GEMM | SPHIP_FORCE_GEMV), 0)) return 1;
    EvalArgs a{d_y, on_dev ? targets : d_t, d_loss, d_pred, d_hit, n, width, loss_func,
               net->act[net->layers - 2] == A_SIGMOID ? 1 : 0};
    sp_eval_rows<<<(n + 3) / 4, 256, 0, g_stream>>>(a);
    sp_eval_total<<<1, 1024, 0, g_stream>>>(d_loss, d_hit, n, d_tot, d_hits);
    HCHECK(hipGetLastError());
    struct { double loss; uint32_t hits; uint32_t pad; } tot;
    HCHECK(hipMemcpyAsync(&tot, d_tot, 16, hipMemcpyDeviceToHost, g_stream));
    if (predictions) HCHECK(hipMemcpyAsync(predictions, d_pred, (size_t)n * sizeof(uint32_t), hipMemcpyDeviceToHost, g_stream));
    HCHECK(hipStreamSynchronize(g_stream));
    if (total_loss) *total_loss = (float)tot.loss;
    if (correct) *correct = tot.hits;
    return 0;
}

int sphip_decode(sphip_net *net, uint32_t l, int which, int mode, float *host_out)
{
    if (!net || l + 1 >= net->layers || (which != 0 && which != 1) || !host_out || (mode != 0 && mode != 1))
        return fail_msg("sphip_decode: invalid argument");
    const DevArray &a = which == 0 ? net->W[l] : net->B[l];
    if (!a.uploaded) return fail_msg("sphip_decode: array not uploaded");
    float *d_out = nullptr;
    HCHECK(hipMalloc((void **)&d_out, a.count * sizeof(float)));
    DecodeParams p{};
    p.codes = a.base;
    p.out = d_out;
    p.n = a.count;
    p.max_val = a.max_val;
    p.mode = mode;
    const float d = fmt_divisor(net->prec);
    {
        volatile float r = 1.0f / d;
        volatile float s = a.max_val * r;
        p.rel_scale = s;
    }
    if (net->prec == I8) for (int q = -128; q < 128; ++q) { volatile float fq = (float)q; volatile float tq = fq / 127.0f; p.lut[q + 128] = tq; }
    if (net->prec == I4) for (int q = -8; q < 8; ++q) { volatile float fq = (float)q; volatile float tq = fq / 7.0f; p.lut[q + 8] = tq; }
    const uint32_t grid = (uint32_t)((a.count + 255) / 256);
    switch (net->prec) {
    case F32:  sp_decode<F32><<<grid, 256, 0, g_stream>>>(p); break;
    case F16:  sp_decode<F16><<<grid, 256, 0, g_stream>>>(p); break;
    case BF16: sp_decode<BF16><<<grid, 256, 0, g_stream>>>(p); break;
    case I8:   sp_decode<I8><<<grid, 256, 0, g_stream>>>(p); break;
    case I4:   sp_decode<I4><<<grid, 256, 0, g_stream>>>(p); break;
    default:   sp_decode<I2><<<grid, 256, 0, g_stream>>>(p); break;
    }
    hipError_t e = hipGetLastError();
    if (e == hipSuccess) e = hipMemcpyAsync(host_out, d_out, a.count * sizeof(float), hipMemcpyDeviceToHost, g_stream);
    if (e == hipSuccess) e = hipStreamSynchronize(g_stream);
    (void)hipFree(d_out);
    if (e != hipSuccess) return fail_hip("sphip_decode", e);
    return 0;
}

int sphip_synchronize(void)
{
    if (!g_stream) return 0;
    HCHECK(hipStreamSynchronize(g_stream));
    return 0;
}

int sphip_malloc(void **dptr, size_t bytes)
{
    if (!dptr) return fail_msg("sphip_malloc: null");
    if (ensure_stream()) return 1;
    HCHECK(hipMalloc(dptr, bytes ? bytes : 1));
    return 0;
}

int sphip_free(void *dptr)
{
    if (dptr) HCHECK(hipFree(dptr));
    return 0;
}

int sphip_memcpy_h2d(void *dst, const void *src, size_t bytes)
{
    if (ensure_stream()) return 1;
    HCHECK(hipMemcpyAsync(dst, src, bytes, hipMemcpyHostToDevice, g_stream));
    HCHECK(hipStreamSynchronize(g_stream));
    return 0;
}

int sphip_memcpy_d2h(void *dst, const void *src, size_t bytes)
{
    if (ensure_stream()) return 1;
    HCHECK(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToHost, g_stream));
    HCHECK(hipStreamSynchronize(g_stream));
    return 0;
}

static int time_common(sphip_net *const *nets, int count, const float *d_x, uint32_t n, float *d_y,
                       uint32_t flags, int iters, float *ms, uint32_t only_layer)
{
    if (!nets || count <= 0 || iters <= 0 || !ms) return fail_msg("sphip_time: invalid argument");
    for (int i = 0; i < count; ++i) {
        if (!nets[i]) return fail_msg("sphip_time: null net");
        if (check_uploaded(nets[i])) return 1;
        if (reserve(nets[i], n, false)) return 1;
    }
    hipEvent_t e0, e1;
    HCHECK(hipEventCreate(&e0));
    HCHECK(hipEventCreate(&e1));
    int rc = 0;
    HCHECK(hipEventRecord(e0, g_stream));
    for (int it = 0; it < iters && !rc; ++it) rc = enqueue_forward(nets[it % count], d_x, n, d_y, flags, only_layer);
    hipError_t e = hipEventRecord(e1, g_stream);
    if (e == hipSuccess) e = hipEventSynchronize(e1);
    if (e == hipSuccess) e = hipEventElapsedTime(ms, e0, e1);
    (void)hipEventDestroy(e0);
    (void)hipEventDestroy(e1);
    if (rc) return rc;
    if (e != hipSuccess) return fail_hip("sphip_time", e);
    return 0;
}

int sphip_time_forward(sphip_net *const *nets, int count, const float *d_x, uint32_t n, float *d_y,
                       uint32_t flags, int iters, float *ms)
{
    if (!d_x || !d_y || n == 0) return fail_msg("sphip_time_forward: invalid argument");
    return time_common(nets, count, d_x, n, d_y, flags, iters, ms, 0);
}

int sphip_time_layer(sphip_net *const *nets, int count, uint32_t layer, uint32_t n, uint32_t flags,
                     int iters, float *ms)
{
    if (!nets || count <= 0 || !nets[0] || layer == 0 || layer >= nets[0]->layers || n == 0)
        return fail_msg("sphip_time_layer: invalid argument");
    // inputs and outputs are the nets' own scratch buffers (contents irrelevant for timing)
    for (int i = 0; i < count; ++i) {
        if (reserve(nets[i], n, false)) return 1;
        if (grow(&nets[i]->stage_y, &nets[i]->stage_y_cap, (uint64_t)n * nets[i]->topo[nets[i]->layers - 1])) return 1;
        if (grow(&nets[i]->stage_x, &nets[i]->stage_x_cap, (uint64_t)n * nets[i]->topo[0])) return 1;
    }
    return time_common(nets, count, nets[0]->stage_x, n, nets[0]->stage_y, flags, iters, ms, layer);
}

const char *sphip_layer_kernel_name(sphip_net *net, uint32_t layer, uint32_t n, uint32_t flags)
{
    (void)n; (void)flags;
    if (!net || layer == 0 || layer >= net->layers) return "";
    return g_last_kernel;
}

}  // extern "C"

// the batched training step (its own kernels and entry points)
#include "hip_train.inl"
