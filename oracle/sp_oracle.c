/*
 * sp_oracle.c — CPU restatement of Spingalett's quantized-load + forward path.
 * TEST INFRASTRUCTURE ONLY (see sp_oracle.h).  Build with strict IEEE
 * semantics: -O2 -ffp-contract=off, never -ffast-math.
 */
#define _POSIX_C_SOURCE 200809L
#include "sp_oracle.h"

#include <float.h>
#include <math.h>
#include <stdlib.h>
#include <string.h>
#include <time.h>

#if defined(_OPENMP)
#include <omp.h>
#endif

/* ------------------------------------------------------------------ */
/* scalar codecs                                                       */
/* ------------------------------------------------------------------ */

static inline uint32_t f2u(float x) { uint32_t u; memcpy(&u, &x, 4); return u; }
static inline float    u2f(uint32_t u) { float x; memcpy(&x, &u, 4); return x; }

/* Serialize.c:45-72.  Exact binary16 -> binary32, every NaN collapses to the
 * quiet NaN with the input's sign (payload dropped). */
float orc_fp16_to_f32(uint16_t h)
{
    uint32_t s = (uint32_t)(h >> 15) << 31;
    uint32_t e = (h >> 10) & 31u;
    uint32_t m = h & 1023u;
    if (e == 31u) return u2f(s | (m ? 0x7FC00000u : 0x7F800000u));
    if (e != 0u)  return u2f(s | ((e + 112u) << 23) | (m << 13));
    if (m == 0u)  return u2f(s);
    /* subnormal half: value = m * 2^-24; normalise the leading one */
    int shift = 0;
    while (!(m & 1024u)) { m <<= 1; ++shift; }
    return u2f(s | ((uint32_t)(113 - shift) << 23) | ((m & 1023u) << 13));
}

/* Serialize.c:12-43.  Truncating (round-toward-zero) encode; binary32
 * subnormals and anything below 2^-24 become signed zero; above 2^15 -> inf. */
uint16_t orc_f32_to_fp16(float x)
{
    uint32_t u = f2u(x);
    uint16_t s = (uint16_t)((u >> 16) & 0x8000u);
    uint32_t e = (u >> 23) & 255u;
    uint32_t m = u & 0x7FFFFFu;
    if (e == 0u)   return s;
    if (e == 255u) return (uint16_t)(s | (m ? 0x7E00u : 0x7C00u));
    int ue = (int)e - 127;
    if (ue > 15)  return (uint16_t)(s | 0x7C00u);
    if (ue < -24) return s;
    if (ue < -14) return (uint16_t)(s | ((0x800000u | m) >> (-1 - ue)));
    return (uint16_t)(s | ((uint32_t)(ue + 15) << 10) | (m >> 13));
}

/* Serialize.c:80-85 */
float orc_bf16_to_f32(uint16_t h) { return u2f((uint32_t)h << 16); }
/* Serialize.c:74-78 (truncation) */
uint16_t orc_f32_to_bf16(float x) { return (uint16_t)(f2u(x) >> 16); }

/* ------------------------------------------------------------------ */
/* array codecs                                                        */
/* ------------------------------------------------------------------ */

size_t orc_array_bytes(uint32_t n, int precision)
{
    switch (precision) {
    case ORC_PREC_F32:  return 4u * (size_t)n;
    case ORC_PREC_F16:
    case ORC_PREC_BF16: return 2u * (size_t)n;
    case ORC_PREC_I8:   return 4u + (size_t)n;
    case ORC_PREC_I4:   return 4u + ((size_t)n + 1u) / 2u;
    case ORC_PREC_I2:   return 4u + ((size_t)n + 3u) / 4u;
    default:            return 0;
    }
}

/* One integer code -> float under the chosen evaluation of
 * ((float)q / d) * max  (Serialize.c:233 d=127, :258 d=7, :285 no divisor). */
static inline float dequant_code(int q, float d, float max_val, int mode)
{
    volatile float fq = (float)q;           /* volatile: no reassociation */
    if (d == 1.0f) return fq * max_val;
    if (mode == ORC_DEQUANT_RELEASE) {
        volatile float r = 1.0f / d;
        volatile float s = max_val * r;
        return fq * s;
    }
    volatile float t = fq / d;
    return t * max_val;
}

/* Serialize.c:195-297 */
size_t orc_decode_array(const uint8_t *src, size_t avail, uint32_t n,
                        int precision, int mode, float *dst)
{
    size_t need = orc_array_bytes(n, precision);
    if (need == 0 && n != 0) return 0;
    if (avail < need) return 0;

    if (precision == ORC_PREC_F32) { memcpy(dst, src, need); return need; }
    if (precision == ORC_PREC_F16 || precision == ORC_PREC_BF16) {
        for (uint32_t i = 0; i < n; ++i) {
            uint16_t h; memcpy(&h, src + 2u * (size_t)i, 2);
            dst[i] = precision == ORC_PREC_F16 ? orc_fp16_to_f32(h) : orc_bf16_to_f32(h);
        }
        return need;
    }

    float max_val; memcpy(&max_val, src, 4);
    const uint8_t *p = src + 4;
    if (!(max_val > 0.0f)) {                 /* 0, negative, NaN -> zeros */
        memset(dst, 0, 4u * (size_t)n);
        return need;
    }
    for (uint32_t i = 0; i < n; ++i) {
        int q; float d;
        if (precision == ORC_PREC_I8) {
            q = (int8_t)p[i]; d = 127.0f;
        } else if (precision == ORC_PREC_I4) {
            unsigned nib = (i & 1u) ? (p[i >> 1] >> 4) : (p[i >> 1] & 15u);
            q = (int)nib - ((nib & 8u) ? 16 : 0); d = 7.0f;
        } else {
            unsigned c = (p[i >> 2] >> ((i & 3u) * 2u)) & 3u;
            q = (int)c - ((c & 2u) ? 4 : 0); d = 1.0f;
        }
        dst[i] = dequant_code(q, d, max_val, mode);
    }
    return need;
}

static float array_absmax(const float *x, uint32_t n)
{
    float m = 0.0f;
    for (uint32_t i = 0; i < n; ++i) { float a = fabsf(x[i]); if (a > m) m = a; }
    return m;
}

/* Serialize.c:87-193 */
size_t orc_encode_array(const float *src, uint32_t n, int precision, uint8_t *dst)
{
    size_t need = orc_array_bytes(n, precision);
    if (precision == ORC_PREC_F32) { memcpy(dst, src, need); return need; }
    if (precision == ORC_PREC_F16 || precision == ORC_PREC_BF16) {
        for (uint32_t i = 0; i < n; ++i) {
            uint16_t h = precision == ORC_PREC_F16 ? orc_f32_to_fp16(src[i])
                                                   : orc_f32_to_bf16(src[i]);
            memcpy(dst + 2u * (size_t)i, &h, 2);
        }
        return need;
    }
    float max_val = array_absmax(src, n);
    memcpy(dst, &max_val, 4);
    uint8_t *p = dst + 4;
    memset(p, 0, need - 4u);
    if (!(max_val > 0.0f)) return need;
    for (uint32_t i = 0; i < n; ++i) {
        volatile float r = src[i] / max_val;
        if (precision == ORC_PREC_I8) {
            volatile float sc = r * 127.0f;
            p[i] = (uint8_t)(int8_t)roundf(sc);
        } else if (precision == ORC_PREC_I4) {
            volatile float sc = r * 7.0f;
            int q = (int8_t)roundf(sc);
            if (q > 7) q = 7;
            if (q < -8) q = -8;
            p[i >> 1] |= (uint8_t)(((unsigned)q & 15u) << ((i & 1u) * 4u));
        } else {
            int q = r > 0.5f ? 1 : (r < -0.5f ? -1 : 0);
            p[i >> 2] |= (uint8_t)(((unsigned)q & 3u) << ((i & 3u) * 2u));
        }
    }
    return need;
}

/* ------------------------------------------------------------------ */
/* network container + file format                                     */
/* ------------------------------------------------------------------ */

/* Offsets as in Network.c:16-32: layer l's matrix starts after all earlier
 * matrices; row-major [out][in] (Private.h:16). */
orc_net *orc_new(uint32_t layers, const uint32_t *topology, const uint8_t *act)
{
    if (layers < 2) return NULL;
    orc_net *n = (orc_net *)calloc(1, sizeof *n);
    if (!n) return NULL;
    n->layers = layers;
    n->topology = (uint32_t *)malloc(sizeof(uint32_t) * layers);
    n->act  = (uint8_t *)malloc(layers - 1);
    n->woff = (uint64_t *)malloc(sizeof(uint64_t) * (layers - 1));
    n->boff = (uint64_t *)malloc(sizeof(uint64_t) * (layers - 1));
    memcpy(n->topology, topology, sizeof(uint32_t) * layers);
    memcpy(n->act, act, layers - 1);
    uint64_t w = 0, b = 0;
    for (uint32_t l = 0; l + 1 < layers; ++l) {
        n->woff[l] = w; n->boff[l] = b;
        w += (uint64_t)topology[l] * topology[l + 1];
        b += topology[l + 1];
    }
    n->total_weights = w; n->total_biases = b;
    n->weights = (float *)calloc(w ? w : 1, sizeof(float));
    n->biases  = (float *)calloc(b ? b : 1, sizeof(float));
    if (!n->weights || !n->biases) { orc_free(n); return NULL; }
    return n;
}

void orc_free(orc_net *n)
{
    if (!n) return;
    free(n->topology); free(n->act); free(n->woff); free(n->boff);
    free(n->weights); free(n->biases); free(n);
}

/* Header and payload order: Serialize.c:348-407 (writer), :438-591 (reader).
 *   u16 version(=1) u32 layers u8 loss u8 has_opt [u64 time_step] u8 precision
 *   u32 topology[L] u8 act[L-1]
 *   per layer: W [mW vW] b [mb vb], every array in the file's one precision. */
orc_net *orc_parse(const uint8_t *buf, size_t len, int mode, int *err)
{
    size_t pos = 0;
    int dummy; if (!err) err = &dummy;
    *err = 0;
#define TAKE(dst, nbytes) do { if (pos + (nbytes) > len) { *err = 1; return NULL; } \
                               memcpy((dst), buf + pos, (nbytes)); pos += (nbytes); } while (0)
    uint16_t version; TAKE(&version, 2);
    if (version != 1) { *err = 2; return NULL; }
    uint32_t layers; TAKE(&layers, 4);
    if (layers < 2) { *err = 3; return NULL; }
    uint8_t loss; TAKE(&loss, 1);
    if (loss >= 2) { *err = 4; return NULL; }
    uint8_t has_opt; TAKE(&has_opt, 1);
    uint64_t ts = 0;
    if (has_opt) TAKE(&ts, 8);
    uint8_t prec; TAKE(&prec, 1);
    if (prec >= ORC_PREC_COUNT) { *err = 5; return NULL; }
    if ((len - pos) / 4u < layers) { *err = 1; return NULL; }
    uint32_t *topo = (uint32_t *)malloc(4u * (size_t)layers);
    uint8_t  *act  = (uint8_t *)malloc(layers - 1);
    memcpy(topo, buf + pos, 4u * (size_t)layers); pos += 4u * (size_t)layers;
    for (uint32_t i = 0; i + 1 < layers; ++i) {
        if (pos >= len) { *err = 1; free(topo); free(act); return NULL; }
        act[i] = buf[pos++];
        if (act[i] >= ORC_ACT_COUNT) { *err = 6; free(topo); free(act); return NULL; }
    }
#undef TAKE
    orc_net *n = orc_new(layers, topo, act);
    free(topo); free(act);
    if (!n) { *err = 1; return NULL; }
    n->loss = loss; n->has_optimizer = has_opt; n->precision = prec; n->time_step = ts;

    for (uint32_t l = 0; l + 1 < layers && !n->truncated; ++l) {
        /* element count is a 32-bit product in the reference (Serialize.c:573) */
        uint32_t wcount = n->topology[l] * n->topology[l + 1];
        uint32_t bcount = n->topology[l + 1];
        size_t wbytes = orc_array_bytes(wcount, prec), bbytes = orc_array_bytes(bcount, prec);
        size_t got = orc_decode_array(buf + pos, len - pos, wcount, prec, mode,
                                      n->weights + n->woff[l]);
        if (!got) { n->truncated = 1; break; }
        pos += got;
        if (has_opt) {                        /* m and v of the weights: skipped */
            if (len - pos < 2 * wbytes) { n->truncated = 1; break; }
            pos += 2 * wbytes;
        }
        got = orc_decode_array(buf + pos, len - pos, bcount, prec, mode,
                               n->biases + n->boff[l]);
        if (!got) { n->truncated = 1; break; }
        pos += got;
        if (has_opt) {
            if (len - pos < 2 * bbytes) { n->truncated = 1; break; }
            pos += 2 * bbytes;
        }
    }
    return n;
}

size_t orc_serialized_size(const orc_net *n, int precision, int with_opt)
{
    size_t s = 2 + 4 + 1 + 1 + (with_opt ? 8 : 0) + 1 + 4u * (size_t)n->layers + (n->layers - 1);
    size_t mult = with_opt ? 3 : 1;
    for (uint32_t l = 0; l + 1 < n->layers; ++l) {
        s += mult * orc_array_bytes(n->topology[l] * n->topology[l + 1], precision);
        s += mult * orc_array_bytes(n->topology[l + 1], precision);
    }
    return s;
}

/* Optimizer moments are written as zeros (a freshly built net has zero m, v). */
size_t orc_serialize(const orc_net *n, int precision, int with_opt, uint8_t *dst)
{
    size_t pos = 0;
#define PUT(src, nbytes) do { memcpy(dst + pos, (src), (nbytes)); pos += (nbytes); } while (0)
    uint16_t version = 1; PUT(&version, 2);
    PUT(&n->layers, 4);
    PUT(&n->loss, 1);
    uint8_t ho = with_opt ? 1 : 0; PUT(&ho, 1);
    if (with_opt) PUT(&n->time_step, 8);
    uint8_t pr = (uint8_t)precision; PUT(&pr, 1);
    PUT(n->topology, 4u * (size_t)n->layers);
    PUT(n->act, n->layers - 1);
#undef PUT
    for (uint32_t l = 0; l + 1 < n->layers; ++l) {
        uint32_t wcount = n->topology[l] * n->topology[l + 1];
        uint32_t bcount = n->topology[l + 1];
        pos += orc_encode_array(n->weights + n->woff[l], wcount, precision, dst + pos);
        if (with_opt) {
            float *z = (float *)calloc(wcount ? wcount : 1, sizeof(float));
            pos += orc_encode_array(z, wcount, precision, dst + pos);
            pos += orc_encode_array(z, wcount, precision, dst + pos);
            free(z);
        }
        pos += orc_encode_array(n->biases + n->boff[l], bcount, precision, dst + pos);
        if (with_opt) {
            float *z = (float *)calloc(bcount ? bcount : 1, sizeof(float));
            pos += orc_encode_array(z, bcount, precision, dst + pos);
            pos += orc_encode_array(z, bcount, precision, dst + pos);
            free(z);
        }
    }
    return pos;
}

/* ------------------------------------------------------------------ */
/* activations                                                         */
/* ------------------------------------------------------------------ */

/* Activation.c:23-38; the leak factor 0.01f is fixed. */
float orc_activate(float x, int act)
{
    switch (act) {
    case ORC_ACT_SIGMOID:    return 1.0f / (1.0f + expf(-x));
    case ORC_ACT_RELU:       return x > 0.0f ? x : 0.0f;
    case ORC_ACT_TANH:       return tanhf(x);
    case ORC_ACT_LEAKY_RELU: return x > 0.0f ? x : 0.01f * x;
    case ORC_ACT_FOO52:
        if (x > 1.0f) return 1.0f + 0.01f * (x - 1.0f);
        return x < 0.0f ? 0.01f * x : x;
    default:                 return x;       /* SOFTMAX handled per row, NONE */
    }
}

/* Activation.c:5-21: max, exp(x-max), serial FP32 sum, scale by 1/sum when the
 * sum is positive.  (The reference indexes with uint16_t and cannot finish for
 * rows of 65,536 or more; this restatement uses a 32-bit index.) */
void orc_softmax(float *row, uint32_t n)
{
    float m = -FLT_MAX;
    for (uint32_t i = 0; i < n; ++i) if (row[i] > m) m = row[i];
    float s = 0.0f;
    for (uint32_t i = 0; i < n; ++i) { row[i] = expf(row[i] - m); s += row[i]; }
    if (s > 0.0f) {
        float inv = 1.0f / s;
        for (uint32_t i = 0; i < n; ++i) row[i] *= inv;
    }
}

/* SIMD.c:21-88 / Training.c:338-343 */
void orc_apply_activation(float *data, uint64_t rows, uint32_t width, int act)
{
    if (act == ORC_ACT_NONE || act >= ORC_ACT_COUNT) return;
    if (act == ORC_ACT_SOFTMAX) {
        for (uint64_t r = 0; r < rows; ++r) orc_softmax(data + r * width, width);
        return;
    }
    uint64_t total = rows * width;
    for (uint64_t i = 0; i < total; ++i) data[i] = orc_activate(data[i], act);
}

/* ------------------------------------------------------------------ */
/* forward                                                             */
/* ------------------------------------------------------------------ */

static uint32_t max_width(const orc_net *n)
{
    uint32_t m = 0;
    for (uint32_t l = 0; l < n->layers; ++l) if (n->topology[l] > m) m = n->topology[l];
    return m;
}

/* Network.c:202-251 (scalar branch: y = b; y[j] += dot(x, W_j); activation) */
void orc_forward_single(const orc_net *n, const float *x, float *out)
{
    uint32_t mw = max_width(n);
    float *cur = (float *)malloc(4u * (size_t)mw), *nxt = (float *)malloc(4u * (size_t)mw);
    memcpy(cur, x, 4u * (size_t)n->topology[0]);
    for (uint32_t l = 1; l < n->layers; ++l) {
        uint32_t in = n->topology[l - 1], o = n->topology[l];
        const float *W = n->weights + n->woff[l - 1], *b = n->biases + n->boff[l - 1];
        for (uint32_t j = 0; j < o; ++j) {
            float acc = 0.0f;
            const float *row = W + (uint64_t)j * in;
            for (uint32_t k = 0; k < in; ++k) acc += cur[k] * row[k];
            nxt[j] = b[j] + acc;
        }
        orc_apply_activation(nxt, 1, o, n->act[l - 1]);
        float *t = cur; cur = nxt; nxt = t;
    }
    memcpy(out, cur, 4u * (size_t)n->topology[n->layers - 1]);
    free(cur); free(nxt);
}

/* Built-in C = A W^T used when no BLAS is supplied: rows of A across threads,
 * 8 running sums per output so the compiler can vectorise along k. */
static void own_sgemm_nt(uint32_t N, uint32_t o, uint32_t in,
                         const float *A, const float *W, float *C)
{
#if defined(_OPENMP)
#pragma omp parallel for schedule(static)
#endif
    for (int64_t s = 0; s < (int64_t)N; ++s) {
        const float *a = A + (uint64_t)s * in;
        for (uint32_t j = 0; j < o; ++j) {
            const float *w = W + (uint64_t)j * in;
            float p[8] = {0, 0, 0, 0, 0, 0, 0, 0};
            uint32_t k = 0;
            for (; k + 8 <= in; k += 8)
                for (int u = 0; u < 8; ++u) p[u] += a[k + u] * w[k + u];
            float acc = ((p[0] + p[1]) + (p[2] + p[3])) + ((p[4] + p[5]) + (p[6] + p[7]));
            for (; k < in; ++k) acc += a[k] * w[k];
            C[(uint64_t)s * o + j] = acc;
        }
    }
}

typedef void (*sgemm_t)(int order, int ta, int tb, int M, int Nn, int K, float alpha,
                        const float *A, int lda, const float *B, int ldb, float beta,
                        float *C, int ldc);

/* Training.c:313-345 with the GEMM supplied by the caller. */
static void forward_batch_impl(const orc_net *n, const float *X, uint32_t N, float *out,
                               sgemm_t gemm, float *bufA, float *bufB)
{
    const float *A = X;
    float *C = bufA;
    for (uint32_t l = 1; l < n->layers; ++l) {
        uint32_t in = n->topology[l - 1], o = n->topology[l];
        const float *W = n->weights + n->woff[l - 1], *b = n->biases + n->boff[l - 1];
        C = (l == n->layers - 1) ? out : ((l & 1u) ? bufA : bufB);
        if (gemm)   /* RowMajor=101, NoTrans=111, Trans=112 (Training.c:327-333) */
            gemm(101, 111, 112, (int)N, (int)o, (int)in, 1.0f, A, (int)in, W, (int)in, 0.0f, C, (int)o);
        else
            own_sgemm_nt(N, o, in, A, W, C);
        /* C += ones (x) bias  (the cblas_sger at Training.c:335-336) */
        for (uint64_t s = 0; s < N; ++s)
            for (uint32_t j = 0; j < o; ++j) C[s * o + j] += b[j];
        orc_apply_activation(C, N, o, n->act[l - 1]);
        A = C;
    }
}

void orc_forward_batch(const orc_net *n, const float *X, uint32_t N, float *out)
{
    uint32_t mw = max_width(n);
    float *a = (float *)malloc(4u * (size_t)mw * N), *b = (float *)malloc(4u * (size_t)mw * N);
    /* plain k-sequential FP32 sums: single-threaded, unblocked */
    const float *A = X;
    for (uint32_t l = 1; l < n->layers; ++l) {
        uint32_t in = n->topology[l - 1], o = n->topology[l];
        const float *W = n->weights + n->woff[l - 1], *bias = n->biases + n->boff[l - 1];
        float *C = (l == n->layers - 1) ? out : ((l & 1u) ? a : b);
        for (uint64_t s = 0; s < N; ++s)
            for (uint32_t j = 0; j < o; ++j) {
                float acc = 0.0f;
                const float *xr = A + s * in, *wr = W + (uint64_t)j * in;
                for (uint32_t k = 0; k < in; ++k) acc += xr[k] * wr[k];
                C[s * o + j] = acc + bias[j];
            }
        orc_apply_activation(C, N, o, n->act[l - 1]);
        A = C;
    }
    free(a); free(b);
}

static double act_f64(double x, int act)
{
    switch (act) {
    case ORC_ACT_SIGMOID:    return 1.0 / (1.0 + exp(-x));
    case ORC_ACT_RELU:       return x > 0.0 ? x : 0.0;
    case ORC_ACT_TANH:       return tanh(x);
    case ORC_ACT_LEAKY_RELU: return x > 0.0 ? x : (double)0.01f * x;
    case ORC_ACT_FOO52:
        if (x > 1.0) return 1.0 + (double)0.01f * (x - 1.0);
        return x < 0.0 ? (double)0.01f * x : x;
    default:                 return x;
    }
}

void orc_forward_batch_f64(const orc_net *n, const float *X, uint32_t N, double *out)
{
    uint32_t mw = max_width(n);
    double *a = (double *)malloc(8u * (size_t)mw * N), *b = (double *)malloc(8u * (size_t)mw * N);
    for (uint64_t i = 0; i < (uint64_t)N * n->topology[0]; ++i) a[i] = X[i];
    double *A = a, *C = b;
    for (uint32_t l = 1; l < n->layers; ++l) {
        uint32_t in = n->topology[l - 1], o = n->topology[l];
        const float *W = n->weights + n->woff[l - 1], *bias = n->biases + n->boff[l - 1];
        for (uint64_t s = 0; s < N; ++s) {
            double *row = C + s * o;
            for (uint32_t j = 0; j < o; ++j) {
                double acc = bias[j];
                const double *xr = A + s * in; const float *wr = W + (uint64_t)j * in;
                for (uint32_t k = 0; k < in; ++k) acc += xr[k] * (double)wr[k];
                row[j] = acc;
            }
            if (n->act[l - 1] == ORC_ACT_SOFTMAX) {
                double m = row[0]; for (uint32_t j = 1; j < o; ++j) if (row[j] > m) m = row[j];
                double sum = 0; for (uint32_t j = 0; j < o; ++j) { row[j] = exp(row[j] - m); sum += row[j]; }
                for (uint32_t j = 0; j < o; ++j) row[j] /= sum;
            } else {
                for (uint32_t j = 0; j < o; ++j) row[j] = act_f64(row[j], n->act[l - 1]);
            }
        }
        double *t = A; A = C; C = t;
    }
    memcpy(out, A, 8u * (size_t)N * n->topology[n->layers - 1]);
    free(a); free(b);
}

/* ------------------------------------------------------------------ evaluation */
/* SIMD.c:522-552 (compute_sample_loss) */
float orc_sample_loss(const float *output, const float *target, uint32_t width, int loss, int output_act)
{
    const float eps = 1e-9f;
    float acc = 0.0f;
    if (loss == 0) {
        for (uint32_t k = 0; k < width; ++k) {
            const float d = output[k] - target[k];
            acc += d * d;
        }
    } else if (loss == 1) {
        if (output_act == ORC_ACT_SIGMOID) {
            for (uint32_t k = 0; k < width; ++k) {
                float o = output[k];
                const float t = target[k];
                if (o < eps) o = eps;
                if (o > 1.0f - eps) o = 1.0f - eps;
                acc -= (t * logf(o) + (1.0f - t) * logf(1.0f - o));
            }
        } else {
            for (uint32_t k = 0; k < width; ++k) {
                float o = output[k];
                if (o < eps) o = eps;
                acc -= target[k] * logf(o);
            }
        }
    }
    return acc;
}

/* Training.c:421-435 (batch_compute_loss) */
float orc_batch_loss(const float *outputs, const float *targets, uint32_t N, uint32_t width, int loss, int output_act)
{
    float total = 0.0f;
    for (uint32_t s = 0; s < N; ++s)
        total += orc_sample_loss(outputs + (size_t)s * width, targets + (size_t)s * width, width, loss, output_act);
    return total;
}

uint32_t orc_argmax(const float *row, uint32_t width)
{
    uint32_t best = 0;
    for (uint32_t k = 1; k < width; ++k)
        if (row[k] > row[best]) best = k;
    return best;
}


/* ------------------------------------------------------------------ batched training step */
/* Activation.c:40-56 (derivative) — the scalar form apply_derivative_batch (SIMD.c:90-188)
 * multiplies by; its argument is the activation's OUTPUT. */
float orc_derivative(float a, int act)
{
    switch (act) {
    case ORC_ACT_RELU:       return a > 0.0f ? 1.0f : 0.0f;
    case ORC_ACT_LEAKY_RELU: return a > 0.0f ? 1.0f : 0.01f;
    case ORC_ACT_SIGMOID:
    case ORC_ACT_SOFTMAX:    return a * (1.0f - a);
    case ORC_ACT_TANH:       return 1.0f - a * a;
    case ORC_ACT_FOO52:      return (a > 1.0f || a < 0.0f) ? 0.01f : 1.0f;
    default:                 return 1.0f;
    }
}

/* batch_forward keeping every layer (Training.c:313-345 with the BatchWorkspace of :254-311),
 * batch_compute_deltas (:347-394) and batch_accumulate_gradients (:396-419).  The three matrix
 * products are summed in double and rounded once (the reference calls sgemm; neither its
 * blocking nor its summation order is restated).  gW / gB are laid out like weights / biases. */
void orc_batch_gradients(const orc_net *n, const float *X, const float *T, uint32_t N, float grad_scale,
                         float *gW, float *gB, float *outputs)
{
    const uint32_t last = n->layers - 1;
    float **act = (float **)calloc(n->layers, sizeof(float *));
    float **delta = (float **)calloc(n->layers, sizeof(float *));
    act[0] = (float *)X;
    for (uint32_t l = 1; l <= last; ++l) {
        act[l] = (float *)malloc(4u * (size_t)N * n->topology[l]);
        delta[l] = (float *)malloc(4u * (size_t)N * n->topology[l]);
    }
    for (uint32_t l = 1; l <= last; ++l) {
        const uint32_t in = n->topology[l - 1], o = n->topology[l];
        const float *W = n->weights + n->woff[l - 1], *b = n->biases + n->boff[l - 1];
        for (uint64_t s = 0; s < N; ++s)
            for (uint32_t j = 0; j < o; ++j) {
                double acc = 0.0;
                for (uint32_t k = 0; k < in; ++k) acc += (double)act[l - 1][s * in + k] * (double)W[(uint64_t)j * in + k];
                act[l][s * o + j] = (float)acc + b[j];
            }
        orc_apply_activation(act[l], N, o, n->act[l - 1]);
    }
    const uint32_t n_out = n->topology[last];
    const int last_act = n->act[last - 1];
    if (outputs) memcpy(outputs, act[last], 4u * (size_t)N * n_out);

    /* output layer (Training.c:357-378) */
    if (n->loss == 0 && last_act == ORC_ACT_SOFTMAX) {
        for (uint64_t s = 0; s < N; ++s) {
            const float *a = act[last] + s * n_out, *t = T + s * n_out;
            float *d = delta[last] + s * n_out;
            float sum = 0.0f;
            for (uint32_t j = 0; j < n_out; ++j) sum += (a[j] - t[j]) * a[j];
            for (uint32_t j = 0; j < n_out; ++j) d[j] = a[j] * ((a[j] - t[j]) - sum);
        }
    } else if (n->loss == 1 && (last_act == ORC_ACT_SOFTMAX || last_act == ORC_ACT_SIGMOID)) {
        for (uint64_t i = 0; i < (uint64_t)N * n_out; ++i) delta[last][i] = act[last][i] + -1.0f * T[i];
    } else {
        for (uint64_t i = 0; i < (uint64_t)N * n_out; ++i)
            delta[last][i] = (act[last][i] - T[i]) * orc_derivative(act[last][i], last_act);
    }
    /* hidden layers (Training.c:380-393): delta_l = (delta_{l+1} W_{l+1}) .* f'(act_l) */
    for (uint32_t l = last - 1; l > 0; --l) {
        const uint32_t cur = n->topology[l], nxt = n->topology[l + 1];
        const float *W = n->weights + n->woff[l];
        for (uint64_t s = 0; s < N; ++s)
            for (uint32_t k = 0; k < cur; ++k) {
                double acc = 0.0;
                for (uint32_t j = 0; j < nxt; ++j) acc += (double)delta[l + 1][s * nxt + j] * (double)W[(uint64_t)j * cur + k];
                delta[l][s * cur + k] = (float)acc * orc_derivative(act[l][s * cur + k], n->act[l - 1]);
            }
    }
    /* gradients (Training.c:399-418): gW = scale * delta^T act, gB = scale * delta^T ones */
    for (uint32_t l = 0; l < last; ++l) {
        const uint32_t in = n->topology[l], o = n->topology[l + 1];
        float *gw = gW + n->woff[l], *gb = gB + n->boff[l];
        for (uint32_t j = 0; j < o; ++j) {
            for (uint32_t k = 0; k < in; ++k) {
                double acc = 0.0;
                for (uint64_t s = 0; s < N; ++s) acc += (double)delta[l + 1][s * o + j] * (double)act[l][s * in + k];
                gw[(uint64_t)j * in + k] = (float)((double)grad_scale * acc);
            }
            double accb = 0.0;
            for (uint64_t s = 0; s < N; ++s) accb += (double)delta[l + 1][s * o + j];
            gb[j] = (float)((double)grad_scale * accb);
        }
    }
    for (uint32_t l = 1; l <= last; ++l) { free(act[l]); free(delta[l]); }
    free(act); free(delta);
}

/* spingalett_clip_grad_norm (SIMD.c:496-520); the squares are added in double here. */
float orc_clip_grad_norm(const orc_net *n, float *gW, float *gB, float max_norm)
{
    if (max_norm <= 0.0f) return 0.0f;
    double total = 0.0;
    for (uint64_t i = 0; i < n->total_weights; ++i) total += (double)gW[i] * (double)gW[i];
    for (uint64_t i = 0; i < n->total_biases; ++i) total += (double)gB[i] * (double)gB[i];
    const float norm = sqrtf((float)total);
    if (norm > max_norm) {
        const float scale = max_norm / norm;
        for (uint64_t i = 0; i < n->total_weights; ++i) gW[i] *= scale;
        for (uint64_t i = 0; i < n->total_biases; ++i) gB[i] *= scale;
    }
    return norm;
}

/* one array of apply_gradients_batch_prescaled (Training.c:439-507) with the update rules of
 * SIMD.c:279-494 in their scalar form; decay is 0 for bias arrays as at the call sites. */
static void opt_update(const orc_opt_args *a, float *W, float *g, float *m, float *v, uint64_t cnt, float decay,
                       float beta1_pow_t, float beta2_pow_t)
{
    const float lr = a->learning_rate, b1 = a->beta1, b2 = a->beta2, eps = a->epsilon;
    const float omb1 = 1.0f - b1, omb2 = 1.0f - b2;
    switch (a->optimizer) {
    case ORC_OPT_SGD:
        for (uint64_t i = 0; i < cnt; ++i) {
            if (decay > 0.0f) W[i] -= lr * (g[i] + decay * W[i]);     /* sgd_decay_update, SIMD.c:401-422 */
            else W[i] -= lr * g[i];                                   /* sgd_update, :384-399 */
        }
        break;
    case ORC_OPT_MOMENTUM:                                            /* :424-453 */
        for (uint64_t i = 0; i < cnt; ++i) {
            m[i] = a->momentum * m[i] + decay * W[i] + g[i];
            W[i] -= lr * m[i];
        }
        break;
    case ORC_OPT_ADAM:
    case ORC_OPT_ADAMW: {
        const float mf = 1.0f / (1.0f - beta1_pow_t), vf = 1.0f / (1.0f - beta2_pow_t);
        const int adamw = a->optimizer == ORC_OPT_ADAMW;
        const float wd = (adamw && decay > 0.0f) ? 1.0f - lr * decay : 1.0f;
        for (uint64_t i = 0; i < cnt; ++i) {
            if (!adamw && decay > 0.0f) g[i] += decay * W[i];         /* vec_axpy at Training.c:489-491 */
            m[i] = b1 * m[i] + omb1 * g[i];                           /* adam / adamw update, SIMD.c:279-382 */
            v[i] = b2 * v[i] + omb2 * (g[i] * g[i]);
            const float m_hat = m[i] * mf, v_hat = v[i] * vf + eps;
            if (adamw && decay > 0.0f) W[i] = W[i] * wd - lr * (m_hat / sqrtf(v_hat));
            else W[i] -= lr * (m_hat / sqrtf(v_hat));
        }
        break;
    }
    case ORC_OPT_RMSPROP:                                             /* :455-494 */
        for (uint64_t i = 0; i < cnt; ++i) {
            if (a->decay_in_grad) {                                   /* backpropagation(), Training.c:196-211 */
                float grad = g[i];
                if (decay > 0.0f) grad += decay * W[i];
                v[i] = b2 * v[i] + omb2 * (grad * grad);
                W[i] -= lr * grad / sqrtf(v[i] + eps);
                continue;
            }
            v[i] = b2 * v[i] + omb2 * (g[i] * g[i]);
            const float v_hat = v[i] + eps;
            W[i] -= lr * (decay * W[i] + g[i] / sqrtf(v_hat));
        }
        break;
    default: break;
    }
}

void orc_apply_gradients(orc_net *n, const orc_opt_args *a, float *gW, float *gB, float *mW, float *vW,
                         float *mB, float *vB, float beta1_pow_t, float beta2_pow_t)
{
    if (a->max_grad_norm > 0.0f) orc_clip_grad_norm(n, gW, gB, a->max_grad_norm);
    for (uint32_t l = 0; l + 1 < n->layers; ++l) {
        const uint64_t wc = (uint64_t)n->topology[l] * n->topology[l + 1], bc = n->topology[l + 1];
        const uint64_t wo = n->woff[l], bo = n->boff[l];
        opt_update(a, n->weights + wo, gW + wo, mW + wo, vW + wo, wc, a->weight_decay, beta1_pow_t, beta2_pow_t);
        opt_update(a, n->biases + bo, gB + bo, mB + bo, vB + bo, bc, 0.0f, beta1_pow_t, beta2_pow_t);
    }
}

double orc_time_forward_batch(const orc_net *n, const float *X, uint32_t N, float *out,
                              int iters, void *sgemm_fn, int threads)
{
#if defined(_OPENMP)
    if (threads > 0) omp_set_num_threads(threads);
#else
    (void)threads;
#endif
    uint32_t mw = max_width(n);
    float *a = (float *)malloc(4u * (size_t)mw * N), *b = (float *)malloc(4u * (size_t)mw * N);
    forward_batch_impl(n, X, N, out, (sgemm_t)sgemm_fn, a, b);      /* warm-up */
    struct timespec t0, t1;
    clock_gettime(CLOCK_MONOTONIC, &t0);
    for (int i = 0; i < iters; ++i) forward_batch_impl(n, X, N, out, (sgemm_t)sgemm_fn, a, b);
    clock_gettime(CLOCK_MONOTONIC, &t1);
    free(a); free(b);
    return ((double)(t1.tv_sec - t0.tv_sec) + 1e-9 * (double)(t1.tv_nsec - t0.tv_nsec)) / (iters > 0 ? iters : 1);
}

/* CPU-baseline leg of the public single-sample forward (Network.c:218-247): per layer y = bias (memcpy, :227), then
 * either cblas_sgemv NoTrans with alpha = beta = 1 (:229-236) or an OpenMP loop over the output rows, each a dot
 * product with four 8-wide accumulators over 32-float blocks and a scalar tail (:238-245 with SIMD.c:190-240), then
 * the activation (:247). */
typedef void (*sgemv_t)(int order, int trans, int m, int n, float alpha, const float *a, int lda, const float *x,
                        int incx, float beta, float *y, int incy);

static float dot_rows(const float *a, const float *b, uint32_t n)
{
    float p[4][8] = {{0}};
    uint32_t k = 0;
    for (; k + 32 <= n; k += 32)
        for (int u = 0; u < 4; ++u)
            for (int v = 0; v < 8; ++v) p[u][v] += a[k + 8 * u + v] * b[k + 8 * u + v];
    for (; k + 8 <= n; k += 8)
        for (int v = 0; v < 8; ++v) p[0][v] += a[k + v] * b[k + v];
    float q[8];
    for (int v = 0; v < 8; ++v) q[v] = (p[0][v] + p[1][v]) + (p[2][v] + p[3][v]);
    float acc = ((q[0] + q[4]) + (q[1] + q[5])) + ((q[2] + q[6]) + (q[3] + q[7]));
    for (; k < n; ++k) acc += a[k] * b[k];
    return acc;
}

static void forward_single_impl(const orc_net *n, const float *x, float *out, sgemv_t gemv, float *cur, float *nxt)
{
    memcpy(cur, x, 4u * (size_t)n->topology[0]);
    for (uint32_t l = 1; l < n->layers; ++l) {
        const uint32_t in = n->topology[l - 1], o = n->topology[l];
        const float *W = n->weights + n->woff[l - 1], *b = n->biases + n->boff[l - 1];
        memcpy(nxt, b, 4u * (size_t)o);
        if (gemv) {
            gemv(101 /* row major */, 111 /* no transpose */, (int)o, (int)in, 1.0f, W, (int)in, cur, 1, 1.0f, nxt, 1);
        } else {
#if defined(_OPENMP)
#pragma omp parallel for schedule(static)
#endif
            for (int64_t j = 0; j < (int64_t)o; ++j) nxt[j] += dot_rows(cur, W + (uint64_t)j * in, in);
        }
        orc_apply_activation(nxt, 1, o, n->act[l - 1]);
        float *t = cur; cur = nxt; nxt = t;
    }
    memcpy(out, cur, 4u * (size_t)n->topology[n->layers - 1]);
}

double orc_time_forward_single(const orc_net *n, const float *x, float *out, int iters, void *sgemv_fn, int threads)
{
#if defined(_OPENMP)
    if (threads > 0) omp_set_num_threads(threads);
#else
    (void)threads;
#endif
    uint32_t mw = max_width(n);
    float *a = (float *)malloc(4u * (size_t)mw), *b = (float *)malloc(4u * (size_t)mw);
    forward_single_impl(n, x, out, (sgemv_t)sgemv_fn, a, b);       /* warm-up */
    struct timespec t0, t1;
    clock_gettime(CLOCK_MONOTONIC, &t0);
    for (int i = 0; i < iters; ++i) forward_single_impl(n, x, out, (sgemv_t)sgemv_fn, a, b);
    clock_gettime(CLOCK_MONOTONIC, &t1);
    free(a); free(b);
    return ((double)(t1.tv_sec - t0.tv_sec) + 1e-9 * (double)(t1.tv_nsec - t0.tv_nsec)) / (iters > 0 ? iters : 1);
}
