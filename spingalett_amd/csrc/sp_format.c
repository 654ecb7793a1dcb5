/*
 * sp_format.c — the versioned .nn container: array codecs, load, save.
 *
 * File layout (Serialize.c:348-407, little-endian, no padding):
 *   u16 version=1 | u32 layers | u8 loss | u8 has_optimizer | [u64 time_step]
 *   | u8 precision | u32 topology[L] | u8 activation[L-1]
 *   then per layer:  W [mW vW]  b [mb vb]      (bracketed only with optimizer)
 * Array encodings (Serialize.c:87-193): FP32 raw; FP16/BF16 u16 codes;
 *   INT8 f32 max + i8[n]; INT4 f32 max + packed nibbles (even index low);
 *   INT2 f32 max + packed 2-bit fields (index i at bits 2(i%4)).
 *
 * Unlike the reference loader this one keeps the file's bytes: the device is
 * fed the packed arrays, the public FP32 arrays are filled for API
 * compatibility.  Compile without fast-math: the decode expressions are
 * meant to be evaluated exactly as written.
 */
#define _GNU_SOURCE
#include "sp_internal.h"

#include <math.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

static inline uint32_t f2u(float x) { uint32_t u; memcpy(&u, &x, 4); return u; }
static inline float    u2f(uint32_t u) { float x; memcpy(&x, &u, 4); return x; }

/* ------------------------------------------------------------------ */
/* scalar conversions                                                  */
/* ------------------------------------------------------------------ */

/* half -> single, exact; NaNs lose their payload (Serialize.c:45-72) */
static float half_to_float(uint16_t h)
{
    const uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    const uint32_t exp5 = (h >> 10) & 0x1Fu;
    uint32_t frac = h & 0x3FFu;
    if (exp5 == 0x1Fu) return u2f(sign | 0x7F800000u | (frac ? 0x400000u : 0u));
    if (exp5) return u2f(sign | ((exp5 + 112u) << 23) | (frac << 13));
    if (!frac) return u2f(sign);
    uint32_t e = 113u;                       /* biased exponent of 2^-14 */
    do { frac <<= 1; --e; } while (!(frac & 0x400u));
    return u2f(sign | (e << 23) | ((frac & 0x3FFu) << 13));
}

/* single -> half by truncation (Serialize.c:12-43) */
static uint16_t float_to_half_trunc(float x)
{
    const uint32_t u = f2u(x);
    const uint16_t sign = (uint16_t)((u >> 16) & 0x8000u);
    const uint32_t exp8 = (u >> 23) & 0xFFu, frac = u & 0x7FFFFFu;
    if (exp8 == 0) return sign;                                  /* zero and FP32 subnormals */
    if (exp8 == 0xFF) return (uint16_t)(sign | (frac ? 0x7E00u : 0x7C00u));
    const int e = (int)exp8 - 127;
    if (e > 15) return (uint16_t)(sign | 0x7C00u);
    if (e < -24) return sign;
    if (e < -14) return (uint16_t)(sign | ((frac | 0x800000u) >> (-1 - e)));
    return (uint16_t)(sign | ((uint32_t)(e + 15) << 10) | (frac >> 13));
}

/* ------------------------------------------------------------------ */
/* array codecs                                                        */
/* ------------------------------------------------------------------ */

size_t sp_array_bytes(uint64_t n, PrecisionMode p)
{
    switch (p) {
    case PRECISION_FLOAT32:  return (size_t)(n * 4u);
    case PRECISION_FP16:
    case PRECISION_BFLOAT16: return (size_t)(n * 2u);
    case PRECISION_INT8:     return (size_t)(4u + n);
    case PRECISION_INT4:     return (size_t)(4u + (n + 1u) / 2u);
    case PRECISION_INT2:     return (size_t)(4u + (n + 3u) / 4u);
    default:                 return 0;
    }
}

/* Integer decode (Serialize.c:222-294).  The per-code factor is tabulated once
 * per array: strict = fl(q/d) then fl(t*max); release = fl(q * fl(max*fl(1/d))). */
static void decode_int_array(const uint8_t *codes, uint32_t n, PrecisionMode p, float max_val,
                             SpingalettDequantMode mode, float *dst)
{
    if (!(max_val > 0.0f)) {                 /* 0, negative or NaN scale: all zeros */
        memset(dst, 0, (size_t)n * sizeof(float));
        return;
    }
    const int lo = p == PRECISION_INT8 ? -128 : p == PRECISION_INT4 ? -8 : -2;
    const int cnt = p == PRECISION_INT8 ? 256 : p == PRECISION_INT4 ? 16 : 4;
    const float d = p == PRECISION_INT8 ? 127.0f : p == PRECISION_INT4 ? 7.0f : 1.0f;
    float table[256];
    for (int c = 0; c < cnt; ++c) {
        volatile float q = (float)(lo + c);
        if (p == PRECISION_INT2) {
            table[c] = q * max_val;
        } else if (mode == SPINGALETT_DEQUANT_RELEASE) {
            volatile float r = 1.0f / d;
            volatile float s = max_val * r;
            table[c] = q * s;
        } else {
            volatile float t = q / d;
            table[c] = t * max_val;
        }
    }
    if (p == PRECISION_INT8) {
        for (uint32_t i = 0; i < n; ++i) dst[i] = table[(int)(int8_t)codes[i] + 128];
    } else if (p == PRECISION_INT4) {
        for (uint32_t i = 0; i < n; ++i) {
            const unsigned nib = (codes[i >> 1] >> ((i & 1u) * 4u)) & 0xFu;
            dst[i] = table[(nib ^ 8u)];      /* two's complement nibble: index = q + 8 */
        }
    } else {
        for (uint32_t i = 0; i < n; ++i) {
            const unsigned c = (codes[i >> 2] >> ((i & 3u) * 2u)) & 3u;
            dst[i] = table[(c ^ 2u)];        /* index = q + 2 */
        }
    }
}

bool sp_decode_array(const uint8_t *src, size_t avail, uint32_t n, PrecisionMode p,
                     SpingalettDequantMode mode, float *dst)
{
    const size_t need = sp_array_bytes(n, p);
    if (avail < need) return false;
    switch (p) {
    case PRECISION_FLOAT32:
        memcpy(dst, src, need);
        return true;
    case PRECISION_FP16:
        for (uint32_t i = 0; i < n; ++i) { uint16_t h; memcpy(&h, src + 2u * (size_t)i, 2); dst[i] = half_to_float(h); }
        return true;
    case PRECISION_BFLOAT16:
        for (uint32_t i = 0; i < n; ++i) { uint16_t h; memcpy(&h, src + 2u * (size_t)i, 2); dst[i] = u2f((uint32_t)h << 16); }
        return true;
    default: {
        float max_val;
        memcpy(&max_val, src, 4);
        decode_int_array(src + 4, n, p, max_val, mode, dst);
        return true;
    }
    }
}

/* Serialize.c:87-193 */
size_t sp_encode_array(const float *src, uint32_t n, PrecisionMode p, uint8_t *dst)
{
    const size_t need = sp_array_bytes(n, p);
    if (p == PRECISION_FLOAT32) { memcpy(dst, src, need); return need; }
    if (p == PRECISION_FP16) {
        for (uint32_t i = 0; i < n; ++i) { uint16_t h = float_to_half_trunc(src[i]); memcpy(dst + 2u * (size_t)i, &h, 2); }
        return need;
    }
    if (p == PRECISION_BFLOAT16) {
        for (uint32_t i = 0; i < n; ++i) { uint16_t h = (uint16_t)(f2u(src[i]) >> 16); memcpy(dst + 2u * (size_t)i, &h, 2); }
        return need;
    }
    float max_val = 0.0f;
    for (uint32_t i = 0; i < n; ++i) { const float a = fabsf(src[i]); if (a > max_val) max_val = a; }
    memcpy(dst, &max_val, 4);
    uint8_t *codes = dst + 4;
    memset(codes, 0, need - 4u);
    if (!(max_val > 0.0f)) return need;
    for (uint32_t i = 0; i < n; ++i) {
        volatile float ratio = src[i] / max_val;
        if (p == PRECISION_INT8) {
            volatile float scaled = ratio * 127.0f;
            codes[i] = (uint8_t)(int8_t)roundf(scaled);
        } else if (p == PRECISION_INT4) {
            volatile float scaled = ratio * 7.0f;
            int q = (int8_t)roundf(scaled);
            q = q > 7 ? 7 : (q < -8 ? -8 : q);
            codes[i >> 1] |= (uint8_t)(((unsigned)q & 0xFu) << ((i & 1u) * 4u));
        } else {
            const int q = ratio > 0.5f ? 1 : (ratio < -0.5f ? -1 : 0);
            codes[i >> 2] |= (uint8_t)(((unsigned)q & 3u) << ((i & 3u) * 2u));
        }
    }
    return need;
}

void sp_drop_packed(sp_net *sn)
{
    free(sn->file_blob);
    free(sn->packed_w);
    free(sn->packed_b);
    sn->file_blob = NULL;
    sn->file_bytes = 0;
    sn->packed_w = sn->packed_b = NULL;
    sn->packed_precision = PRECISION_FLOAT32;
}

/* ------------------------------------------------------------------ */
/* load                                                                */
/* ------------------------------------------------------------------ */

typedef struct { const uint8_t *p; size_t left; } cursor;

static bool take(cursor *c, void *dst, size_t n)
{
    if (c->left < n) return false;
    memcpy(dst, c->p, n);
    c->p += n;
    c->left -= n;
    return true;
}

/* Reads one array into dst; fills `keep` (may be NULL) with where its codes sit.
 * A short FP32 array keeps its leading whole values (fread semantics at
 * Serialize.c:197); other formats decode nothing when short (:203-208). */
static bool read_array(cursor *c, uint32_t n, PrecisionMode p, SpingalettDequantMode mode,
                       float *dst, sp_packed_array *keep)
{
    const size_t need = sp_array_bytes(n, p);
    if (c->left < need) {
        if (p == PRECISION_FLOAT32) memcpy(dst, c->p, c->left & ~(size_t)3u);
        c->p += c->left;
        c->left = 0;
        return false;
    }
    sp_decode_array(c->p, c->left, n, p, mode, dst);
    if (keep) {
        const bool scaled = p >= PRECISION_INT8;
        keep->codes = c->p + (scaled ? 4 : 0);
        keep->bytes = need - (scaled ? 4u : 0u);
        keep->max_val = 0.0f;
        if (scaled) memcpy(&keep->max_val, c->p, 4);
    }
    c->p += need;
    c->left -= need;
    return true;
}

/* Takes ownership of blob (freed on failure). */
static NeuralNetwork *load_from_blob(uint8_t *blob, size_t bytes, const char *label)
{
    cursor c = {blob, bytes};
#define FAIL(msg) do { sp_set_error(SPINGALETT_ERR_INVALID, msg); free(blob); return NULL; } while (0)
    uint16_t version = 0;
    if (!take(&c, &version, 2)) FAIL("load: failed to read format version");
    if (version != SPINGALETT_FORMAT_VERSION) {
        sp_log(LOG_ERROR, "Unsupported file format version %u (expected %u)", (unsigned)version,
               (unsigned)SPINGALETT_FORMAT_VERSION);
        FAIL("load: unsupported format version");
    }
    uint32_t layers = 0;
    if (!take(&c, &layers, 4)) FAIL("load: failed to read layer count");
    if (layers < 2) FAIL("load: network must have at least 2 layers");
    uint8_t loss = 0, has_opt = 0, prec = 0;
    if (!take(&c, &loss, 1) || loss >= LOSS_COUNT) FAIL("load: invalid loss type");
    if (!take(&c, &has_opt, 1)) FAIL("load: failed to read optimizer flag");
    uint64_t time_step = 0;
    if (has_opt && !take(&c, &time_step, 8)) FAIL("load: failed to read time step");
    if (!take(&c, &prec, 1) || prec >= PRECISION_COUNT) FAIL("load: invalid precision type");
    if (c.left / 4u < layers) FAIL("load: failed to read topology");
    const uint8_t *topo_raw = c.p;                    /* unaligned in the file: copied, never read in place */
    uint32_t *topology = (uint32_t *)malloc((size_t)layers * 4u);
    uint8_t *acts = (uint8_t *)malloc(layers - 1);
    if (!topology || !acts) {
        free(topology); free(acts); free(blob);
        sp_set_error(SPINGALETT_ERR_ALLOC, "load: topology allocation failed");
        return NULL;
    }
    memcpy(topology, topo_raw, (size_t)layers * 4u);
    c.p += (size_t)layers * 4u;
    c.left -= (size_t)layers * 4u;
    bool bad = false;
    for (uint32_t i = 0; i + 1 < layers && !bad; ++i)
        if (!take(&c, &acts[i], 1) || acts[i] >= ACT_COUNT) bad = true;
    for (uint32_t l = 0; l < layers && !bad; ++l) {
        if (topology[l] == 0) bad = true;                /* layer() rejects empty layers (Network.c:53) */
        if (l && (uint64_t)topology[l - 1] * topology[l] > 0xFFFFFFFFull) bad = true;
    }
    if (bad) {
        free(topology); free(acts);
        FAIL("load: invalid activation function or layer size");
    }
#undef FAIL

    /* The reference builds the net with layer() and then tests the sticky error
     * slot without clearing it first (Serialize.c:556): an error left over from
     * an earlier call makes the load fail.  Kept, since callers may rely on it. */
    if (spingalett_last_error_code() != SPINGALETT_OK) {
        free(topology); free(acts); free(blob);
        return NULL;
    }
    NeuralNetwork *net = sp_net_build((LossFunction)loss, layers, topology, acts);
    free(topology);
    free(acts);
    if (!net) {
        free(blob);
        sp_set_error(SPINGALETT_ERR_ALLOC, "load: network creation failed");
        return NULL;
    }
    net->time_step = time_step;
    sp_net *sn = sp_owned(net);           /* sp_net_build() just made it */
    sn->packed_w = (sp_packed_array *)calloc(layers - 1, sizeof(sp_packed_array));
    sn->packed_b = (sp_packed_array *)calloc(layers - 1, sizeof(sp_packed_array));
    if (!sn->packed_w || !sn->packed_b) {
        free(blob);
        free_network(net);
        sp_set_error(SPINGALETT_ERR_ALLOC, "load: descriptor allocation failed");
        return NULL;
    }
    sn->file_blob = blob;
    sn->file_bytes = bytes;
    sn->packed_precision = (PrecisionMode)prec;
    sn->opt_loaded = has_opt != 0;

    const SpingalettDequantMode mode = spingalett_get_dequant_mode();
    const PrecisionMode p = (PrecisionMode)prec;
    bool ok = true;
    for (uint32_t l = 0; l + 1 < layers && ok; ++l) {
        const uint32_t wcount = net->topology[l] * net->topology[l + 1], bcount = net->topology[l + 1];
        const uint64_t wo = net->weight_offsets[l], bo = net->bias_offsets[l];
        ok = read_array(&c, wcount, p, mode, net->weights + wo, &sn->packed_w[l]);
        if (ok && has_opt)
            ok = read_array(&c, wcount, p, mode, net->opt_m_weights + wo, NULL)
              && read_array(&c, wcount, p, mode, net->opt_v_weights + wo, NULL);
        if (ok) ok = read_array(&c, bcount, p, mode, net->biases + bo, &sn->packed_b[l]);
        if (ok && has_opt)
            ok = read_array(&c, bcount, p, mode, net->opt_m_biases + bo, NULL)
              && read_array(&c, bcount, p, mode, net->opt_v_biases + bo, NULL);
    }
    if (!ok) {                                   /* Serialize.c:596-599: the net is still returned */
        sp_set_error(SPINGALETT_ERR_INVALID, "load: file appears truncated or corrupt");
        sp_log(LOG_WARNING, "Network file may be truncated: %s", label);
        sp_drop_packed(sn);                      /* incomplete: the device will be fed the FP32 arrays */
    }
    sp_log(LOG_INFO, "Network loaded from %s", label);
    sp_log(LOG_INFO, "Load info: format=v%u, layers=%u, weights=%llu, biases=%llu, precision=%s, optimizer=%s",
           (unsigned)version, layers, (unsigned long long)net->total_weights, (unsigned long long)net->total_biases,
           sp_precision_names[prec], has_opt ? "ON" : "OFF");
    return net;
}

NeuralNetwork *load_spingalett(const char *filename)
{
    if (!filename) {
        sp_set_error(SPINGALETT_ERR_INVALID, "load: filename is NULL");
        return NULL;
    }
    FILE *fp = fopen(filename, "rb");
    if (!fp) {
        sp_set_error(SPINGALETT_ERR_INVALID, "load: cannot open file for reading");
        return NULL;
    }
    size_t cap = 1u << 16, len = 0;
    if (fseek(fp, 0, SEEK_END) == 0) {
        const long end = ftell(fp);
        if (end > 0) cap = (size_t)end;
        rewind(fp);
    }
    uint8_t *blob = (uint8_t *)malloc(cap ? cap : 1);
    while (blob) {
        const size_t got = fread(blob + len, 1, cap - len, fp);
        len += got;
        if (len < cap || got == 0) break;
        uint8_t *bigger = (uint8_t *)realloc(blob, cap * 2);   /* unseekable stream */
        if (!bigger) { free(blob); blob = NULL; break; }
        blob = bigger;
        cap *= 2;
    }
    fclose(fp);
    if (!blob) {
        sp_set_error(SPINGALETT_ERR_ALLOC, "load: file buffer allocation failed");
        return NULL;
    }
    return load_from_blob(blob, len, filename);
}

NeuralNetwork *load_spingalett_memory(const void *data, size_t bytes)
{
    if (!data) {
        sp_set_error(SPINGALETT_ERR_INVALID, "load: data is NULL");
        return NULL;
    }
    uint8_t *blob = (uint8_t *)malloc(bytes ? bytes : 1);
    if (!blob) {
        sp_set_error(SPINGALETT_ERR_ALLOC, "load: file buffer allocation failed");
        return NULL;
    }
    memcpy(blob, data, bytes);
    return load_from_blob(blob, bytes, "<memory>");
}

/* ------------------------------------------------------------------ */
/* save (Serialize.c:307-424)                                          */
/* ------------------------------------------------------------------ */

static bool write_array(FILE *fp, const float *src, uint32_t n, PrecisionMode p, uint8_t **scratch, size_t *cap)
{
    const size_t need = sp_array_bytes(n, p);
    if (need > *cap) {
        uint8_t *s = (uint8_t *)realloc(*scratch, need);
        if (!s) { sp_set_error(SPINGALETT_ERR_ALLOC, "save: write buffer allocation failed"); return false; }
        *scratch = s;
        *cap = need;
    }
    sp_encode_array(src, n, p, *scratch);
    return fwrite(*scratch, 1, need, fp) == need;
}

void save_spingalett_struct_arguments(SaveArgs args)
{
    if (!args.net || !args.filename) {
        sp_set_error(SPINGALETT_ERR_INVALID, "save: net or filename is NULL");
        return;
    }
    if ((unsigned)args.precision >= PRECISION_COUNT) {
        sp_set_error(SPINGALETT_ERR_INVALID, "save: invalid precision mode");
        return;
    }
    /* ".nn" is appended when the last path component has no dot (Serialize.c:321-336) */
    const char *name = args.filename;
    const char *slash = strrchr(name, '/'), *bslash = strrchr(name, '\\');
    const char *sep = (slash && bslash) ? (slash > bslash ? slash : bslash) : (slash ? slash : bslash);
    const char *dot = strrchr(name, '.');
    char *owned = NULL;
    if (!(dot && (!sep || dot > sep))) {
        owned = (char *)malloc(strlen(name) + 4);
        if (!owned) { sp_set_error(SPINGALETT_ERR_ALLOC, "save: filename allocation failed"); return; }
        sprintf(owned, "%s.nn", name);
        name = owned;
    }
    FILE *fp = fopen(name, "wb");
    if (!fp) {
        sp_set_error(SPINGALETT_ERR_INVALID, "save: cannot open file for writing");
        free(owned);
        return;
    }
    const NeuralNetwork *net = args.net;
    const uint8_t has_opt = args.do_not_save_optimizer ? 0 : 1;
    uint8_t head[32];
    size_t h = 0;
    const uint16_t version = SPINGALETT_FORMAT_VERSION;
    memcpy(head + h, &version, 2); h += 2;
    memcpy(head + h, &net->layers, 4); h += 4;
    head[h++] = (uint8_t)net->loss_func;
    head[h++] = has_opt;
    if (has_opt) { memcpy(head + h, &net->time_step, 8); h += 8; }
    head[h++] = (uint8_t)args.precision;
    bool ok = fwrite(head, 1, h, fp) == h;
    ok = ok && fwrite(net->topology, 4, net->layers, fp) == net->layers;
    for (uint32_t i = 0; i + 1 < net->layers && ok; ++i) {
        const uint8_t a = (uint8_t)net->act_func[i];
        ok = fwrite(&a, 1, 1, fp) == 1;
    }
    if (!ok) {
        sp_set_error(SPINGALETT_ERR_INVALID, "save: failed to write header");
        sp_log(LOG_ERROR, "Failed to write file header to %s", name);
        fclose(fp);
        free(owned);
        return;
    }
    uint8_t *scratch = NULL;
    size_t cap = 0;
    const PrecisionMode p = args.precision;
    for (uint32_t l = 0; l + 1 < net->layers && ok; ++l) {
        const uint32_t wcount = net->topology[l] * net->topology[l + 1], bcount = net->topology[l + 1];
        const uint64_t wo = net->weight_offsets[l], bo = net->bias_offsets[l];
        ok = write_array(fp, net->weights + wo, wcount, p, &scratch, &cap);
        if (ok && has_opt)
            ok = write_array(fp, net->opt_m_weights + wo, wcount, p, &scratch, &cap)
              && write_array(fp, net->opt_v_weights + wo, wcount, p, &scratch, &cap);
        if (ok) ok = write_array(fp, net->biases + bo, bcount, p, &scratch, &cap);
        if (ok && has_opt)
            ok = write_array(fp, net->opt_m_biases + bo, bcount, p, &scratch, &cap)
              && write_array(fp, net->opt_v_biases + bo, bcount, p, &scratch, &cap);
    }
    free(scratch);
    if (fclose(fp) != 0) ok = false;
    if (!ok) {
        sp_set_error(SPINGALETT_ERR_INVALID, "save: write error (disk full?)");
        sp_log(LOG_ERROR, "Write error saving to %s", name);
    } else {
        sp_log(LOG_INFO, "Network saved to %s", name);
        sp_log(LOG_INFO, "Save info: format=v%u, layers=%u, weights=%llu, biases=%llu, precision=%s, optimizer=%s",
               (unsigned)version, net->layers, (unsigned long long)net->total_weights,
               (unsigned long long)net->total_biases, sp_precision_names[p], has_opt ? "ON" : "OFF");
    }
    free(owned);
}
