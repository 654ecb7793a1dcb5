/* host_sanitize.c — the host side of the library (container parser, codecs, lifecycle, error slot) under
 * AddressSanitizer and UndefinedBehaviorSanitizer, on the CPU.
 *
 * Built by `make -C spingalett_amd/csrc asan` from the library's own C sources plus the stand-ins below for the
 * kernel translation unit's entry points (every one reports "no GPU": nothing here computes a forward).  The loader
 * parses bytes it did not write (Serialize.c:426-609 is the code it replaces), so besides the well-formed files of
 * every format, with and without an optimizer block, it gets every prefix of the small files and seeded bit flips
 * and byte overwrites of them.  A sanitizer report aborts the program; exit status 0 means none was raised.
 * tests/test_host_sanitizers.py builds and runs it. */
#define _GNU_SOURCE
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>
#include <unistd.h>

#include "spingalett.h"
#include "spingalett_hip.h"

/* ---- stand-ins for the kernel TU (no device in this program) ---- */
int sphip_device_count(void) { return 0; }
const char *sphip_last_error_string(void) { return "host sanitizer build: no GPU"; }
int sphip_create(const sphip_desc *d, sphip_net **o) { (void)d; (void)o; return 1; }
void sphip_destroy(sphip_net *n) { (void)n; }
int sphip_upload_array(sphip_net *n, uint32_t l, int w, const void *c, size_t b, float m) { (void)n; (void)l; (void)w; (void)c; (void)b; (void)m; return 1; }
int sphip_forward(sphip_net *n, const float *x, uint32_t k, float *y, uint32_t f) { (void)n; (void)x; (void)k; (void)y; (void)f; return 1; }
int sphip_forward_layers(sphip_net *n, const float *x, float *h) { (void)n; (void)x; (void)h; return 1; }
int sphip_evaluate(sphip_net *n, const float *x, const float *t, uint32_t k, int lf, uint32_t f, float *tl, uint32_t *p, uint32_t *c)
{ (void)n; (void)x; (void)t; (void)k; (void)lf; (void)f; (void)tl; (void)p; (void)c; return 1; }
int sphip_decode(sphip_net *n, uint32_t l, int w, int m, float *o) { (void)n; (void)l; (void)w; (void)m; (void)o; return 1; }
int sphip_synchronize(void) { return 0; }
int sphip_train_begin(sphip_net *n) { (void)n; return 1; }
void sphip_train_end(sphip_net *n) { (void)n; }
int sphip_train_set(sphip_net *n, int w, uint32_t l, const float *h) { (void)n; (void)w; (void)l; (void)h; return 1; }
int sphip_train_get(sphip_net *n, int w, uint32_t l, float *h) { (void)n; (void)w; (void)l; (void)h; return 1; }
int sphip_train_step(sphip_net *n, const float *x, const float *t, uint32_t k, const sphip_train_args *a, uint32_t f, float *tl)
{ (void)n; (void)x; (void)t; (void)k; (void)a; (void)f; (void)tl; return 1; }

/* ---- a small seeded generator (splitmix64) ---- */
static uint64_t g_state = 0x9E3779B97F4A7C15ull;
static uint64_t rnd(void)
{
    uint64_t z = (g_state += 0x9E3779B97F4A7C15ull);
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
    return z ^ (z >> 31);
}
static float rnd_unit(void) { return (float)((double)(rnd() >> 11) / 9007199254740992.0 * 2.0 - 1.0); }

static unsigned long g_loaded = 0, g_refused = 0, g_partial = 0, g_skipped = 0;

/* True when the header (Serialize.c:432-528: u16 version, u32 layers, u8 loss, u8 has_opt, [u64 step], u8 precision,
 * u32 topology[layers]) claims more than 4 M weights.  Like the reference, the loader allocates what the header says
 * before it reads the arrays (Network.c:87-105: nine FP32 arrays), so a damaged width costs gigabytes of zeroed
 * memory; that is a matter of resources, not of memory safety, and is kept out of this run. */
static int claims_too_much(const unsigned char *d, size_t bytes)
{
    if (bytes < 9) return 0;
    uint32_t layers;
    memcpy(&layers, d + 2, 4);
    size_t off = 8 + (d[7] ? 8u : 0u) + 1;
    if (layers < 2 || layers > 4096 || bytes < off + (size_t)layers * 4u) return 0;     /* refused before any allocation */
    uint64_t weights = 0, prev = 0;
    for (uint32_t l = 0; l < layers; ++l) {
        uint32_t w;
        memcpy(&w, d + off + (size_t)l * 4u, 4);
        if (l) weights += prev * (uint64_t)w;
        prev = w;
        if (weights > (4ull << 20) || w > (1u << 24)) return 1;
    }
    return 0;
}

static NeuralNetwork *make_net(const uint32_t *topo, uint32_t layers)
{
    spingalett_clear_error();
    NeuralNetwork *net = new_spingalett(.loss_func = LOSS_CROSS_ENTROPY);
    if (!net) return NULL;
    layer(.net = net, .neurons_amount = topo[0]);
    for (uint32_t l = 1; l < layers; ++l)
        layer(.net = net, .neurons_amount = topo[l], .act_func = (ActivationFunction)(l % ACT_COUNT),
              .weight_initialization = (WeightInitialization)(l % WEIGHT_INITIALIZATION_COUNT));
    for (uint64_t i = 0; i < net->total_weights; ++i) net->weights[i] = rnd_unit();
    for (uint64_t i = 0; i < net->total_biases; ++i) net->biases[i] = rnd_unit() * 0.1f;
    return net;
}

static unsigned char *slurp(const char *path, size_t *bytes)
{
    FILE *f = fopen(path, "rb");
    if (!f) return NULL;
    fseek(f, 0, SEEK_END);
    long n = ftell(f);
    fseek(f, 0, SEEK_SET);
    unsigned char *buf = (unsigned char *)malloc(n > 0 ? (size_t)n : 1);
    if (buf && fread(buf, 1, (size_t)n, f) != (size_t)n) { free(buf); buf = NULL; }
    fclose(f);
    *bytes = (size_t)n;
    return buf;
}

/* Loads a byte string; whatever comes back is walked (every array the struct claims to hold is read) and freed. */
static void try_load(const unsigned char *data, size_t bytes)
{
    if (claims_too_much(data, bytes)) { ++g_skipped; return; }
    spingalett_clear_error();
    /* an exact-size heap copy: a read past the end of the input is a report, not a silent read of neighbours */
    unsigned char *copy = (unsigned char *)malloc(bytes ? bytes : 1);
    if (!copy) abort();
    memcpy(copy, data, bytes);
    NeuralNetwork *net = load_spingalett_memory(copy, bytes);
    free(copy);
    if (!net) { ++g_refused; return; }
    if (spingalett_last_error_code() != SPINGALETT_OK) ++g_partial; else ++g_loaded;
    volatile double sink = 0.0;
    for (uint64_t i = 0; i < net->total_weights; ++i) sink += net->weights[i];
    for (uint64_t i = 0; i < net->total_biases; ++i) sink += net->biases[i];
    for (uint32_t l = 0; l < net->layers; ++l) sink += net->topology[l];
    for (uint32_t l = 0; l + 1 < net->layers; ++l) sink += (double)net->act_func[l];
    (void)spingalett_hip_precision(net);
    float x[64] = {0};
    (void)forward(.net = net, .input = x);      /* no device: must fail cleanly, not crash */
    free_network(net);
}

int main(void)
{
    spingalett_set_verbose(false);
    spingalett_set_log_level(LOG_NONE);
    char dir[] = "/tmp/sp_sanitize_XXXXXX";
    if (!mkdtemp(dir)) { perror("mkdtemp"); return 2; }
    const uint32_t topos[][4] = {{5, 7, 3, 0}, {9, 4, 0, 0}, {3, 6, 5, 2}, {16, 1, 0, 0}};
    const uint32_t nlayers[] = {3, 2, 4, 2};
    unsigned long files = 0, cuts = 0, flips = 0;
    for (int t = 0; t < 4; ++t) {
        for (int prec = 0; prec < PRECISION_COUNT; ++prec) {
            for (int with_opt = 0; with_opt < 2; ++with_opt) {
                NeuralNetwork *net = make_net(topos[t], nlayers[t]);
                if (!net) { fprintf(stderr, "make_net failed: %s\n", spingalett_last_error_message()); return 2; }
                if (with_opt) {
                    net->time_step = 17;
                    for (uint64_t i = 0; i < net->total_weights; ++i) {
                        net->opt_m_weights[i] = rnd_unit() * 0.01f;
                        net->opt_v_weights[i] = rnd_unit() * rnd_unit() * 0.001f;
                    }
                }
                char path[256];
                snprintf(path, sizeof path, "%s/n%d_p%d_o%d.nn", dir, t, prec, with_opt);
                spingalett_clear_error();
                save_spingalett(.net = net, .filename = path, .precision = (PrecisionMode)prec,
                                .do_not_save_optimizer = !with_opt);
                if (spingalett_last_error_code() != SPINGALETT_OK) {
                    fprintf(stderr, "save failed: %s\n", spingalett_last_error_message());
                    return 2;
                }
                free_network(net);
                size_t bytes = 0;
                unsigned char *blob = slurp(path, &bytes);
                if (!blob) { fprintf(stderr, "cannot read %s back\n", path); return 2; }
                ++files;
                /* the file as written, through both loaders */
                spingalett_clear_error();
                NeuralNetwork *back = load_spingalett(path);
                if (!back || spingalett_last_error_code() != SPINGALETT_OK) {
                    fprintf(stderr, "a file the library wrote did not load: %s\n", spingalett_last_error_message());
                    return 2;
                }
                free_network(back);
                try_load(blob, bytes);
                /* every prefix */
                for (size_t cut = 0; cut < bytes; ++cut) { try_load(blob, cut); ++cuts; }
                /* seeded damage: single bit flips everywhere in the header, bit flips and byte overwrites at random
                   places, each on a fresh copy */
                unsigned char *work = (unsigned char *)malloc(bytes);
                if (!work) abort();
                const size_t header = bytes < 48 ? bytes : 48;
                for (size_t pos = 0; pos < header; ++pos)
                    for (int bit = 0; bit < 8; ++bit) {
                        memcpy(work, blob, bytes);
                        work[pos] ^= (unsigned char)(1u << bit);
                        try_load(work, bytes);
                        ++flips;
                    }
                for (int k = 0; k < 64; ++k) {
                    memcpy(work, blob, bytes);
                    const int edits = 1 + (int)(rnd() % 4);
                    for (int e = 0; e < edits; ++e) {
                        const size_t pos = (size_t)(rnd() % bytes);
                        if (rnd() & 1) work[pos] ^= (unsigned char)(1u << (rnd() % 8));
                        else work[pos] = (unsigned char)rnd();
                    }
                    try_load(work, (rnd() % 4 == 0) ? (size_t)(rnd() % (bytes + 1)) : bytes);
                    ++flips;
                }
                free(work);
                free(blob);
                unlink(path);
            }
        }
    }
    /* headers that claim far more than the bytes hold: layer counts and widths at the top of their ranges */
    {
        unsigned char h[64];
        for (int k = 0; k < 2000; ++k) {
            for (size_t i = 0; i < sizeof h; ++i) h[i] = (unsigned char)rnd();
            h[0] = 1; h[1] = 0;                               /* version 1 */
            if (k & 1) { h[2] = (unsigned char)(2 + rnd() % 5); h[3] = h[4] = h[5] = 0; }   /* a plausible layer count */
            try_load(h, 8 + (size_t)(rnd() % (sizeof h - 8)));
            ++flips;
        }
    }
    /* lifecycle and argument errors on the host side */
    spingalett_clear_error();
    (void)forward(.net = NULL, .input = NULL);
    free_network(NULL);
    NeuralNetwork fake;
    memset(&fake, 0, sizeof fake);
    float x1[4] = {0};
    (void)forward(.net = &fake, .input = x1);                 /* not one of the library's nets */
    (void)load_spingalett("/nonexistent/dir/file.nn");
    (void)load_spingalett_memory(NULL, 0);
    rmdir(dir);
    printf("host_sanitize: %lu files, %lu prefixes, %lu damaged copies; %lu loaded, %lu loaded with an error, %lu refused, "
           "%lu skipped (header claims more than 4 M weights)\n", files, cuts, flips, g_loaded, g_partial, g_refused, g_skipped);
    return 0;
}
