/*
 * sp_runtime.c — process-wide settings, the per-thread error slot, logging and
 * aligned host memory.  Behaviour follows Settings.c, Error.c and Memory.c of
 * the reference; the code is this library's own.
 */
#define _GNU_SOURCE
#include "sp_internal.h"

#include <stdarg.h>
#include <stdatomic.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>
#include <sys/mman.h>

const char *const sp_act_names[] = {"Sigmoid", "ReLU", "Tanh", "Leaky ReLU", "FOO52", "Softmax", "None"};
const char *const sp_loss_names[] = {"MSE", "Cross-Entropy"};
const char *const sp_init_names[] = {"Random", "Xavier", "He", "None"};
const char *const sp_precision_names[] = {"FP32", "FP16", "BF16", "INT8", "INT4", "INT2"};

/* ---- error slot (Error.c:9-28): one per thread, sticky until cleared ---- */
static _Thread_local int  t_err_code = SPINGALETT_OK;
static _Thread_local char t_err_msg[SP_ERRMSG_MAX];

int spingalett_last_error_code(void) { return t_err_code; }
const char *spingalett_last_error_message(void) { return t_err_msg; }

void spingalett_clear_error(void)
{
    t_err_code = SPINGALETT_OK;
    t_err_msg[0] = '\0';
}

void sp_set_error(int code, const char *msg)
{
    t_err_code = code;
    snprintf(t_err_msg, sizeof t_err_msg, "%s", msg ? msg : "unknown error");
}

/* ---- settings (Settings.c:15-57): atomics shared by all threads ---- */
static _Atomic int      g_mode = COMPUTE_HIP;
static _Atomic unsigned g_threads = 0;
static _Atomic int      g_log_level = LOG_INFO;
static _Atomic(LogCallback) g_log_cb = NULL;
static _Atomic bool     g_verbose = true;
static _Atomic int      g_dequant = SPINGALETT_DEQUANT_STRICT;
static _Atomic bool     g_warned_mode = false;

ComputeMode spingalett_get_compute_mode(void) { return (ComputeMode)atomic_load(&g_mode); }

void spingalett_set_compute_mode(ComputeMode mode)
{
    if ((unsigned)mode < COMPUTE_COUNT) {
        atomic_store(&g_mode, (int)mode);
        atomic_store(&g_warned_mode, false);
    }
}

unsigned spingalett_get_num_threads(void) { return atomic_load(&g_threads); }
void spingalett_set_num_threads(unsigned n) { atomic_store(&g_threads, n); }   /* no host threads here */
void spingalett_set_log_callback(LogCallback cb) { atomic_store(&g_log_cb, cb); }
void spingalett_set_log_level(LogLevel level) { atomic_store(&g_log_level, (int)level); }
void spingalett_set_verbose(bool enabled) { atomic_store(&g_verbose, enabled); }
bool spingalett_get_verbose(void) { return atomic_load(&g_verbose); }

void spingalett_set_dequant_mode(SpingalettDequantMode mode)
{
    if (mode == SPINGALETT_DEQUANT_STRICT || mode == SPINGALETT_DEQUANT_RELEASE)
        atomic_store(&g_dequant, (int)mode);
}

SpingalettDequantMode spingalett_get_dequant_mode(void)
{
    return (SpingalettDequantMode)atomic_load(&g_dequant);
}

static _Atomic int g_bf16_act = SPINGALETT_BF16_ACTIVATIONS_FP16;

void spingalett_set_bf16_activations(SpingalettBf16Activations mode)
{
    if (mode == SPINGALETT_BF16_ACTIVATIONS_BF16 || mode == SPINGALETT_BF16_ACTIVATIONS_FP16)
        atomic_store(&g_bf16_act, (int)mode);
}

SpingalettBf16Activations spingalett_get_bf16_activations(void)
{
    return (SpingalettBf16Activations)atomic_load(&g_bf16_act);
}

/* Settings.c:82-110 maps a mode the build lacks to the one it has, with a
 * warning.  This build has exactly one back-end. */
ComputeMode sp_resolve_compute_mode(void)
{
    ComputeMode m = spingalett_get_compute_mode();
    if (m != COMPUTE_HIP && !atomic_exchange(&g_warned_mode, true))
        sp_log(LOG_WARNING, "Compute mode %d is not part of this build. Using the HIP back-end.", (int)m);
    return COMPUTE_HIP;
}

/* Settings.c:59-80 */
void sp_log(LogLevel level, const char *fmt, ...)
{
    if ((int)level < atomic_load(&g_log_level)) return;
    if (!atomic_load(&g_verbose) && level < LOG_WARNING) return;
    char line[1024];
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(line, sizeof line, fmt, ap);
    va_end(ap);
    LogCallback cb = atomic_load(&g_log_cb);
    if (cb) {
        cb(level, line);
        return;
    }
    static const char *const tags[] = {"DEBUG", "INFO", "WARN", "ERROR", "NONE"};
    fprintf(level >= LOG_WARNING ? stderr : stdout, "[%s] %s\n", tags[level < LOG_NONE ? level : LOG_NONE], line);
}

/* ---- host memory (Memory.c:10-39): 64-byte aligned, zero-filled ----
 * Large blocks come from anonymous mappings, whose pages are zero and are not
 * committed until touched: the gradient and optimizer arrays that layer()
 * allocates for API compatibility cost nothing for an inference-only net.
 * A 64-byte header in front of every block records how to release it. */
typedef struct {
    uint64_t magic;
    uint64_t map_bytes;      /* 0: heap block, else length of the mapping */
    void    *base;
} sp_block_header;

#define SP_BLOCK_MAGIC 0x5350424C4F434B21ull
#define SP_MAP_THRESHOLD ((size_t)1 << 20)
#define SP_MAP_LEAD 4096u

void *sp_aligned_calloc(size_t count, size_t elem_size)
{
    if (elem_size && count > SIZE_MAX / elem_size) return NULL;
    size_t bytes = count * elem_size;
    if (bytes == 0) bytes = SP_ALIGNMENT;
    bytes = (bytes + SP_ALIGNMENT - 1) & ~(size_t)(SP_ALIGNMENT - 1);
    uint8_t *user;
    sp_block_header h = {SP_BLOCK_MAGIC, 0, NULL};
    if (bytes >= SP_MAP_THRESHOLD) {
        size_t total = bytes + SP_MAP_LEAD;
        void *m = mmap(NULL, total, PROT_READ | PROT_WRITE, MAP_PRIVATE | MAP_ANONYMOUS, -1, 0);
        if (m == MAP_FAILED) return NULL;
        h.map_bytes = total;
        h.base = m;
        user = (uint8_t *)m + SP_MAP_LEAD;
    } else {
        void *m = aligned_alloc(SP_ALIGNMENT, bytes + SP_ALIGNMENT);
        if (!m) return NULL;
        memset(m, 0, bytes + SP_ALIGNMENT);
        h.base = m;
        user = (uint8_t *)m + SP_ALIGNMENT;
    }
    memcpy(user - sizeof h, &h, sizeof h);
    return user;
}

void sp_aligned_free(void *p)
{
    if (!p) return;
    sp_block_header h;
    memcpy(&h, (uint8_t *)p - sizeof h, sizeof h);
    if (h.magic != SP_BLOCK_MAGIC) return;     /* not ours: leave it alone */
    if (h.map_bytes) munmap(h.base, h.map_bytes);
    else free(h.base);
}
