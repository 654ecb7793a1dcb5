/*
 * sp_internal.h — declarations shared by the host-side C sources.
 */
#ifndef SP_INTERNAL_H
#define SP_INTERNAL_H

#include "spingalett.h"
#include "spingalett_hip.h"

#define SP_ERRMSG_MAX 256
#define SP_ALIGNMENT  64           /* host arrays, as Memory.c:10-22 */
#define SP_NET_MAGIC  0x53504E47u  /* "SPNG" */

/* One serialized array kept from a loaded file (Serialize.c:87-193 layout):
 * `codes` points at the bytes after the 4-byte scale of the integer formats. */
typedef struct {
    const uint8_t *codes;
    size_t         bytes;
    float          max_val;
} sp_packed_array;

/* The library allocates every NeuralNetwork itself (Network.c:41), so the
 * public record can be the first member of a larger private one. */
typedef struct {
    NeuralNetwork    pub;
    uint32_t         magic;
    /* arrays retained from load_spingalett(); NULL for nets built by layer() */
    uint8_t         *file_blob;
    size_t           file_bytes;
    PrecisionMode    packed_precision;
    sp_packed_array *packed_w;      /* [layers-1] */
    sp_packed_array *packed_b;      /* [layers-1] */
    bool             opt_loaded;    /* opt_m / opt_v / grad_* may hold content: a file's optimizer block was read
                                       into them, or train() copied the device's gradients and moments back */
    int              act_mode;      /* SpingalettNetActivations: this net's own choice of activation type */
    /* device side */
    sphip_net       *dev;
    PrecisionMode    dev_precision;
} sp_net;

/* The private record of a net this library allocated and has not freed, else NULL.  Nothing past the
 * public part of a caller's NeuralNetwork is read before the pointer has been found in the library's own
 * table of live nets (sp_network.c). */
sp_net *sp_owned(const NeuralNetwork *net);

/* sp_runtime.c */
void  sp_set_error(int code, const char *msg);
void  sp_log(LogLevel level, const char *fmt, ...) __attribute__((format(printf, 2, 3)));
void *sp_aligned_calloc(size_t count, size_t elem_size);
void  sp_aligned_free(void *p);
ComputeMode sp_resolve_compute_mode(void);
extern const char *const sp_act_names[];
extern const char *const sp_loss_names[];
extern const char *const sp_init_names[];
extern const char *const sp_precision_names[];

/* sp_network.c */
NeuralNetwork *sp_net_build(LossFunction loss, uint32_t layers, const uint32_t *topology, const uint8_t *acts);

void sp_shuffle_indices(uint32_t *indices, uint32_t n);

/* sp_format.c */
size_t sp_array_bytes(uint64_t n, PrecisionMode p);
/* decodes one serialized array to FP32; returns false if `avail` is too small */
bool   sp_decode_array(const uint8_t *src, size_t avail, uint32_t n, PrecisionMode p,
                       SpingalettDequantMode mode, float *dst);
size_t sp_encode_array(const float *src, uint32_t n, PrecisionMode p, uint8_t *dst);
void   sp_drop_packed(sp_net *sn);

/* Spingalett.HIP.c */
void   sp_hip_release(sp_net *sn);
float *sp_hip_forward_single(sp_net *sn, const float *input);

#endif
