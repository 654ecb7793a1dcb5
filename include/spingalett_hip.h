/*
 * spingalett_hip.h — C ABI of the kernel translation unit (hip_forward.hip).
 *
 * This is the boundary the reference's own glue would bind: plain pointers
 * and sizes, int status (0 = ok), no exceptions, no HIP types.  Each entry
 * cites the reference code whose work it takes over.
 *
 * Data held on the device per net: for every layer the weight array and the
 * bias array exactly as serialized in a .nn file (Serialize.c:87-193): raw
 * FP32, u16 FP16/BF16 codes, or packed INT8/INT4/INT2 codes; the f32 scale
 * that precedes the integer formats travels as `max_val`.  Kernels unpack in
 * their inner loops; no FP32 expansion of the weights exists on the device.
 */
#ifndef SPINGALETT_HIP_ABI_H
#define SPINGALETT_HIP_ABI_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define SPHIP_API __attribute__((visibility("default")))

typedef struct sphip_net sphip_net;

/* Shape of a net: what new_spingalett()/layer() accumulate in NeuralNetwork
 * (Spingalett.h:109-136) reduced to what inference needs.
 *   precision : PrecisionMode value of every array (Spingalett.h:93-101)
 *   act[l]    : ActivationFunction of layer l+1 (Spingalett.h:38-47)       */
typedef struct {
    uint32_t        layers;      /* including the input layer, >= 2 */
    const uint32_t *topology;    /* [layers]                        */
    const uint8_t  *act;         /* [layers-1]                      */
    uint8_t         precision;
} sphip_desc;

/* flags of sphip_forward */
#define SPHIP_X_ON_DEVICE   1u   /* x is a device pointer                       */
#define SPHIP_Y_ON_DEVICE   2u   /* y is a device pointer (call does not wait)  */
#define SPHIP_TRAIN_SAME_BATCH 4u /* sphip_train_step: reuse the host batch the previous step copied in */
#define SPHIP_FORCE_GEMM    8u   /* use the matrix-core path whatever n is      */
#define SPHIP_FORCE_GEMV   16u   /* use the vector path (n <= 64)               */
/* BF16 weights on the matrix-core path (5 samples and more) are multiplied with FP16 activations on the FP16 matrix
 * cores, against an FP16 copy of each weight array that sphip_upload_array makes (the weights times a power of two
 * that brings them into FP16's range: as many bytes again).  This flag selects BF16 activations on the BF16 matrix
 * cores instead: 8 instead of 11 significant bits between layers, a few per cent faster.  Other formats and the
 * vector path ignore it; no counterpart in the reference, whose activations are FP32. */
#define SPHIP_BF16_ACTIVATIONS 32u
/* A batch whose 16-bit activation buffers would exceed the memory-side cache (more than 128 MiB per buffer) runs as
 * equal blocks of rows, all layers per block (at most 64 MiB per buffer, a multiple of 256 rows), so that the layer
 * boundaries stay in that cache; the workspace is sized for a block.  Rows are independent, the outputs are the whole
 * batch's.  This flag runs the whole batch layer by layer instead (benchmark comparisons). */
#define SPHIP_WHOLE_BATCH 64u
/* Split activations on the matrix-core path (5 samples and more; any 16-bit or integer weight format): between the
 * layers every activation travels as two FP16 numbers, hi = the value rounded to FP16 and lo = (value - hi) 2^11, about
 * 22 significant bits together (the reference keeps FP32 activations, Training.c:313-345).  Each layer multiplies the
 * weights with both matrices (twice the matrix-core work) into FP32 partial sums that a second launch adds.  For nets
 * whose decisions hang on differences below FP16's 11 bits (many-class softmax heads); supersedes
 * SPHIP_BF16_ACTIVATIONS.
 * FP32 weights (five samples and more): the weights are split the same way (made on the first such call, six more bytes
 * per weight), and every layer runs as three FP16 products into one FP32 accumulator, hi x hi + lo x hi + hi x lo,
 * instead of on the FP32 matrix instructions: about three times their throughput, outputs as close to the
 * reference's as theirs (the dropped lo x lo term is 2^-22 of the sum).  Activations between the layers stay FP32;
 * magnitudes beyond FP16's 65504 saturate in this mode, as in every 16-bit mode. */
#define SPHIP_SPLIT_ACTIVATIONS 128u

SPHIP_API int  sphip_device_count(void);
SPHIP_API const char *sphip_last_error_string(void);   /* per thread */

/* Replaces the per-net allocation done by layer_struct_arguments
 * (Network.c:83-105) on the device side. */
SPHIP_API int  sphip_create(const sphip_desc *desc, sphip_net **out);
SPHIP_API void sphip_destroy(sphip_net *net);           /* free_network, Network.c:283 */

/* Replaces read_array_compressed (Serialize.c:195-297): instead of expanding
 * to FP32 the serialized codes are copied to the device as they are.
 *   which   : 0 weights of layer l (topology[l]*topology[l+1] elements), 1 biases
 *   codes   : the array's bytes after the 4-byte scale (host memory)
 *   max_val : the scale read from the file (ignored for FP32/FP16/BF16)     */
SPHIP_API int  sphip_upload_array(sphip_net *net, uint32_t l, int which,
                                  const void *codes, size_t bytes, float max_val);

/* Replaces forward_struct_arguments (Network.c:202-251) for n = 1 and
 * batch_forward (Training.c:313-345) for n > 1:
 *   per layer  y = act(b + W x), x row-major [n][topology[0]], y row-major
 *   [n][topology[last]], FP32.  n <= 4 runs the vector (GEMV) kernels in FP32-grade
 *   arithmetic (integer weights: exact integer dot products on the INT8 matrix
 *   cores); larger n runs the matrix-core kernels with 16-bit activations.  FP32
 *   weights always compute in FP32 (vector kernels up to n = 64). */
SPHIP_API int  sphip_forward(sphip_net *net, const float *x, uint32_t n, float *y,
                             uint32_t flags);
/* sphip_forward for callers that cannot allocate (code under HIP graph capture, tight serving loops, harnesses
 * that forbid hipMalloc).  No counterpart in the reference.  Same kernels and results as sphip_forward with
 * SPHIP_X_ON_DEVICE | SPHIP_Y_ON_DEVICE: d_x [n][in] and d_y [n][out] are device pointers, the call enqueues on the
 * library's stream and does not wait (sphip_synchronize does).  Everything a forward needs beyond those two and the
 * net's arrays (activation ping-pong buffers, softmax logits, digit planes of the integer GEMV, partial sums of K
 * splits, FP16 copies of small integer layers) is laid out in one fixed array of SPHIP_NOALLOC_SCRATCH_BYTES that each
 * GPU holds from library load until the process ends; the call makes no device or pinned allocation and frees none.
 * A batch whose workspace exceeds the array is refused with an error that names both sizes (sphip_forward takes it).
 * Nothing in the array needs clearing between calls: every kernel reads only what this call wrote.  All calls on one
 * GPU share the array, so two calls that overlap in time (from different threads) race; nets of more than 64 layers
 * are refused.  flags: SPHIP_FORCE_GEMM / SPHIP_FORCE_GEMV / SPHIP_BF16_ACTIVATIONS /
 * SPHIP_SPLIT_ACTIVATIONS only (the latter on an FP32 net only after a sphip_forward with that flag has made the
 * FP16 parts of the weights: making them allocates). */
#define SPHIP_NOALLOC_SCRATCH_BYTES (64u << 20)
SPHIP_API int  sphip_forward_noalloc(sphip_net *net, const float *d_x, uint32_t n, float *d_y, uint32_t flags);
/* The evaluation step that follows batch_forward in the reference's epoch loop, on the device:
 * forward of n samples, then per sample compute_sample_loss (SIMD.c:522-552) and the index of
 * the first largest output, then the batch total (batch_compute_loss, Training.c:421-435;
 * added in FP64 here).  Only the totals and, when asked for, n indices travel back.
 *   x, targets  : [n][in], [n][out] FP32; host memory, or both device memory with SPHIP_X_ON_DEVICE
 *   loss_func   : LossFunction value (Spingalett.h:49-53): 0 squared error, 1 cross-entropy (binary
 *                 form when the output layer is a sigmoid)
 *   total_loss  : sum of the per-sample losses;  predictions: [n] host array or NULL;
 *   correct     : samples whose prediction equals the index of the target's first largest entry, or NULL */
SPHIP_API int  sphip_evaluate(sphip_net *net, const float *x, const float *targets, uint32_t n, int loss_func,
                              uint32_t flags, float *total_loss, uint32_t *predictions, uint32_t *correct);
/* forward_struct_arguments as its callers see it (Network.c:214-250): one sample, and every
 * layer's activations (the input included) left in a host array laid out like
 * NeuralNetwork.neurons (Network.c:16-32).  One call, one wait. */
SPHIP_API int  sphip_forward_layers(sphip_net *net, const float *x, float *host_neurons);

/* The device form of the decoders in read_array_compressed
 * (Serialize.c:195-297) and fp16_to_float / bf16_to_float (:45-85): writes the
 * FP32 value of every element of one array to host memory.
 *   mode 0: ((float)q/d)*max evaluated as written; 1: q*(max*(1/d)).       */
SPHIP_API int  sphip_decode(sphip_net *net, uint32_t l, int which, int mode,
                            float *host_out);

SPHIP_API int  sphip_synchronize(void);

/* ---- batched training step (FP32 nets) ----
 * Takes over what one iteration of the reference's batched epoch loop does between
 * batch_forward and the end of apply_gradients_batch_prescaled (Training.c:735-748, 769-784):
 * forward keeping every layer (:313-345), batch_compute_deltas (:347-394),
 * batch_accumulate_gradients with grad_scale = 1/n (:396-419), optional
 * spingalett_clip_grad_norm (SIMD.c:496-520) and the optimizer update of every array
 * (Training.c:439-507, SIMD.c:279-494).  Weights, gradients and moments live on the device
 * between steps; sphip_train_get copies an array back. */
typedef struct {
    int32_t optimizer;      /* OptimizerType (Spingalett.h:76-83): 0 SGD, 1 momentum, 2 RMSprop, 3 Adam,
                               4 AdamW; negative: gradients only, nothing is updated */
    int32_t loss_func;      /* LossFunction (Spingalett.h:49-53) */
    float learning_rate, weight_decay, momentum, beta1, beta2, epsilon;
    float max_grad_norm;    /* > 0: gradients are scaled to this global L2 norm when they exceed it */
    float beta1_pow_t, beta2_pow_t;   /* beta^t of the step being applied (Training.c:743-745) */
    int32_t decay_in_grad;  /* RMSprop only.  0: the batched rule, W -= lr (decay W + g / sqrt(v + eps)) with v from g
                               (SIMD.c:455-494); 1: the per-sample rule of backpropagation(), decay W joins g before
                               v is updated (Training.c:196-211) */
} sphip_train_args;

/* arrays of sphip_train_set / sphip_train_get; layer l = 0 .. layers-2, weights row-major [out][in] */
enum { SPHIP_TRAIN_W = 0, SPHIP_TRAIN_B, SPHIP_TRAIN_MW, SPHIP_TRAIN_VW, SPHIP_TRAIN_MB, SPHIP_TRAIN_VB,
       SPHIP_TRAIN_GW, SPHIP_TRAIN_GB };

/* Allocates gradients and moments (zeroed).  The net must hold FP32 arrays and no hidden softmax
 * (train_struct_arguments rejects that too, Training.c:621-627).  Idempotent. */
SPHIP_API int  sphip_train_begin(sphip_net *net);
SPHIP_API void sphip_train_end(sphip_net *net);
SPHIP_API int  sphip_train_set(sphip_net *net, int which, uint32_t l, const float *host);
SPHIP_API int  sphip_train_get(sphip_net *net, int which, uint32_t l, float *host);
/* x [n][in], targets [n][out]: host memory, or both device memory with SPHIP_X_ON_DEVICE (then the
 * call only enqueues); with SPHIP_TRAIN_SAME_BATCH x and targets are ignored and the batch of the
 * previous host-memory step (same n) is used again without a copy.  total_loss, when not NULL, receives batch_compute_loss (Training.c:421-435)
 * of the forward before the update, and the call waits for it. */
SPHIP_API int  sphip_train_step(sphip_net *net, const float *x, const float *targets, uint32_t n,
                                const sphip_train_args *args, uint32_t flags, float *total_loss);

/* ---- measurement helpers (benchmark harness; not part of the data path) ---- */
SPHIP_API int  sphip_malloc(void **dptr, size_t bytes);
SPHIP_API int  sphip_free(void *dptr);
/* Free and total bytes of the current device's memory (hipMemGetInfo): lets a harness check that a call allocated
 * nothing. */
SPHIP_API int  sphip_device_memory(size_t *free_bytes, size_t *total_bytes);
SPHIP_API int  sphip_memcpy_h2d(void *dst, const void *src, size_t bytes);
SPHIP_API int  sphip_memcpy_d2h(void *dst, const void *src, size_t bytes);
/* A second device copy of a net's arrays (so a timing loop can rotate over
 * copies larger than the last-level cache). */
SPHIP_API int  sphip_clone(const sphip_net *src, sphip_net **out);
/* Runs `iters` forwards of n samples, rotating over nets[0..count), between two
 * HIP events recorded on the library's stream; *ms = total elapsed. */
SPHIP_API int  sphip_time_forward(sphip_net *const *nets, int count, const float *d_x,
                                  uint32_t n, float *d_y, uint32_t flags, int iters, float *ms);
/* Same for the main kernel of one layer only (layer index 1..layers-1). */
SPHIP_API int  sphip_time_layer(sphip_net *const *nets, int count, uint32_t layer,
                                uint32_t n, uint32_t flags, int iters, float *ms);
/* `iters` training steps on device-resident inputs and targets, timed like sphip_time_forward. */
SPHIP_API int  sphip_time_train_step(sphip_net *net, const float *d_x, const float *d_targets, uint32_t n,
                                     const sphip_train_args *args, int iters, float *ms);
/* Rows per pass of a forward of n samples with these flags: n, or the block size when the batch runs in blocks of rows
 * (SPHIP_WHOLE_BATCH has the rule); every layer kernel is then launched once per block. */
SPHIP_API uint32_t sphip_batch_block_rows(sphip_net *net, uint32_t n, uint32_t flags);
/* Name of the main kernel that a forward of n samples with these flags runs for the given layer (1..layers-1):
 * the library's routing evaluated without launching anything. */
SPHIP_API const char *sphip_layer_kernel_name(sphip_net *net, uint32_t layer, uint32_t n,
                                              uint32_t flags);

#ifdef __cplusplus
}
#endif
#endif /* SPINGALETT_HIP_ABI_H */
