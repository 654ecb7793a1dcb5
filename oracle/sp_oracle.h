/*
 * sp_oracle.h — CPU restatement of Spingalett's quantized-load + forward path.
 *
 * TEST INFRASTRUCTURE ONLY.  Nothing in the shipped library links, loads or
 * calls this code; it exists so that tests, the smoke check and the benchmark's
 * CPU-baseline leg have an independent statement of what the reference
 * computes.  Every function cites the reference lines it restates
 * (paths relative to the reference tree).
 *
 * Pin status (what fixes each function besides this restatement itself):
 *   orc_fp16_to_f32 / orc_bf16_to_f32 ....... pinned: all 65,536 codes against
 *        numpy's IEEE half->single conversion plus the NaN-canonicalisation
 *        rule, and against the closed form code<<16.
 *   orc_decode_array ........................ pinned: every INT8/INT4/INT2 code
 *        against IEEE float32 arithmetic done by numpy, hand-derived
 *        known-answer bytes (nibble/crumb order, sign extension, max<=0 -> 0).
 *   orc_encode_array ........................ pinned: round trips, hand-derived
 *        known answers (ties round half away from zero, INT4 clamp, ternary
 *        thresholds, FP16/BF16 truncation).
 *   orc_parse / orc_serialize ............... pinned: hand-assembled files and
 *        byte counts (8+5L header, 16+5L with optimizer block).
 *   orc_forward_* ........................... pinned: float64 brute force on
 *        small nets, numpy matmul + scipy special functions at size, closed
 *        forms for the piecewise-linear activations, softmax invariants.
 *   orc_sample_loss / orc_batch_loss ........ pinned: closed forms (MSE of known
 *        vectors, -log of the target's probability for one-hot targets, the
 *        1e-9 clamps at 0 and 1, binary cross-entropy symmetry).
 *   orc_argmax .............................. pinned: numpy argmax (first maximum).
 *   orc_derivative .......................... pinned: central differences of orc_activate
 *        away from the kinks, the piecewise constants on either side of them.
 *   orc_batch_gradients ..................... pinned: central differences in float64 of the
 *        objective each output-layer rule is the gradient of (half the squared error, or the
 *        cross-entropy through softmax / sigmoid), weight by weight, on small nets; the bias
 *        gradient against the gradient of a weight fed by a constant-one input.
 *   orc_clip_grad_norm ...................... pinned: numpy norm; the norm afterwards equals
 *        max_norm when it was exceeded and is untouched otherwise.
 *   orc_apply_gradients ..................... pinned: first-step closed forms (SGD w - lr g;
 *        Adam and AdamW -lr g / sqrt(g^2 + eps) whatever beta1, beta2; RMSprop
 *        -lr g / sqrt((1 - beta2) g^2 + eps); momentum's geometric sum over repeated steps
 *        with a constant gradient), and decay placement per optimizer.
 *   The last-bit summation order of the reference's BLAS / AVX dot product is
 *   deliberately not reproduced (tolerance 1e-4, not bits).
 */
#ifndef SP_ORACLE_H
#define SP_ORACLE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* enum values follow Include/Spingalett/Spingalett.h:38-47 and :93-101 */
enum { ORC_ACT_SIGMOID = 0, ORC_ACT_RELU, ORC_ACT_TANH, ORC_ACT_LEAKY_RELU,
       ORC_ACT_FOO52, ORC_ACT_SOFTMAX, ORC_ACT_NONE, ORC_ACT_COUNT };
enum { ORC_PREC_F32 = 0, ORC_PREC_F16, ORC_PREC_BF16, ORC_PREC_I8,
       ORC_PREC_I4, ORC_PREC_I2, ORC_PREC_COUNT };

/* How the INT8 / INT4 decode expression is evaluated.
 *   STRICT : ((float)q / d) * max  exactly as written (Serialize.c:233,258).
 *   RELEASE: (float)q * (max * (1.0f/d)) — what the reference's own Release
 *            flag set (-freciprocal-math -fassociative-math,
 *            CMakeLists.txt:143-157) turns that expression into. */
enum { ORC_DEQUANT_STRICT = 0, ORC_DEQUANT_RELEASE = 1 };

typedef struct {
    uint32_t  layers;          /* including the input layer            */
    uint32_t *topology;        /* [layers]                             */
    uint8_t  *act;             /* [layers-1]                           */
    uint8_t   loss;
    uint8_t   has_optimizer;
    uint8_t   precision;       /* of the file the net was parsed from  */
    uint64_t  time_step;
    uint64_t *woff;            /* [layers-1] offsets into weights      */
    uint64_t *boff;            /* [layers-1] offsets into biases       */
    uint64_t  total_weights, total_biases;
    float    *weights;         /* row-major [out][in] per layer        */
    float    *biases;
    int       truncated;       /* payload ended early (Serialize.c:596) */
} orc_net;

/* --- scalar codecs (Serialize.c:12-85) --- */
float    orc_fp16_to_f32(uint16_t h);
uint16_t orc_f32_to_fp16(float x);
float    orc_bf16_to_f32(uint16_t h);
uint16_t orc_f32_to_bf16(float x);

/* --- array codecs (Serialize.c:87-297) --- */
size_t orc_array_bytes(uint32_t n, int precision);
/* returns bytes consumed, 0 when `avail` is too small */
size_t orc_decode_array(const uint8_t *src, size_t avail, uint32_t n,
                        int precision, int mode, float *dst);
/* returns bytes written (dst must hold orc_array_bytes) */
size_t orc_encode_array(const float *src, uint32_t n, int precision, uint8_t *dst);

/* --- file (Serialize.c:307-609) --- */
orc_net *orc_new(uint32_t layers, const uint32_t *topology, const uint8_t *act);
void     orc_free(orc_net *net);
/* err: 0 ok, 1 short header, 2 bad version, 3 layers<2, 4 bad loss,
 *      5 bad precision, 6 bad activation */
orc_net *orc_parse(const uint8_t *buf, size_t len, int mode, int *err);
size_t   orc_serialized_size(const orc_net *net, int precision, int with_optimizer);
size_t   orc_serialize(const orc_net *net, int precision, int with_optimizer,
                       uint8_t *dst);

/* --- activations (Activation.c:5-38, SIMD.c:21-88) --- */
float orc_activate(float x, int act);
void  orc_softmax(float *row, uint32_t n);
void  orc_apply_activation(float *data, uint64_t rows, uint32_t width, int act);

/* --- forward --- */
/* Network.c:202-251, scalar: y = act(b + W x); out holds the last layer. */
void orc_forward_single(const orc_net *net, const float *x, float *out);
/* Training.c:313-345: C = A W^T, C += 1 (x) b, activation; FP32, k-sequential. */
void orc_forward_batch(const orc_net *net, const float *X, uint32_t N, float *out);
/* Same mathematics in float64 end to end (brute-force check, not the reference). */
void orc_forward_batch_f64(const orc_net *net, const float *X, uint32_t N, double *out);

/* --- evaluation after the batched forward --- */
/* compute_sample_loss (SIMD.c:522-552): loss 0 = MSE sum of squared differences,
 * 1 = cross-entropy (-sum t log max(o, 1e-9); with a sigmoid output layer the
 * binary form with o clamped to [1e-9, 1 - 1e-9]). */
float orc_sample_loss(const float *output, const float *target, uint32_t width, int loss, int output_act);
/* batch_compute_loss (Training.c:421-435): the per-sample losses added in sample order, FP32. */
float orc_batch_loss(const float *outputs, const float *targets, uint32_t N, uint32_t width,
                     int loss, int output_act);
/* index of the first largest element of a row (the prediction compared with the label) */
uint32_t orc_argmax(const float *row, uint32_t width);

/* --- batched training step (Training.c:347-419, 439-507; SIMD.c:279-520) --- */
enum { ORC_OPT_SGD = 0, ORC_OPT_MOMENTUM, ORC_OPT_RMSPROP, ORC_OPT_ADAM, ORC_OPT_ADAMW };   /* Spingalett.h:76-83 */
typedef struct {
    int   optimizer;
    float learning_rate, weight_decay, momentum, beta1, beta2, epsilon, max_grad_norm;
    int   decay_in_grad;   /* RMSprop: 1 = the per-sample rule of backpropagation() (Training.c:196-211) */
} orc_opt_args;
/* derivative of an activation as a function of its output (Activation.c:40-56) */
float orc_derivative(float a, int act);
/* forward keeping all layers, output and hidden deltas, gW = grad_scale * delta^T act and
 * gB = grad_scale * column sums of delta; gW / gB laid out like weights / biases; outputs
 * ([N][topology[last]], may be NULL) receives the last layer of the forward. */
void orc_batch_gradients(const orc_net *net, const float *X, const float *T, uint32_t N, float grad_scale,
                         float *gW, float *gB, float *outputs);
/* global L2 norm over gW and gB; both are scaled by max_norm / norm when the norm exceeds it */
float orc_clip_grad_norm(const orc_net *net, float *gW, float *gB, float max_norm);
/* one optimizer step over every array of the net (clipping first when max_grad_norm > 0);
 * beta*_pow_t are beta^t for the step being applied */
void orc_apply_gradients(orc_net *net, const orc_opt_args *args, float *gW, float *gB, float *mW, float *vW,
                         float *mB, float *vB, float beta1_pow_t, float beta2_pow_t);

/* CPU-baseline leg: same call sequence with a threaded sgemm.  sgemm_fn is a
 * cblas_sgemm-compatible pointer found at run time, or NULL for the built-in
 * OpenMP kernel.  Returns seconds per call averaged over `iters`. */
double orc_time_forward_batch(const orc_net *net, const float *X, uint32_t N,
                              float *out, int iters, void *sgemm_fn, int threads);
/* The same for the public single-sample forward (Network.c:218-247): bias copy, then cblas_sgemv (sgemv_fn) or,
 * with NULL, an OpenMP loop over output rows of 4 x 8-lane dot products (SIMD.c:190-240), then the activation. */
double orc_time_forward_single(const orc_net *net, const float *x, float *out, int iters, void *sgemv_fn, int threads);

#ifdef __cplusplus
}
#endif
#endif
