/*
 * spingalett.h — public C interface of the MI355X build of the Spingalett
 * inference path.
 *
 * Binary contract: every type and function in the section "reference
 * interface" has the name, value, field order and calling convention of the
 * reference's public header (Include/Spingalett/Spingalett.h), so a program
 * compiled against that header links and runs against this library
 * unchanged.  The section "additive interface" lists what this build adds;
 * nothing in the reference interface is altered to make room for it.
 *
 * train() runs on the device (all three strategies; MODE_GENERATOR_FUNCTION is
 * rejected with an error as in the reference).
 */
#ifndef SPINGALETT_AMD_H
#define SPINGALETT_AMD_H

#include <stdbool.h>
#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define SPINGALETT_API __attribute__((visibility("default")))

/* ===================================================================== *
 *  reference interface                                                   *
 * ===================================================================== */

#define SPINGALETT_FORMAT_VERSION 1             /* Spingalett.h:26 */

/* Spingalett.h:198-200 — codes kept by the thread-local error slot. */
#define SPINGALETT_OK          0
#define SPINGALETT_ERR_ALLOC   1
#define SPINGALETT_ERR_INVALID 2

/* Spingalett.h:28-34 */
typedef enum { LOG_DEBUG, LOG_INFO, LOG_WARNING, LOG_ERROR, LOG_NONE } LogLevel;
typedef void (*LogCallback)(LogLevel level, const char *message);

/* Spingalett.h:38-47 — the byte stored per layer in a .nn file. */
typedef enum {
    ACT_SIGMOID,      /* 1/(1+exp(-x))                                  */
    ACT_RELU,         /* x>0 ? x : 0                                    */
    ACT_TANH,
    ACT_LEAKY_RELU,   /* x>0 ? x : 0.01 x                               */
    ACT_FOO52,        /* x>1 ? 1+0.01(x-1) : (x<0 ? 0.01 x : x)         */
    ACT_SOFTMAX,      /* per sample, over the layer                     */
    ACT_NONE,
    ACT_COUNT
} ActivationFunction;

/* Spingalett.h:49-53 */
typedef enum { LOSS_MSE, LOSS_CROSS_ENTROPY, LOSS_COUNT } LossFunction;

/* Spingalett.h:55-61 */
typedef enum {
    WEIGHT_INITIALIZATION_RANDOM,   /* U(-1,1)              */
    WEIGHT_INITIALIZATION_XAVIER,   /* N(0,1)*sqrt(1/in)    */
    WEIGHT_INITIALIZATION_HE,       /* N(0,1)*sqrt(2/in)    */
    WEIGHT_INITIALIZATION_NONE,     /* zeros                */
    WEIGHT_INITIALIZATION_COUNT
} WeightInitialization;

/* Spingalett.h:63-83 */
typedef enum { MODE_ARRAY, MODE_GENERATOR_FUNCTION, MODE_COUNT } TrainingMode;
typedef enum { STRATEGY_SAMPLE, STRATEGY_FULL_BATCH, STRATEGY_SMALL_BATCH, STRATEGY_COUNT } TrainingStrategy;
typedef enum {
    OPTIMIZER_SGD, OPTIMIZER_MOMENTUM, OPTIMIZER_RMSPROP, OPTIMIZER_ADAM, OPTIMIZER_ADAMW, OPTIMIZER_COUNT
} OptimizerType;

/* Spingalett.h:85-91, with COMPUTE_HIP appended in front of the sentinel.
 * COMPUTE_HIP is the only back-end this library implements; the other
 * values are accepted by spingalett_set_compute_mode() and resolve to
 * COMPUTE_HIP with one warning (the reference resolves an unavailable mode
 * to its single-threaded path the same way, Settings.c:82-110). */
typedef enum {
    COMPUTE_SINGLE_THREADED,
    COMPUTE_OPENMP,
    COMPUTE_OPENBLAS,
    COMPUTE_CUDA,
    COMPUTE_HIP,
    COMPUTE_COUNT
} ComputeMode;

/* Spingalett.h:93-101 — the precision byte of a .nn file. */
typedef enum {
    PRECISION_FLOAT32,
    PRECISION_FP16,
    PRECISION_BFLOAT16,
    PRECISION_INT8,     /* f32 max | i8[n]        w = (q/127)*max         */
    PRECISION_INT4,     /* f32 max | u8[(n+1)/2]  w = (q/7)*max, low nibble first */
    PRECISION_INT2,     /* f32 max | u8[(n+3)/4]  w = q*max, bits 2(i%4)  */
    PRECISION_COUNT
} PrecisionMode;

/* Spingalett.h:103-107 */
typedef enum { AUTOSAVE_OFF, AUTOSAVE_OVERWRITE, AUTOSAVE_NEW_FILES } AutoSaveMode;

/* Spingalett.h:109-136.  Plain data, every field readable and writable by
 * the caller.  weights of layer l start at weight_offsets[l] and are
 * row-major [out][in]; activations of layer l start at neuron_offsets[l]. */
typedef struct {
    uint32_t layers;
    uint32_t *topology;
    ActivationFunction *act_func;

    float *weights;
    float *biases;
    float *neurons;

    float *grad_weights;
    float *grad_biases;

    float *opt_m_weights;
    float *opt_m_biases;
    float *opt_v_weights;
    float *opt_v_biases;

    uint64_t *neuron_offsets;
    uint64_t *weight_offsets;
    uint64_t *bias_offsets;

    uint64_t total_neurons;
    uint64_t total_weights;
    uint64_t total_biases;

    uint64_t time_step;
    LossFunction loss_func;
} NeuralNetwork;

/* Spingalett.h:140-154, 191-196 — by-value argument records. */
typedef struct { LossFunction loss_func; } NeuralNetworkArgs;

typedef struct {
    NeuralNetwork *net;
    uint32_t neurons_amount;
    ActivationFunction act_func;
    WeightInitialization weight_initialization;
} LayerArgs;

typedef struct {
    NeuralNetwork *net;
    const float *input;
} ForwardArgs;

/* Spingalett.h:138, 156-189.  Zero fields take the defaults of train_struct_arguments
 * (Training.c:593-600, 629-632): learning_rate 0.01, momentum 0.9, beta1 0.9, beta2 0.999,
 * epsilon 1e-8, batch_size 32, callback_interval 1. */
typedef bool (*TrainCallback)(NeuralNetwork *net, size_t epoch, float current_error);
typedef struct {
    NeuralNetwork *net;
    TrainingMode training_mode;
    TrainingStrategy training_strategy;
    OptimizerType optimizer_type;

    float *inputs;               /* [sample_count][topology[0]]    */
    float *targets;              /* [sample_count][topology[last]] */
    uint32_t sample_count;
    uint32_t batch_size;
    size_t epochs;

    float learning_rate;
    float weight_decay;
    float momentum;
    float beta1;
    float beta2;
    float epsilon;
    float max_grad_norm;

    bool reset_optimizer;
    size_t nan_check_interval;

    size_t report_interval;

    AutoSaveMode autosave_mode;
    size_t autosave_interval;
    const char *autosave_path;
    bool autosave_do_not_save_optimizer;
    PrecisionMode autosave_precision;

    TrainCallback callback;
    size_t callback_interval;
} TrainArgs;

typedef struct {
    NeuralNetwork *net;
    const char *filename;
    bool do_not_save_optimizer;
    PrecisionMode precision;
} SaveArgs;

/* Spingalett.h:202-204 (Error.c:12-28): sticky, per thread. */
SPINGALETT_API int         spingalett_last_error_code(void);
SPINGALETT_API const char *spingalett_last_error_message(void);
SPINGALETT_API void        spingalett_clear_error(void);

/* Spingalett.h:206-215 (Settings.c:22-57): process-wide atomics. */
SPINGALETT_API ComputeMode spingalett_get_compute_mode(void);
SPINGALETT_API void        spingalett_set_compute_mode(ComputeMode mode);
SPINGALETT_API unsigned    spingalett_get_num_threads(void);
SPINGALETT_API void        spingalett_set_num_threads(unsigned n);
SPINGALETT_API void        spingalett_set_log_callback(LogCallback cb);
SPINGALETT_API void        spingalett_set_log_level(LogLevel level);
SPINGALETT_API void        spingalett_set_verbose(bool enabled);
SPINGALETT_API bool        spingalett_get_verbose(void);

/* Spingalett.h:217-218 (Network.c:34-45) */
SPINGALETT_API NeuralNetwork *new_spingalett_struct_arguments(NeuralNetworkArgs args);
/* Spingalett.h:220-221 (Network.c:47-200): appends a layer, re-seats every
 * flat array, initialises the new matrix.  Invalidates the device copy. */
SPINGALETT_API void layer_struct_arguments(LayerArgs args);
/* Spingalett.h:223 (Activation.c:23-38) */
SPINGALETT_API float activate(float x, ActivationFunction act_func);
/* Spingalett.h:224 (Activation.c:40-56): slope of the activation as a function of its output. */
SPINGALETT_API float derivative(float x, ActivationFunction act_func);
/* Spingalett.h:226-227 (Network.c:202-251): one sample.  Returns a pointer
 * into net->neurons (last layer), valid until the next call on that net;
 * NULL without an error for a NULL net/input, NULL + ERR_INVALID for fewer
 * than two layers or when no GPU can run it. */
SPINGALETT_API float *forward_struct_arguments(ForwardArgs args);
/* Spingalett.h:229-230 (Training.c:584-949).  Every step runs on the device in FP32 (forward keeping all
 * layers, deltas, gradients scaled by 1/batch, optional clipping by the global norm, SGD / momentum /
 * RMSprop / Adam / AdamW update), with the reference's epoch loop around them: shuffle per epoch
 * (mini-batches), loss report, NaN check, autosave, callback.  STRATEGY_SAMPLE (the zero value) applies one
 * update per sample in the given order with the rules of backpropagation() (Training.c:78-213: no
 * clipping, RMSprop folds the decay into the gradient); it costs one small device step per sample, so the
 * two batched strategies are the ones to use for speed.
 * The host arrays (weights, biases, gradients, moments) are current whenever the callback, the NaN
 * check or autosave look at them and when the call returns; time_step advances once per step.
 * A net loaded from a quantized file is trained from its FP32 host arrays (what the reference's
 * loader leaves), and later forwards use the trained FP32 weights.  Errors go to the error slot. */
SPINGALETT_API void train_struct_arguments(TrainArgs args);
/* Spingalett.h:232-233 (Serialize.c:307-424) */
SPINGALETT_API void save_spingalett_struct_arguments(SaveArgs args);
/* Spingalett.h:235 (Serialize.c:426-609).  Same FP32 host arrays as the
 * reference; additionally keeps the packed arrays so the device receives the
 * serialized bytes, not the FP32 expansion. */
SPINGALETT_API NeuralNetwork *load_spingalett(const char *filename);
/* Spingalett.h:237 (Network.c:253-281): loss, activations, every bias and weight of the host arrays as LOG_INFO lines. */
SPINGALETT_API void print_parameters(NeuralNetwork *net);
/* Spingalett.h:238 (Network.c:283-301); also releases device memory. */
SPINGALETT_API void free_network(NeuralNetwork *net);

#ifndef __cplusplus
/* Spingalett.h:217,220,226,232 — designated-initialiser front ends (C only). */
#define new_spingalett(...)  new_spingalett_struct_arguments((NeuralNetworkArgs){__VA_ARGS__})
#define layer(...)           layer_struct_arguments((LayerArgs){__VA_ARGS__})
#define forward(...)         forward_struct_arguments((ForwardArgs){__VA_ARGS__})
#define train(...)           train_struct_arguments((TrainArgs){__VA_ARGS__})
#define save_spingalett(...) save_spingalett_struct_arguments((SaveArgs){__VA_ARGS__})
#endif

/* ===================================================================== *
 *  additive interface                                                    *
 * ===================================================================== */

/* Which evaluation of the INT8/INT4 decode expression the library produces
 * (host arrays of load_spingalett and the device decode):
 *   STRICT  — ((float)q / d) * max as written (Serialize.c:233,258), IEEE.
 *   RELEASE — (float)q * (max * (1.0f/d)): what the reference's Release
 *             flags (-freciprocal-math, CMakeLists.txt:143-157) compile it to.
 * Default STRICT.  Applies to nets loaded afterwards. */
typedef enum { SPINGALETT_DEQUANT_STRICT, SPINGALETT_DEQUANT_RELEASE } SpingalettDequantMode;
SPINGALETT_API void spingalett_set_dequant_mode(SpingalettDequantMode mode);
SPINGALETT_API SpingalettDequantMode spingalett_get_dequant_mode(void);

/* Activation type between the layers of a BF16 net on the matrix-core path (5 samples and more; the reference keeps
 * FP32 activations, Training.c:313-345):
 *   FP16 — FP16 activations (11 significant bits) on the FP16 matrix cores, against an FP16 copy of the weights that
 *          is made when they reach the device (twice the weight memory); the default.
 *   BF16 — BF16 activations (8 bits) on the BF16 matrix cores: a few per cent faster, further from the reference's
 *          outputs.
 * Other weight formats always run FP16 activations (integer and FP16 weights) or FP32 arithmetic (FP32 weights). */
typedef enum { SPINGALETT_BF16_ACTIVATIONS_FP16, SPINGALETT_BF16_ACTIVATIONS_BF16 } SpingalettBf16Activations;
SPINGALETT_API void spingalett_set_bf16_activations(SpingalettBf16Activations mode);
SPINGALETT_API SpingalettBf16Activations spingalett_get_bf16_activations(void);

/* The same choice per net, and one more: SPLIT carries every activation between the layers as two FP16 numbers (the
 * value rounded to FP16, and the rounding error times 2^11: about 22 significant bits together) at twice the
 * matrix-core work per layer, for nets whose decisions hang on differences smaller than FP16's 11 bits — a softmax
 * over a thousand classes agrees with the reference's FP32 argmax on 99.9 % of random samples only this way.  For a
 * net with FP32 weights SPLIT is the fast setting for large batches: weights and activations are
 * both taken as two FP16 numbers and every layer runs as three FP16 matrix-core products into one FP32 sum, about
 * three times the throughput of the FP32 matrix instructions at the same distance from the reference's outputs
 * (activations beyond FP16's 65504 saturate; six more bytes per weight on the device).  DEFAULT follows the
 * process-wide setting above.
 * Returns 0, or 1 with the error slot set (not one of this library's nets, or an unknown mode). */
typedef enum { SPINGALETT_NET_ACTIVATIONS_DEFAULT, SPINGALETT_NET_ACTIVATIONS_BF16, SPINGALETT_NET_ACTIVATIONS_SPLIT } SpingalettNetActivations;
SPINGALETT_API int spingalett_set_net_activations(NeuralNetwork *net, SpingalettNetActivations mode);

/* Batched forward: the public form of the reference's static
 * batch_forward(net, ws, inputs, N) (Training.c:313-345).  inputs is
 * row-major [n][topology[0]], outputs row-major [n][topology[last]], both
 * host memory.  Returns outputs, or NULL with the error slot set. */
SPINGALETT_API float *spingalett_forward_batch(NeuralNetwork *net, const float *inputs,
                                               uint32_t n, float *outputs);
/* Same with device-resident inputs and outputs (no PCIe traffic).  The call
 * returns after enqueueing; spingalett_hip_synchronize() waits.  0 on success. */
SPINGALETT_API int spingalett_forward_batch_device(NeuralNetwork *net, const float *d_inputs,
                                                   uint32_t n, float *d_outputs);
SPINGALETT_API int spingalett_hip_synchronize(void);

/* Evaluation of a labelled batch on the device: the forward, then what the reference's epoch
 * loop does with the outputs — compute_sample_loss per sample (SIMD.c:522-552) with the net's
 * loss_func and output activation, added over the batch (batch_compute_loss, Training.c:421-435)
 * — plus the index of the largest output per sample.  inputs [n][topology[0]] and targets
 * [n][topology[last]] are host memory; total_loss receives the sum of the per-sample losses,
 * predictions (n entries) and correct (samples whose prediction is the index of the target's
 * largest entry) may be NULL.  Only these results cross PCIe, not the [n][out] outputs.
 * Returns 0, or 1 with the error slot set. */
SPINGALETT_API int spingalett_evaluate_batch(NeuralNetwork *net, const float *inputs, const float *targets,
                                             uint32_t n, float *total_loss, uint32_t *predictions,
                                             uint32_t *correct);

/* The device copy is made at the first forward and kept.  Call this after
 * writing net->weights / net->biases by hand: the next forward re-uploads
 * from the FP32 host arrays (the packed arrays of a loaded file are dropped,
 * since they no longer describe the net). */
SPINGALETT_API void spingalett_hip_invalidate(NeuralNetwork *net);

/* Precision of the arrays the device holds for this net (the file's
 * precision for a loaded net, PRECISION_FLOAT32 otherwise). */
SPINGALETT_API PrecisionMode spingalett_hip_precision(const NeuralNetwork *net);

/* Runs the device decoder over one array and copies the FP32 result to the
 * host: which = 0 weights of layer l (topology[l]*topology[l+1] values),
 * 1 biases.  Used to check the device dequantisation bit for bit.
 * 0 on success. */
SPINGALETT_API int spingalett_hip_decode(NeuralNetwork *net, uint32_t l, int which,
                                         float *host_out);

/* Opaque kernel-side handle of a net (see spingalett_hip.h), uploading first
 * if needed; NULL on failure. */
SPINGALETT_API void *spingalett_hip_handle(NeuralNetwork *net);

/* Loader for a file already in memory (same parser as load_spingalett). */
SPINGALETT_API NeuralNetwork *load_spingalett_memory(const void *data, size_t bytes);

#ifdef __cplusplus
}
#endif
#endif /* SPINGALETT_AMD_H */
