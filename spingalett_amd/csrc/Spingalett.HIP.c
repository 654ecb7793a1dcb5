/*
 * Spingalett.HIP.c — glue between the public C API and the kernel translation
 * unit (hip_forward.hip, reached only through spingalett_hip.h).
 *
 * Holds the device state of a net: created at the first forward, fed with the
 * packed arrays of a loaded file (or the FP32 host arrays of a net built by
 * layer()), kept until the net changes shape, is invalidated, or is freed.
 * Every failure of the device layer is reported through the library's
 * thread-local error slot; there is no host compute path to fall back to.
 */
#define _GNU_SOURCE
#include "sp_internal.h"

#include <math.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

static void report(int code, const char *where)
{
    char msg[SP_ERRMSG_MAX];
    snprintf(msg, sizeof msg, "%s: %s", where, sphip_last_error_string());
    sp_set_error(code, msg);
    sp_log(LOG_ERROR, "%s", msg);
}

void sp_hip_release(sp_net *sn)
{
    if (sn->dev) {
        sphip_destroy(sn->dev);
        sn->dev = NULL;
    }
}

/* Copies every array of the net (the file's packed ones, else the FP32 host arrays) into the device net. */
static bool upload_arrays(sp_net *sn, sphip_net *dev)
{
    NeuralNetwork *net = &sn->pub;
    const bool packed = sn->packed_w && sn->packed_b;
    for (uint32_t l = 0; l + 1 < net->layers; ++l) {
        int e;
        if (packed) {
            e = sphip_upload_array(dev, l, 0, sn->packed_w[l].codes, sn->packed_w[l].bytes, sn->packed_w[l].max_val)
             || sphip_upload_array(dev, l, 1, sn->packed_b[l].codes, sn->packed_b[l].bytes, sn->packed_b[l].max_val);
        } else {
            const size_t wb = (size_t)net->topology[l] * net->topology[l + 1] * sizeof(float);
            const size_t bb = (size_t)net->topology[l + 1] * sizeof(float);
            e = sphip_upload_array(dev, l, 0, net->weights + net->weight_offsets[l], wb, 0.0f)
             || sphip_upload_array(dev, l, 1, net->biases + net->bias_offsets[l], bb, 0.0f);
        }
        if (e) {
            report(SPINGALETT_ERR_ALLOC, "HIP back-end: upload");
            return false;
        }
    }
    return true;
}

/* Creates the device net and uploads every array; idempotent. */
static bool ensure_device(sp_net *sn)
{
    if (sn->dev) return true;
    NeuralNetwork *net = &sn->pub;
    if (net->layers < 2) {
        sp_set_error(SPINGALETT_ERR_INVALID, "Network must have at least 2 layers for forward pass");
        return false;
    }
    if (sphip_device_count() <= 0) {
        sp_set_error(SPINGALETT_ERR_INVALID, "HIP back-end: no GPU visible to this process");
        sp_log(LOG_ERROR, "HIP back-end: no GPU visible to this process");
        return false;
    }
    const bool packed = sn->packed_w && sn->packed_b;
    const PrecisionMode prec = packed ? sn->packed_precision : PRECISION_FLOAT32;
    uint8_t *acts = (uint8_t *)malloc(net->layers - 1);
    if (!acts) {
        sp_set_error(SPINGALETT_ERR_ALLOC, "HIP back-end: descriptor allocation failed");
        return false;
    }
    for (uint32_t i = 0; i + 1 < net->layers; ++i) acts[i] = (uint8_t)net->act_func[i];
    const sphip_desc desc = {net->layers, net->topology, acts, (uint8_t)prec};
    sphip_net *dev = NULL;
    const int rc = sphip_create(&desc, &dev);
    free(acts);
    if (rc) {
        report(SPINGALETT_ERR_ALLOC, "HIP back-end: create");
        return false;
    }
    if (!upload_arrays(sn, dev)) {
        sphip_destroy(dev);
        return false;
    }
    sn->dev = dev;
    sn->dev_precision = prec;
    return true;
}

/* what spingalett_set_net_activations, or else spingalett_set_bf16_activations, asks of the batched entry points */
static uint32_t activation_flags(const sp_net *sn)
{
    if (sn->act_mode == SPINGALETT_NET_ACTIVATIONS_SPLIT) return SPHIP_SPLIT_ACTIVATIONS;
    if (sn->act_mode == SPINGALETT_NET_ACTIVATIONS_BF16) return SPHIP_BF16_ACTIVATIONS;
    return spingalett_get_bf16_activations() == SPINGALETT_BF16_ACTIVATIONS_BF16 ? SPHIP_BF16_ACTIVATIONS : 0u;
}

static sp_net *checked(NeuralNetwork *net, const char *who)
{
    if (!net) {
        sp_set_error(SPINGALETT_ERR_INVALID, "net is NULL");
        return NULL;
    }
    sp_net *sn = sp_owned(net);
    if (!sn) {
        char msg[SP_ERRMSG_MAX];
        snprintf(msg, sizeof msg, "%s: network was not created by this library", who);
        sp_set_error(SPINGALETT_ERR_INVALID, msg);
        return NULL;
    }
    return sn;
}

/* forward(), Network.c:202-251: the sample goes in, every layer's activations
 * come back into net->neurons, the result pointer aims at the last layer. */
float *sp_hip_forward_single(sp_net *sn, const float *input)
{
    NeuralNetwork *net = &sn->pub;
    if (!ensure_device(sn)) return NULL;
    float *out = net->neurons + net->neuron_offsets[net->layers - 1];
    if (sphip_forward_layers(sn->dev, input, net->neurons)) {
        report(SPINGALETT_ERR_INVALID, "HIP back-end: forward");
        return NULL;
    }
    return out;
}

int spingalett_set_net_activations(NeuralNetwork *net, SpingalettNetActivations mode)
{
    sp_net *sn = checked(net, "set_net_activations");
    if (!sn) return 1;
    if ((unsigned)mode > SPINGALETT_NET_ACTIVATIONS_SPLIT) {
        sp_set_error(SPINGALETT_ERR_INVALID, "set_net_activations: unknown mode");
        return 1;
    }
    sn->act_mode = (int)mode;
    return 0;
}

float *spingalett_forward_batch(NeuralNetwork *net, const float *inputs, uint32_t n, float *outputs)
{
    (void)sp_resolve_compute_mode();
    if (!net || !inputs || !outputs) return NULL;            /* silent, as forward() */
    sp_net *sn = checked(net, "forward_batch");
    if (!sn) return NULL;
    if (n == 0) return outputs;
    if (!ensure_device(sn)) return NULL;
    if (sphip_forward(sn->dev, inputs, n, outputs, activation_flags(sn))) {
        report(SPINGALETT_ERR_INVALID, "HIP back-end: forward_batch");
        return NULL;
    }
    return outputs;
}

int spingalett_forward_batch_device(NeuralNetwork *net, const float *d_inputs, uint32_t n, float *d_outputs)
{
    sp_net *sn = checked(net, "forward_batch_device");
    if (!sn) return 1;
    if (!d_inputs || !d_outputs || n == 0) {
        sp_set_error(SPINGALETT_ERR_INVALID, "forward_batch_device: null pointer or empty batch");
        return 1;
    }
    if (!ensure_device(sn)) return 1;
    if (sphip_forward(sn->dev, d_inputs, n, d_outputs, SPHIP_X_ON_DEVICE | SPHIP_Y_ON_DEVICE | activation_flags(sn))) {
        report(SPINGALETT_ERR_INVALID, "HIP back-end: forward_batch_device");
        return 1;
    }
    return 0;
}

int spingalett_evaluate_batch(NeuralNetwork *net, const float *inputs, const float *targets, uint32_t n,
                              float *total_loss, uint32_t *predictions, uint32_t *correct)
{
    (void)sp_resolve_compute_mode();
    sp_net *sn = checked(net, "evaluate_batch");
    if (!sn) return 1;
    if (!inputs || !targets || n == 0) {
        sp_set_error(SPINGALETT_ERR_INVALID, "evaluate_batch: null pointer or empty batch");
        return 1;
    }
    if (net->loss_func >= LOSS_COUNT) {
        sp_set_error(SPINGALETT_ERR_INVALID, "evaluate_batch: unknown loss function");
        return 1;
    }
    if (!ensure_device(sn)) return 1;
    if (sphip_evaluate(sn->dev, inputs, targets, n, (int)net->loss_func, activation_flags(sn), total_loss, predictions, correct)) {
        report(SPINGALETT_ERR_INVALID, "HIP back-end: evaluate_batch");
        return 1;
    }
    return 0;
}

int spingalett_hip_synchronize(void)
{
    if (sphip_synchronize()) {
        report(SPINGALETT_ERR_INVALID, "HIP back-end: synchronize");
        return 1;
    }
    return 0;
}

void spingalett_hip_invalidate(NeuralNetwork *net)
{
    sp_net *sn = checked(net, "hip_invalidate");
    if (!sn) return;
    sp_hip_release(sn);
    sp_drop_packed(sn);
}

PrecisionMode spingalett_hip_precision(const NeuralNetwork *net)
{
    const sp_net *sn = sp_owned(net);
    if (!sn) return PRECISION_FLOAT32;
    if (sn->dev) return sn->dev_precision;
    return (sn->packed_w && sn->packed_b) ? sn->packed_precision : PRECISION_FLOAT32;
}

int spingalett_hip_decode(NeuralNetwork *net, uint32_t l, int which, float *host_out)
{
    sp_net *sn = checked(net, "hip_decode");
    if (!sn) return 1;
    if (!host_out || l + 1 >= net->layers || (which != 0 && which != 1)) {
        sp_set_error(SPINGALETT_ERR_INVALID, "hip_decode: invalid argument");
        return 1;
    }
    if (!ensure_device(sn)) return 1;
    if (sphip_decode(sn->dev, l, which, (int)spingalett_get_dequant_mode(), host_out)) {
        report(SPINGALETT_ERR_INVALID, "HIP back-end: decode");
        return 1;
    }
    return 0;
}

void *spingalett_hip_handle(NeuralNetwork *net)
{
    sp_net *sn = checked(net, "hip_handle");
    if (!sn || !ensure_device(sn)) return NULL;
    return sn->dev;
}

/* ------------------------------------------------------------------------- *
 *  train(), Training.c:584-949, for the two batched strategies: the epoch
 *  loop, reporting, NaN check, autosave and callback run here; each step
 *  (forward, deltas, gradients, update) runs on the device.
 * ------------------------------------------------------------------------- */
static const char *const optimizer_names[] = {"SGD", "MOMENTUM", "RMSPROP", "ADAM", "ADAMW"};
static const char *const strategy_names[] = {"SGD", "FULL_BATCH", "SMALL_BATCH"};          /* Names.c */

static inline bool should_report(size_t epoch, size_t epochs, size_t interval)      /* Training.c:580-582 */
{
    return interval > 0 && ((epoch % interval == 0) || (epoch == epochs));
}

/* weights, biases, moments and the last gradients back into the host arrays (what the reference's
 * loop leaves in NeuralNetwork after a step) */
static bool train_download(sp_net *sn)
{
    NeuralNetwork *net = &sn->pub;
    sn->opt_loaded = true;            /* the host gradient / moment arrays hold content from here on: layer() carries them */
    for (uint32_t l = 0; l + 1 < net->layers; ++l) {
        const uint64_t wo = net->weight_offsets[l], bo = net->bias_offsets[l];
        if (sphip_train_get(sn->dev, SPHIP_TRAIN_W, l, net->weights + wo) || sphip_train_get(sn->dev, SPHIP_TRAIN_B, l, net->biases + bo) ||
            sphip_train_get(sn->dev, SPHIP_TRAIN_MW, l, net->opt_m_weights + wo) || sphip_train_get(sn->dev, SPHIP_TRAIN_VW, l, net->opt_v_weights + wo) ||
            sphip_train_get(sn->dev, SPHIP_TRAIN_MB, l, net->opt_m_biases + bo) || sphip_train_get(sn->dev, SPHIP_TRAIN_VB, l, net->opt_v_biases + bo) ||
            sphip_train_get(sn->dev, SPHIP_TRAIN_GW, l, net->grad_weights + wo) || sphip_train_get(sn->dev, SPHIP_TRAIN_GB, l, net->grad_biases + bo)) {
            report(SPINGALETT_ERR_INVALID, "HIP back-end: train (download)");
            return false;
        }
    }
    return true;
}

static bool has_nan_inf(const NeuralNetwork *net)                                    /* Training.c:11-19 */
{
    for (uint64_t i = 0; i < net->total_weights; ++i) if (!isfinite(net->weights[i])) return true;
    for (uint64_t i = 0; i < net->total_biases; ++i) if (!isfinite(net->biases[i])) return true;
    return false;
}

static void autosave(NeuralNetwork *net, const TrainArgs *args, size_t epoch)        /* Training.c:536-578 */
{
    SaveArgs sa = {.net = net, .do_not_save_optimizer = args->autosave_do_not_save_optimizer, .precision = args->autosave_precision};
    if (args->autosave_mode == AUTOSAVE_OVERWRITE) {
        sa.filename = args->autosave_path;
        save_spingalett_struct_arguments(sa);
        return;
    }
    if (args->autosave_mode != AUTOSAVE_NEW_FILES) return;
    const char *path = args->autosave_path;
    const char *dot = strrchr(path, '.'), *slash = strrchr(path, '/'), *back = strrchr(path, '\\');
    const char *sep = (slash && back) ? (slash > back ? slash : back) : (slash ? slash : back);
    const bool has_ext = dot && (!sep || dot > sep);
    const size_t cap = strlen(path) + 64;
    char *buf = (char *)malloc(cap);
    if (!buf) return;
    if (has_ext) snprintf(buf, cap, "%.*s_epoch_%zu%s", (int)(dot - path), path, epoch, dot);
    else snprintf(buf, cap, "%s_epoch_%zu", path, epoch);
    sa.filename = buf;
    save_spingalett_struct_arguments(sa);
    free(buf);
}

void train_struct_arguments(TrainArgs args)
{
    NeuralNetwork *net = args.net;
    const uint32_t sample_count = args.sample_count;
    const size_t epochs = args.epochs;

    /* defaults and checks in the reference's order (Training.c:593-636) */
    if (args.learning_rate <= 0.0f) args.learning_rate = 0.01f;
    if (args.momentum <= 0.0f) args.momentum = 0.9f;
    if (args.beta1 <= 0.0f) args.beta1 = 0.9f;
    if (args.beta2 <= 0.0f) args.beta2 = 0.999f;
    if (args.epsilon <= 0.0f) args.epsilon = 1e-8f;
    if (args.callback && args.callback_interval == 0) args.callback_interval = 1;

    if (args.training_mode == MODE_GENERATOR_FUNCTION) {
        sp_set_error(SPINGALETT_ERR_INVALID, "Generator function training mode is not implemented yet");
        sp_log(LOG_ERROR, "Generator function training mode is not implemented yet");
        return;
    }
    if (!net || sample_count == 0 || epochs == 0 || !args.inputs || !args.targets) {
        sp_set_error(SPINGALETT_ERR_INVALID, "Invalid training arguments (NULL net/inputs/targets or zero count/epochs)");
        sp_log(LOG_ERROR, "Invalid training arguments");
        return;
    }
    sp_net *sn = checked(net, "train");
    if (!sn) return;
    if (net->layers < 2) {
        sp_set_error(SPINGALETT_ERR_INVALID, "Network must have at least 2 layers for training");
        sp_log(LOG_ERROR, "Network must have at least 2 layers for training");
        return;
    }
    for (uint32_t l = 1; l + 1 < net->layers; ++l) {
        if (net->act_func[l - 1] == ACT_SOFTMAX) {
            sp_set_error(SPINGALETT_ERR_INVALID, "Softmax is not supported in hidden layers");
            sp_log(LOG_ERROR, "Softmax in hidden layer %u is not supported. Use softmax only in the output layer.", l);
            return;
        }
    }
    if ((unsigned)args.optimizer_type >= OPTIMIZER_COUNT || (unsigned)args.training_strategy >= STRATEGY_COUNT ||
        net->loss_func >= LOSS_COUNT) {
        sp_set_error(SPINGALETT_ERR_INVALID, "Invalid training arguments (unknown optimizer, strategy or loss)");
        sp_log(LOG_ERROR, "Invalid training arguments");
        return;
    }
    const bool per_sample = args.training_strategy == STRATEGY_SAMPLE;
    const bool small = args.training_strategy == STRATEGY_SMALL_BATCH;
    if (small && args.batch_size == 0) args.batch_size = 32;
    if (small && args.batch_size > sample_count) args.batch_size = sample_count;

    if (args.reset_optimizer) {                                                      /* Training.c:636-643 */
        memset(net->opt_m_weights, 0, net->total_weights * sizeof(float));
        memset(net->opt_v_weights, 0, net->total_weights * sizeof(float));
        memset(net->opt_m_biases, 0, net->total_biases * sizeof(float));
        memset(net->opt_v_biases, 0, net->total_biases * sizeof(float));
        net->time_step = 0;
        sp_log(LOG_INFO, "Optimizer state reset");
    }
    (void)sp_resolve_compute_mode();

    /* training works on the FP32 host arrays: a device copy holding a file's packed arrays is replaced */
    if (sn->dev && sn->dev_precision != PRECISION_FLOAT32) sp_hip_release(sn);
    sp_drop_packed(sn);
    /* The host arrays may have been written since the last upload: an existing FP32 device net gets them again
     * (its buffers, and the training buffers an earlier call left, are kept: allocating and freeing them costs more
     * than the uploads). */
    if (sn->dev && !upload_arrays(sn, sn->dev)) {
        sp_hip_release(sn);
        return;
    }
    if (!ensure_device(sn)) return;
    if (sphip_train_begin(sn->dev)) {
        report(SPINGALETT_ERR_ALLOC, "HIP back-end: train");
        return;
    }
    for (uint32_t l = 0; l + 1 < net->layers; ++l) {
        const uint64_t wo = net->weight_offsets[l], bo = net->bias_offsets[l];
        if (sphip_train_set(sn->dev, SPHIP_TRAIN_MW, l, net->opt_m_weights + wo) || sphip_train_set(sn->dev, SPHIP_TRAIN_VW, l, net->opt_v_weights + wo) ||
            sphip_train_set(sn->dev, SPHIP_TRAIN_MB, l, net->opt_m_biases + bo) || sphip_train_set(sn->dev, SPHIP_TRAIN_VB, l, net->opt_v_biases + bo)) {
            report(SPINGALETT_ERR_INVALID, "HIP back-end: train (upload)");
            sphip_train_end(sn->dev);
            return;
        }
    }

    if (per_sample)
        sp_log(LOG_WARNING, "HIP back-end: the per-sample strategy runs one small device step per sample; the batched strategies are the fast ones");
    if (small)
        sp_log(LOG_INFO, "Starting training: loss=%s, strategy=%s, mode=ARRAY, optimizer=%s, compute=HIP, batch_size=%u",
               sp_loss_names[net->loss_func], strategy_names[args.training_strategy], optimizer_names[args.optimizer_type], args.batch_size);
    else
        sp_log(LOG_INFO, "Starting training: loss=%s, strategy=%s, mode=ARRAY, optimizer=%s, compute=HIP",
               sp_loss_names[net->loss_func], strategy_names[args.training_strategy], optimizer_names[args.optimizer_type]);

    const uint32_t in_sz = net->topology[0], out_sz = net->topology[net->layers - 1];
    const uint32_t eff_batch = small ? args.batch_size : per_sample ? 1u : sample_count;
    uint32_t *order = NULL;
    float *bx = NULL, *bt = NULL;
    if (small) {
        order = (uint32_t *)malloc((size_t)sample_count * sizeof(uint32_t));
        bx = (float *)sp_aligned_calloc((size_t)eff_batch * in_sz, sizeof(float));
        bt = (float *)sp_aligned_calloc((size_t)eff_batch * out_sz, sizeof(float));
        if (!order || !bx || !bt) {
            sp_set_error(SPINGALETT_ERR_ALLOC, "Mini-batch allocation failed");
            sp_log(LOG_ERROR, "Mini-batch allocation failed");
            free(order); sp_aligned_free(bx); sp_aligned_free(bt);
            sphip_train_end(sn->dev);
            return;
        }
        for (uint32_t i = 0; i < sample_count; ++i) order[i] = i;
    }

    sphip_train_args ta = {
        .optimizer = (int32_t)args.optimizer_type, .loss_func = (int32_t)net->loss_func,
        .learning_rate = args.learning_rate, .weight_decay = args.weight_decay, .momentum = args.momentum,
        .beta1 = args.beta1, .beta2 = args.beta2, .epsilon = args.epsilon, .max_grad_norm = args.max_grad_norm,
        .beta1_pow_t = 1.0f, .beta2_pow_t = 1.0f,                                   /* Training.c:684-685 */
    };
    if (per_sample) {
        /* backpropagation() (Training.c:78-213): one update per sample in the given order, no clipping,
         * RMSprop folds the decay into the gradient */
        ta.max_grad_norm = 0.0f;
        ta.decay_in_grad = 1;
    }
    bool failed = false;
    for (size_t epoch = 1; epoch <= epochs && !failed; ++epoch) {
        const bool need_loss = should_report(epoch, epochs, args.report_interval) ||
                               (args.callback && should_report(epoch, epochs, args.callback_interval));
        float total_error = 0.0f;
        if (per_sample) {
            for (uint32_t s = 0; s < sample_count && !failed; ++s) {
                float loss = 0.0f;
                net->time_step++;
                ta.beta1_pow_t *= args.beta1;
                ta.beta2_pow_t *= args.beta2;
                failed = sphip_train_step(sn->dev, args.inputs + (size_t)s * in_sz, args.targets + (size_t)s * out_sz, 1, &ta, 0,
                                          need_loss ? &loss : NULL) != 0;
                total_error += loss;
            }
        } else if (!small) {
            float loss = 0.0f;
            net->time_step++;
            ta.beta1_pow_t *= args.beta1;
            ta.beta2_pow_t *= args.beta2;
            /* the batch is the same every epoch: it crosses PCIe once */
            failed = sphip_train_step(sn->dev, args.inputs, args.targets, sample_count, &ta,
                                      epoch == 1 ? 0u : SPHIP_TRAIN_SAME_BATCH, need_loss ? &loss : NULL) != 0;
            total_error = loss;
        } else {
            sp_shuffle_indices(order, sample_count);
            for (uint32_t start = 0; start < sample_count && !failed; start += eff_batch) {
                const uint32_t cur = sample_count - start < eff_batch ? sample_count - start : eff_batch;
                for (uint32_t s = 0; s < cur; ++s) {                                 /* gather, Training.c:760-767 */
                    const uint32_t idx = order[start + s];
                    memcpy(bx + (size_t)s * in_sz, args.inputs + (size_t)idx * in_sz, (size_t)in_sz * sizeof(float));
                    memcpy(bt + (size_t)s * out_sz, args.targets + (size_t)idx * out_sz, (size_t)out_sz * sizeof(float));
                }
                float loss = 0.0f;
                net->time_step++;
                ta.beta1_pow_t *= args.beta1;
                ta.beta2_pow_t *= args.beta2;
                failed = sphip_train_step(sn->dev, bx, bt, cur, &ta, 0, need_loss ? &loss : NULL) != 0;
                total_error += loss;
            }
        }
        if (failed) {
            report(SPINGALETT_ERR_INVALID, "HIP back-end: train (step)");
            break;
        }
        const float current_error = total_error / (float)sample_count;
        if (should_report(epoch, epochs, args.report_interval))
            sp_log(LOG_INFO, "Epoch: %zu/%zu, Error: %f", epoch, epochs, (double)current_error);

        /* whoever looks at the host arrays below needs them current */
        const bool nan_now = args.nan_check_interval > 0 && epoch % args.nan_check_interval == 0;
        const bool save_now = args.autosave_mode != AUTOSAVE_OFF && args.autosave_interval > 0 && args.autosave_path &&
                              should_report(epoch, epochs, args.autosave_interval);
        const bool call_now = args.callback && should_report(epoch, epochs, args.callback_interval);
        if ((nan_now || save_now || call_now) && !train_download(sn)) break;
        if (nan_now && has_nan_inf(net)) {
            sp_log(LOG_ERROR, "NaN/Inf detected in weights at epoch %zu, stopping training", epoch);
            break;
        }
        if (save_now) autosave(net, &args, epoch);
        if (call_now && args.callback(net, epoch, current_error)) {
            sp_log(LOG_INFO, "Training interrupted by callback at epoch %zu", epoch);
            break;
        }
    }
    (void)train_download(sn);
    /* no sphip_train_end: the training buffers stay with the device net for the next call and go with it
     * (free_network, layer(), spingalett_hip_invalidate) */
    free(order);
    sp_aligned_free(bx);
    sp_aligned_free(bt);
    sp_log(LOG_INFO, "Training completed.");
}
