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
            sphip_destroy(dev);
            return false;
        }
    }
    sn->dev = dev;
    sn->dev_precision = prec;
    return true;
}

static sp_net *checked(NeuralNetwork *net, const char *who)
{
    if (!net) {
        sp_set_error(SPINGALETT_ERR_INVALID, "net is NULL");
        return NULL;
    }
    sp_net *sn = sp_priv(net);
    if (sn->magic != SP_NET_MAGIC) {
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

float *spingalett_forward_batch(NeuralNetwork *net, const float *inputs, uint32_t n, float *outputs)
{
    (void)sp_resolve_compute_mode();
    if (!net || !inputs || !outputs) return NULL;            /* silent, as forward() */
    sp_net *sn = checked(net, "forward_batch");
    if (!sn) return NULL;
    if (n == 0) return outputs;
    if (!ensure_device(sn)) return NULL;
    if (sphip_forward(sn->dev, inputs, n, outputs, 0)) {
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
    if (sphip_forward(sn->dev, d_inputs, n, d_outputs, SPHIP_X_ON_DEVICE | SPHIP_Y_ON_DEVICE)) {
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
    if (sphip_evaluate(sn->dev, inputs, targets, n, (int)net->loss_func, 0, total_loss, predictions, correct)) {
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
    const sp_net *sn = (const sp_net *)(const void *)net;
    if (!net || sn->magic != SP_NET_MAGIC) return PRECISION_FLOAT32;
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
