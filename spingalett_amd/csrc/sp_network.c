/*
 * sp_network.c — lifecycle of a NeuralNetwork and the single-sample forward
 * entry.  Behaviour follows Network.c of the reference (layout, error
 * conventions, what layer() initialises); compute is delegated to the device.
 */
#define _GNU_SOURCE
#include "sp_internal.h"

#include <math.h>
#include <pthread.h>
#include <stdatomic.h>
#include <stdlib.h>
#include <string.h>
#include <time.h>

/* ---- weight initialisation (Network.c:150-162, Random.c:66-71) ----
 * Unseeded in the reference (time-based), so only the distributions matter:
 * U(-1,1), or N(0,1) by Box-Muller scaled by sqrt(1/in) / sqrt(2/in). */
static _Thread_local uint64_t t_rng[2];
static _Thread_local bool     t_rng_ready;

static uint64_t mix64(uint64_t *s)
{
    uint64_t z = (*s += 0x9E3779B97F4A7C15ull);
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
    return z ^ (z >> 31);
}

static uint32_t rng_u32(void)
{
    if (!t_rng_ready) {
        uint64_t seed = (uint64_t)time(NULL) ^ ((uint64_t)clock() << 20) ^ (uint64_t)(uintptr_t)&seed;
        t_rng[0] = mix64(&seed);
        t_rng[1] = mix64(&seed) | 1u;
        t_rng_ready = true;
    }
    /* xoroshiro128+ */
    uint64_t a = t_rng[0], b = t_rng[1], r = a + b;
    b ^= a;
    t_rng[0] = ((a << 24) | (a >> 40)) ^ b ^ (b << 16);
    t_rng[1] = (b << 37) | (b >> 27);
    return (uint32_t)(r >> 32);
}

/* Fisher-Yates with the library's generator (spingalett_shuffle_indices, Random.c:73-81) */
void sp_shuffle_indices(uint32_t *indices, uint32_t n)
{
    for (uint32_t i = n; i-- > 1;) {
        const uint32_t j = rng_u32() % (i + 1);
        const uint32_t tmp = indices[i];
        indices[i] = indices[j];
        indices[j] = tmp;
    }
}

static float rng_unit(void) { return (float)(rng_u32() >> 8) * (1.0f / 16777216.0f); }

static float rng_normal(void)
{
    float u1 = rng_unit(), u2 = rng_unit();
    if (u1 < 1e-6f) u1 = 1e-6f;
    return sqrtf(-2.0f * logf(u1)) * cosf(6.2831853f * u2);
}

/* ---- activate (Activation.c:23-38) ---- */
float activate(float x, ActivationFunction act)
{
    switch (act) {
    case ACT_SIGMOID:    return 1.0f / (1.0f + expf(-x));
    case ACT_RELU:       return x > 0.0f ? x : 0.0f;
    case ACT_TANH:       return tanhf(x);
    case ACT_LEAKY_RELU: return x > 0.0f ? x : 0.01f * x;
    case ACT_FOO52:
        if (x > 1.0f) return 1.0f + 0.01f * (x - 1.0f);
        return x < 0.0f ? 0.01f * x : x;
    default:             return x;
    }
}

/* ---- derivative (Activation.c:40-56): slope of an activation as a function of its OUTPUT ---- */
float derivative(float x, ActivationFunction act)
{
    switch (act) {
    case ACT_RELU:       return x > 0.0f ? 1.0f : 0.0f;
    case ACT_LEAKY_RELU: return x > 0.0f ? 1.0f : 0.01f;
    case ACT_SIGMOID:
    case ACT_SOFTMAX:    return x * (1.0f - x);
    case ACT_TANH:       return 1.0f - x * x;
    case ACT_FOO52:      return (x > 1.0f || x < 0.0f) ? 0.01f : 1.0f;
    default:             return 1.0f;
    }
}

/* ---- print_parameters (Network.c:253-281): every bias and weight of the host arrays through the log ---- */
void print_parameters(NeuralNetwork *net)
{
    if (!net) return;
    sp_log(LOG_INFO, "========== DEBUG NETWORK PARAMETERS ==========");
    sp_log(LOG_INFO, "Loss Function: %s", sp_loss_names[net->loss_func]);
    for (uint32_t l = 0; l + 1 < net->layers; ++l) {
        const uint32_t in = net->topology[l], out = net->topology[l + 1];
        sp_log(LOG_INFO, "[Connection: Layer %u (%u neurons) -> Layer %u (%u neurons), activation function: %s]",
               l, in, l + 1, out, sp_act_names[net->act_func[l]]);
        sp_log(LOG_INFO, "  Biases (Thresholds) for Layer %u:", l + 1);
        for (uint32_t k = 0; k < out; ++k)
            sp_log(LOG_INFO, "    Neuron %u bias: %12.6g", k, (double)net->biases[net->bias_offsets[l] + k]);
        sp_log(LOG_INFO, "  Weights: (total: %llu)", (unsigned long long)((uint64_t)in * out));
        for (uint32_t k = 0; k < in; ++k)
            for (uint32_t j = 0; j < out; ++j)
                sp_log(LOG_INFO, "    L%u N%u -> L%u N%u: %12.6g", l, k, l + 1, j,
                       (double)net->weights[net->weight_offsets[l] + (uint64_t)j * in + k]);
    }
    sp_log(LOG_INFO, "================================================");
}

/* ---- table of live nets ---- */
static pthread_mutex_t g_live_mu = PTHREAD_MUTEX_INITIALIZER;
static sp_net **g_live = NULL;
static size_t g_live_n = 0, g_live_cap = 0;
/* Changes whenever the table does.  A thread remembers the last net it looked up together with this count, so the
   single-sample latency path neither takes the lock nor scans the table while no net is created or freed. */
static _Atomic uint64_t g_live_gen = 1;
static _Thread_local const void *tl_owned_ptr = NULL;
static _Thread_local uint64_t tl_owned_gen = 0;

static bool live_add(sp_net *sn)
{
    bool ok = true;
    pthread_mutex_lock(&g_live_mu);
    if (g_live_n == g_live_cap) {
        const size_t cap = g_live_cap ? 2 * g_live_cap : 16;
        sp_net **t = (sp_net **)realloc(g_live, cap * sizeof *t);
        if (t) { g_live = t; g_live_cap = cap; } else ok = false;
    }
    if (ok) g_live[g_live_n++] = sn;
    atomic_fetch_add(&g_live_gen, 1);
    pthread_mutex_unlock(&g_live_mu);
    return ok;
}

static void live_remove(sp_net *sn)
{
    pthread_mutex_lock(&g_live_mu);
    for (size_t i = 0; i < g_live_n; ++i)
        if (g_live[i] == sn) { g_live[i] = g_live[--g_live_n]; break; }
    atomic_fetch_add(&g_live_gen, 1);
    pthread_mutex_unlock(&g_live_mu);
}

sp_net *sp_owned(const NeuralNetwork *net)
{
    sp_net *found = NULL;
    if (!net) return NULL;
    if ((const void *)net == tl_owned_ptr && atomic_load(&g_live_gen) == tl_owned_gen)
        return (sp_net *)(uintptr_t)net;              /* looked up before, and the table has not changed since */
    pthread_mutex_lock(&g_live_mu);
    for (size_t i = 0; i < g_live_n; ++i)
        if ((const void *)g_live[i] == (const void *)net) { found = g_live[i]; break; }
    const uint64_t gen = atomic_load(&g_live_gen);
    pthread_mutex_unlock(&g_live_mu);
    if (!found || found->magic != SP_NET_MAGIC) return NULL;
    tl_owned_ptr = net;
    tl_owned_gen = gen;
    return found;
}

/* ---- new_spingalett (Network.c:34-45) ---- */
NeuralNetwork *new_spingalett_struct_arguments(NeuralNetworkArgs args)
{
    if ((unsigned)args.loss_func >= LOSS_COUNT) {
        sp_set_error(SPINGALETT_ERR_INVALID, "Invalid loss function");
        return NULL;
    }
    sp_log(LOG_INFO, "Creating new network with %s loss function", sp_loss_names[args.loss_func]);
    sp_net *sn = (sp_net *)calloc(1, sizeof *sn);
    if (!sn) {
        sp_set_error(SPINGALETT_ERR_ALLOC, "NeuralNetwork calloc failed");
        return NULL;
    }
    sn->magic = SP_NET_MAGIC;
    sn->pub.loss_func = args.loss_func;
    if (!live_add(sn)) {
        free(sn);
        sp_set_error(SPINGALETT_ERR_ALLOC, "NeuralNetwork calloc failed");
        return NULL;
    }
    return &sn->pub;
}

/* Grows one flat FP32 array to new_count elements, keeping old_count. */
static bool regrow(float **arr, uint64_t old_count, uint64_t new_count)
{
    float *n = (float *)sp_aligned_calloc(new_count, sizeof(float));
    if (!n) return false;
    if (*arr && old_count) memcpy(n, *arr, old_count * sizeof(float));
    sp_aligned_free(*arr);
    *arr = n;
    return true;
}

/* Gradient / optimizer arrays: while nothing has written them (no optimizer block loaded, no
 * train() call) they are all zero, and growing them means a fresh zero block instead of a copy;
 * with `carry` the old contents move over like the weights do. */
static bool regrow_lazy(float **arr, uint64_t old_count, uint64_t new_count, bool carry)
{
    if (carry) return regrow(arr, old_count, new_count);
    float *n = (float *)sp_aligned_calloc(new_count, sizeof(float));
    if (!n) return false;
    sp_aligned_free(*arr);
    *arr = n;
    return true;
}

/* ---- layer (Network.c:47-200) ---- */
void layer_struct_arguments(LayerArgs args)
{
    NeuralNetwork *net = args.net;
    if (!net || args.neurons_amount == 0) {
        sp_set_error(SPINGALETT_ERR_INVALID, "Net is NULL or neurons amount is 0");
        return;
    }
    sp_net *sn = sp_owned(net);           /* NULL for a record the caller made up: no device state, nothing loaded */
    const uint32_t old_layers = net->layers, nl = old_layers + 1;
    if (nl > 1) {
        if ((unsigned)args.act_func >= ACT_COUNT) {
            sp_set_error(SPINGALETT_ERR_INVALID, "Invalid activation function");
            return;
        }
        if ((unsigned)args.weight_initialization >= WEIGHT_INITIALIZATION_COUNT) {
            sp_set_error(SPINGALETT_ERR_INVALID, "Invalid weight initialization");
            return;
        }
        sp_log(LOG_INFO, "Layer #%u: Neurons amount: %u, Activation function: %s, Weight initialization: %s",
               nl - 1, args.neurons_amount, sp_act_names[args.act_func], sp_init_names[args.weight_initialization]);
    } else {
        sp_log(LOG_INFO, "Layer #0: Neurons amount: %u", args.neurons_amount);
    }

    const uint32_t prev = old_layers ? net->topology[old_layers - 1] : 0;
    const uint64_t add_w = nl > 1 ? (uint64_t)prev * args.neurons_amount : 0;
    const uint64_t add_b = nl > 1 ? args.neurons_amount : 0;
    const uint64_t tn = net->total_neurons + args.neurons_amount;
    const uint64_t tw = net->total_weights + add_w, tb = net->total_biases + add_b;

    uint32_t *topo = (uint32_t *)realloc(net->topology, nl * sizeof(uint32_t));
    if (topo) net->topology = topo;
    uint64_t *noff = (uint64_t *)realloc(net->neuron_offsets, (nl + 1) * sizeof(uint64_t));
    if (noff) net->neuron_offsets = noff;
    uint64_t *woff = (uint64_t *)realloc(net->weight_offsets, nl * sizeof(uint64_t));
    if (woff) net->weight_offsets = woff;
    uint64_t *boff = (uint64_t *)realloc(net->bias_offsets, nl * sizeof(uint64_t));
    if (boff) net->bias_offsets = boff;
    bool ok = topo && noff && woff && boff;
    if (ok && nl > 1) {
        ActivationFunction *af = (ActivationFunction *)realloc(net->act_func, (nl - 1) * sizeof(ActivationFunction));
        if (af) net->act_func = af;
        ok = af != NULL;
    }
    ok = ok && regrow(&net->neurons, net->total_neurons, tn);
    if (ok && nl > 1) {
        /* gradients and moments are carried over like the weights (Network.c:130-146) whenever they can hold
           anything: after a file's optimizer block was loaded or train() ran; otherwise they are still zero */
        const bool carry = !sn || sn->opt_loaded;
        ok = regrow(&net->weights, net->total_weights, tw) && regrow(&net->biases, net->total_biases, tb)
          && regrow_lazy(&net->grad_weights, net->total_weights, tw, carry)
          && regrow_lazy(&net->grad_biases, net->total_biases, tb, carry)
          && regrow_lazy(&net->opt_m_weights, net->total_weights, tw, carry)
          && regrow_lazy(&net->opt_m_biases, net->total_biases, tb, carry)
          && regrow_lazy(&net->opt_v_weights, net->total_weights, tw, carry)
          && regrow_lazy(&net->opt_v_biases, net->total_biases, tb, carry);
    }
    if (!ok) {
        sp_set_error(SPINGALETT_ERR_ALLOC, "Layer allocation failed");
        return;
    }

    net->topology[old_layers] = args.neurons_amount;
    if (nl > 1) {
        net->act_func[nl - 2] = args.act_func;
        float scale = 1.0f;
        if (args.weight_initialization == WEIGHT_INITIALIZATION_XAVIER) scale = sqrtf(1.0f / (float)prev);
        else if (args.weight_initialization == WEIGHT_INITIALIZATION_HE) scale = sqrtf(2.0f / (float)prev);
        float *w = net->weights + net->total_weights;
        if (args.weight_initialization == WEIGHT_INITIALIZATION_RANDOM)
            for (uint64_t i = 0; i < add_w; ++i) w[i] = rng_unit() * 2.0f - 1.0f;
        else if (args.weight_initialization != WEIGHT_INITIALIZATION_NONE)
            for (uint64_t i = 0; i < add_w; ++i) w[i] = rng_normal() * scale;
    }
    net->layers = nl;

    /* offsets (Network.c:16-32) */
    uint64_t n = 0, w = 0, b = 0;
    for (uint32_t l = 0; l < nl; ++l) {
        net->neuron_offsets[l] = n;
        n += net->topology[l];
        if (l + 1 < nl) {
            net->weight_offsets[l] = w;
            net->bias_offsets[l] = b;
            w += (uint64_t)net->topology[l] * net->topology[l + 1];
            b += net->topology[l + 1];
        }
    }
    net->neuron_offsets[nl] = n;
    net->total_neurons = n;
    net->total_weights = w;
    net->total_biases = b;

    /* shape changed: whatever the device or a loaded file held is stale */
    if (sn) {
        sp_hip_release(sn);
        sp_drop_packed(sn);
    }
}

/* Builds a complete zero-weight net in one step: what load_spingalett gets in
 * the reference by calling layer() once per layer with
 * WEIGHT_INITIALIZATION_NONE (Serialize.c:547-563), without the repeated
 * re-seating of every array. */
NeuralNetwork *sp_net_build(LossFunction loss, uint32_t layers, const uint32_t *topology, const uint8_t *acts)
{
    sp_net *sn = (sp_net *)calloc(1, sizeof *sn);
    if (!sn) return NULL;
    sn->magic = SP_NET_MAGIC;
    if (!live_add(sn)) {
        free(sn);
        return NULL;
    }
    NeuralNetwork *net = &sn->pub;
    net->loss_func = loss;
    net->layers = layers;
    net->topology = (uint32_t *)malloc(layers * sizeof(uint32_t));
    net->act_func = (ActivationFunction *)malloc((layers - 1) * sizeof(ActivationFunction));
    net->neuron_offsets = (uint64_t *)calloc(layers + 1, sizeof(uint64_t));
    net->weight_offsets = (uint64_t *)calloc(layers, sizeof(uint64_t));
    net->bias_offsets = (uint64_t *)calloc(layers, sizeof(uint64_t));
    if (!net->topology || !net->act_func || !net->neuron_offsets || !net->weight_offsets || !net->bias_offsets) {
        free_network(net);
        return NULL;
    }
    uint64_t n = 0, w = 0, b = 0;
    for (uint32_t l = 0; l < layers; ++l) {
        net->topology[l] = topology[l];
        net->neuron_offsets[l] = n;
        n += topology[l];
        if (l + 1 < layers) {
            net->act_func[l] = (ActivationFunction)acts[l];
            net->weight_offsets[l] = w;
            net->bias_offsets[l] = b;
            w += (uint64_t)topology[l] * topology[l + 1];
            b += topology[l + 1];
        }
    }
    net->neuron_offsets[layers] = n;
    net->total_neurons = n;
    net->total_weights = w;
    net->total_biases = b;
    net->neurons = (float *)sp_aligned_calloc(n, sizeof(float));
    net->weights = (float *)sp_aligned_calloc(w, sizeof(float));
    net->biases = (float *)sp_aligned_calloc(b, sizeof(float));
    net->grad_weights = (float *)sp_aligned_calloc(w, sizeof(float));
    net->grad_biases = (float *)sp_aligned_calloc(b, sizeof(float));
    net->opt_m_weights = (float *)sp_aligned_calloc(w, sizeof(float));
    net->opt_m_biases = (float *)sp_aligned_calloc(b, sizeof(float));
    net->opt_v_weights = (float *)sp_aligned_calloc(w, sizeof(float));
    net->opt_v_biases = (float *)sp_aligned_calloc(b, sizeof(float));
    if (!net->neurons || !net->weights || !net->biases || !net->grad_weights || !net->grad_biases ||
        !net->opt_m_weights || !net->opt_m_biases || !net->opt_v_weights || !net->opt_v_biases) {
        free_network(net);
        return NULL;
    }
    return net;
}

/* ---- forward (Network.c:202-251) ---- */
float *forward_struct_arguments(ForwardArgs args)
{
    (void)sp_resolve_compute_mode();          /* resolved before the NULL check, as Network.c:205 */
    NeuralNetwork *net = args.net;
    if (!net || !args.input) return NULL;
    if (net->layers < 2) {
        sp_set_error(SPINGALETT_ERR_INVALID, "Network must have at least 2 layers for forward pass");
        return NULL;
    }
    sp_net *sn = sp_owned(net);
    if (!sn) {
        sp_set_error(SPINGALETT_ERR_INVALID, "forward: network was not created by this library");
        return NULL;
    }
    return sp_hip_forward_single(sn, args.input);
}

/* ---- free_network (Network.c:283-301) ---- */
void free_network(NeuralNetwork *net)
{
    if (!net) return;
    sp_net *sn = sp_owned(net);
    if (sn) {
        sp_hip_release(sn);
        sp_drop_packed(sn);
        live_remove(sn);
        sn->magic = 0;
    }
    sp_aligned_free(net->neurons);
    sp_aligned_free(net->weights);
    sp_aligned_free(net->biases);
    sp_aligned_free(net->grad_weights);
    sp_aligned_free(net->grad_biases);
    sp_aligned_free(net->opt_m_weights);
    sp_aligned_free(net->opt_m_biases);
    sp_aligned_free(net->opt_v_weights);
    sp_aligned_free(net->opt_v_biases);
    free(net->neuron_offsets);
    free(net->weight_offsets);
    free(net->bias_offsets);
    free(net->topology);
    free(net->act_func);
    free(net);
    sp_log(LOG_DEBUG, "Memory freed.");
}
