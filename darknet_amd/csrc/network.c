/*
 * network.c - the inference runtime: forward_network / network_predict and the small helpers
 * around them.  Restates the GPU branch of the reference's src/network.c for net.train == 0.
 */
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include "host.h"
#include "hip.h"

/* written as a declaration so that it can stand before the function's own declarations */
#define DN_NEED_DEVICE(what) const int need_device_ = (hip_require_device(what), 0); (void)need_device_

/* src/network.c:177-186 */
network *make_network(int n)
{
    network *net = (network *)dn_calloc(1, sizeof(network));
    net->n = n;
    net->layers = (layer *)dn_calloc((size_t)n, sizeof(layer));
    net->seen = (size_t *)dn_calloc(1, sizeof(size_t));
    return net;
}

/* src/network.c:699-716 */
void free_network(network *net)
{
    int i;
    if (!net) return;
    for (i = 0; i < net->n; ++i) {
        layer l = net->layers[i];
        free_layer(l); /* leaves the buffers a layer only borrows: dropout, one-source routes */
    }
    free(net->layers);
    free(net->input);
    free(net->seen);
    if (net->input_gpu) hip_free(net->input_gpu);
    if (net->det_rows_gpu) hip_free(net->det_rows_gpu);
    if (net->det_count_gpu) hip_free((float *)net->det_count_gpu);
    dn_pipeline_free(net);
    free(net);
}

/* src/network.c:689-697 */
layer get_network_output_layer(network *net)
{
    int i;
    for (i = net->n - 1; i >= 0; --i)
        if (net->layers[i].type != COST) break;
    if (i < 0) dn_fatal("network has no layers");
    return net->layers[i];
}

float *network_output(network *net) { return get_network_output_layer(net).output; }
int network_width(network *net) { return net->w; }
int network_height(network *net) { return net->h; }

/* src/network.c:339-356.  Buffers were sized at parse time, so the batch can only shrink. */
void set_batch_network(network *net, int b)
{
    int i;
    if (b < 1) dn_fatal("set_batch_network: batch must be at least 1");
    if (network_predict_in_flight(net))
        dn_fatal("set_batch_network: batches submitted with network_predict_submit are in flight; collect them first");
    if (net->max_batch < net->batch) net->max_batch = net->batch; /* a network built without the parser */
    if (b > net->max_batch)
        dn_fatal("set_batch_network: buffers were allocated for a smaller batch (the cfg's batch is the limit)");
    net->batch = b;
    for (i = 0; i < net->n; ++i) net->layers[i].batch = b;
}

static int g_fuse_shortcut = 1; /* 0 off, 1 on, 2 on and lean */

/* 0: every layer runs on its own, as in src/network.c:773-785.
 * 1 (default): layer pairs run as one launch where a kernel serves both - a convolution and the
 *    same-geometry shortcut or the yolo head behind it, an xnor convolution and the 2x2 stride-2
 *    maxpool behind it - and an xnor convolution writes the sign bits the next xnor convolution
 *    reads.  Every layer's output buffer is written and holds the bits of the unfused sequence.
 * 2 (lean): as 1, but the map of an xnor convolution that only the maxpool fused behind it reads
 *    is not written (its output buffer keeps whatever it held; layer_output_host refuses it). */
void network_set_fusion(int on) { g_fuse_shortcut = on < 0 ? 0 : on > 2 ? 2 : on; }

/* An xnor convolution and the maxpool behind it that the pooled kernel serves: 3x3 / stride 1 /
 * pad 1 into an even-sized map, pooled 2x2 with stride 2 from the map's first pixel. */
static int xnor_pool_pair(const network *net, int i)
{
    const layer *l, *m;
    if (!g_fuse_shortcut || i < 0 || i + 1 >= net->n) return 0;
    l = &net->layers[i];
    m = &net->layers[i + 1];
    if (l->type != CONVOLUTIONAL || !l->xnor || m->type != MAXPOOL) return 0;
    if (l->size != 3 || l->stride != 1 || l->pad != 1 || (l->out_h & 1) || (l->out_w & 1)) return 0;
    if (m->size != 2 || m->stride != 2 || m->pad / 2 != 0) return 0;
    if (m->h != l->out_h || m->w != l->out_w || m->c != l->out_c || m->batch != l->batch) return 0;
    if (m->out_h * 2 != m->h || m->out_w * 2 != m->w) return 0;
    return 1;
}

/* A first layer (3 channels, 3x3 / stride 1 / pad 1) and the 2x2 stride-2 maxpool behind it that
 * forward_convolutional_maxpool_gpu serves in one pass. */
static int conv_pool_pair(const network *net, int i)
{
    const layer *l, *m;
    if (!g_fuse_shortcut || i < 0 || i + 1 >= net->n) return 0;
    l = &net->layers[i];
    m = &net->layers[i + 1];
    if (l->type != CONVOLUTIONAL || l->xnor || m->type != MAXPOOL) return 0;
    if (m->size != 2 || m->stride != 2 || m->pad / 2 != 0) return 0;
    if (m->h != l->out_h || m->w != l->out_w || m->c != l->out_c || m->batch != l->batch) return 0;
    if (m->out_h * 2 != m->h || m->out_w * 2 != m->w) return 0;
    return conv_maxpool_fusable(l->batch, l->c, l->h, l->w, l->n, l->groups, l->size, l->stride, l->pad,
                                (int)l->activation);
}

/* The xnor convolution that reads layer q's output as its input and can take its sign bits from
 * the kernel that wrote that output: the layer right behind it.  -1: none. */
static int xnor_bits_consumer(const network *net, int q)
{
    const layer *p, *k;
    if (!g_fuse_shortcut || q < 0 || q + 1 >= net->n) return -1;
    p = &net->layers[q];
    k = &net->layers[q + 1];
    if (k->type != CONVOLUTIONAL || !k->xnor || !k->xnor_xbits_gpu) return -1;
    if (k->c != p->out_c || k->h != p->out_h || k->w != p->out_w || k->batch != p->batch) return -1;
    return q + 1;
}

/* Whether xnor convolution i finds its input's sign bits already written by the layer in front. */
static int xnor_bits_ready(const network *net, int i)
{
    if (i >= 1 && net->layers[i - 1].type == CONVOLUTIONAL && net->layers[i - 1].xnor)
        return xnor_bits_consumer(net, i - 1) == i;
    if (i >= 2 && net->layers[i - 1].type == MAXPOOL && (xnor_pool_pair(net, i - 2) || conv_pool_pair(net, i - 2)))
        return xnor_bits_consumer(net, i - 1) == i;
    return 0;
}

/* Whether anything but the layer right behind it reads layer i's output. */
static int layer_output_read_elsewhere(const network *net, int i)
{
    int k, j;
    if (i >= net->n - 1) return 1;
    for (k = i + 1; k < net->n; ++k) {
        const layer *l = &net->layers[k];
        if (l->type == ROUTE)
            for (j = 0; j < l->n; ++j)
                if (l->input_layers[j] == i) return 1;
        if (l->type == SHORTCUT && l->index == i) return 1;
    }
    return 0;
}

/* lean mode: the map of convolution i, which only the maxpool fused behind it reads, is not written */
static int xnor_map_skipped(const network *net, int i)
{
    return g_fuse_shortcut == 2 && (xnor_pool_pair(net, i) || conv_pool_pair(net, i)) &&
           !layer_output_read_elsewhere(net, i);
}

/* Runs convolution i and the maxpool behind it as one pass when conv_pool_pair says so.  Returns 1 if it did. */
static int forward_conv_pool_pair(network net, int i)
{
    layer l, m;
    int k;
    if (!conv_pool_pair(&net, i)) return 0;
    l = net.layers[i];
    m = net.layers[i + 1];
    k = xnor_bits_consumer(&net, i + 1);
    forward_convolutional_maxpool_gpu(net.input_gpu, l.weights_gpu, l.biases_gpu, l.scales_gpu, l.rolling_mean_gpu,
                                      l.rolling_variance_gpu, xnor_map_skipped(&net, i) ? 0 : l.output_gpu,
                                      m.output_gpu, k >= 0 ? net.layers[k].xnor_xbits_gpu : 0, l.batch, l.c, l.h, l.w,
                                      l.n, l.groups, l.size, l.stride, l.pad, l.batch_normalize, (int)l.activation);
    return 1;
}

/* Runs xnor convolution i, with the maxpool behind it when xnor_pool_pair says so.  Returns the
 * number of layers it ran beyond i (0 or 1). */
static int forward_xnor(network net, int i)
{
    const layer l = net.layers[i];
    const int pooled = xnor_pool_pair(&net, i);
    const int q = i + pooled;
    const int k = xnor_bits_consumer(&net, q);
    forward_convolutional_xnor_fused_gpu(net.input_gpu, l.xnor_wbits_gpu, l.xnor_wmean_gpu, l.xnor_xbits_gpu,
                                         xnor_bits_ready(&net, i), l.biases_gpu, l.scales_gpu, l.rolling_mean_gpu,
                                         l.rolling_variance_gpu, xnor_map_skipped(&net, i) ? 0 : l.output_gpu,
                                         pooled ? net.layers[i + 1].output_gpu : 0,
                                         k >= 0 ? net.layers[k].xnor_xbits_gpu : 0, l.batch, l.c, l.h, l.w, l.n, l.size,
                                         l.stride, l.pad, l.batch_normalize, (int)l.activation);
    return pooled;
}

/* Runs layers i and i+1 together when they are a convolution and the residual add of a
 * darknet53 block (src/shortcut_layer.c:77-83 with equal geometries).  Returns 1 if it did. */
static int conv_shortcut_pair(const network *net, int i)
{
    const layer *l, *s;
    if (!g_fuse_shortcut || i < 0 || i + 1 >= net->n) return 0;
    l = &net->layers[i];
    s = &net->layers[i + 1];
    if (l->type != CONVOLUTIONAL || l->xnor || s->type != SHORTCUT) return 0;
    if (s->index < 0 || s->index >= i) return 0; /* the residual must come from an earlier layer */
    if (s->w != s->out_w || s->h != s->out_h || s->c != s->out_c) return 0;
    if (s->out_w != l->out_w || s->out_h != l->out_h || s->out_c != l->out_c || s->batch != l->batch) return 0;
    return 1;
}

static int forward_conv_shortcut_pair(network net, int i)
{
    layer l, s;
    if (!conv_shortcut_pair(&net, i)) return 0;
    l = net.layers[i];
    s = net.layers[i + 1];
    forward_convolutional_shortcut_gpu(net.input_gpu, l.weights_gpu, l.weights_packed_gpu, l.biases_gpu,
                                       l.scales_gpu, l.rolling_mean_gpu, l.rolling_variance_gpu, l.output_gpu,
                                       l.batch, l.c, l.h, l.w, l.n, l.groups, l.size, l.stride, l.pad,
                                       l.batch_normalize, (int)l.activation, net.layers[s.index].output_gpu,
                                       s.output_gpu, s.alpha, s.beta, (int)s.activation);
    return 1;
}

/* Runs layers i and i+1 together when they are a convolution and the yolo head it feeds
 * (src/yolo_layer.c:347-361): the head's copy + logistic rides in the convolution's epilogue.
 * Returns 1 if it did. */
static int conv_yolo_pair(const network *net, int i)
{
    const layer *l, *y;
    if (!g_fuse_shortcut || i < 0 || i + 1 >= net->n) return 0;
    l = &net->layers[i];
    y = &net->layers[i + 1];
    if (l->type != CONVOLUTIONAL || l->xnor || y->type != YOLO) return 0;
    if (y->w != l->out_w || y->h != l->out_h || y->batch != l->batch || y->n * (5 + y->classes) != l->n) return 0;
    return 1;
}

static int forward_conv_yolo_pair(network net, int i)
{
    layer l, y;
    if (!conv_yolo_pair(&net, i)) return 0;
    l = net.layers[i];
    y = net.layers[i + 1];
    forward_convolutional_yolo_gpu(net.input_gpu, l.weights_gpu, l.weights_packed_gpu, l.biases_gpu, l.scales_gpu,
                                   l.rolling_mean_gpu, l.rolling_variance_gpu, l.output_gpu, l.batch, l.c, l.h,
                                   l.w, l.n, l.groups, l.size, l.stride, l.pad, l.batch_normalize,
                                   (int)l.activation, y.output_gpu, y.n, y.classes);
    return 1;
}

/* Whether layer i runs inside the kernel of the convolution in front of it at the present fusion
 * level (a residual add, a yolo head, a 2x2 stride-2 maxpool), so that no launch is its own; and
 * whether, in lean mode, layer i's own output is left unwritten. */
int network_layer_runs_fused(network *net, int i)
{
    if (i < 1 || i >= net->n) return 0;
    return conv_shortcut_pair(net, i - 1) || conv_yolo_pair(net, i - 1) || xnor_pool_pair(net, i - 1) ||
           conv_pool_pair(net, i - 1);
}

int network_layer_output_skipped(network *net, int i)
{
    if (i < 0 || i >= net->n) return 0;
    return xnor_map_skipped(net, i);
}

/* The layer loop of src/network.c:773-785 without the copies around it.  `gate` (may be NULL) is
 * called once, before the launch that first writes the output of a layer at or after `gate_layer`
 * (a convolution writes the output of the shortcut or yolo layer fused behind it, hence i + 1). */
void dn_forward_gated(network *netp, int gate_layer, void (*gate)(void *), void *gate_arg)
{
    DN_NEED_DEVICE("forward_network_device");
    network net = *netp;
    int i;
    net.train = 0;
    for (i = 0; i < net.n; ++i) {
        layer l = net.layers[i];
        net.index = i;
        if (!l.forward_gpu) dn_fatal("layer without a GPU forward");
        if (gate && gate_layer >= 0 && i + 1 >= gate_layer) {
            gate(gate_arg);
            gate = 0;
        }
        if (l.type == CONVOLUTIONAL && l.xnor && g_fuse_shortcut) {
            i += forward_xnor(net, i);
            l = net.layers[i];
        } else if (forward_conv_shortcut_pair(net, i) || forward_conv_yolo_pair(net, i) ||
                   forward_conv_pool_pair(net, i)) {
            ++i;
            l = net.layers[i];
        } else {
            l.forward_gpu(l, net);
        }
        net.input_gpu = l.output_gpu;
    }
}

void forward_network_device(network *netp) { dn_forward_gated(netp, -1, 0, 0); }

/* The same loop with a HIP event between consecutive layers; layer_ms[i] receives layer i's
 * time on the device (a shortcut that ran inside the convolution before it reports 0), and, when
 * kernel_ms is not NULL, kernel_ms[i] the duration of a convolution's main kernel alone as stamped
 * on its dispatch (-1 for layers without one).  Returns the total (first event to last) in
 * milliseconds.  Events are created once per network size and reused. */
float forward_network_profiled_kernels(network *netp, float *layer_ms, float *kernel_ms)
{
    DN_NEED_DEVICE("forward_network_profiled_kernels");
    static void **ev = 0, **ks = 0, **ke = 0;
    static int nev = 0;
    network net = *netp;
    int i;
    float total;
    if (nev < net.n + 1) {
        ev = (void **)realloc(ev, sizeof(void *) * (size_t)(net.n + 1));
        ks = (void **)realloc(ks, sizeof(void *) * (size_t)(net.n + 1));
        ke = (void **)realloc(ke, sizeof(void *) * (size_t)(net.n + 1));
        if (!ev || !ks || !ke) dn_fatal("Malloc error");
        for (i = nev; i < net.n + 1; ++i) {
            ev[i] = hip_event_create();
            ks[i] = hip_event_create();
            ke[i] = hip_event_create();
        }
        nev = net.n + 1;
    }
    net.train = 0;
    hip_event_record(ev[0]);
    for (i = 0; i < net.n; ++i) {
        layer l = net.layers[i];
        const int first = i;
        int timed = 0;
        net.index = i;
        if (kernel_ms && (l.type == CONVOLUTIONAL || l.type == CONNECTED) && !l.xnor) {
            conv_profile_next(ks[i], ke[i]);
            timed = 1;
        }
        if (l.type == CONVOLUTIONAL && l.xnor && g_fuse_shortcut) {
            if (forward_xnor(net, i)) {
                hip_event_record(ev[i + 1]);
                ++i;
                if (kernel_ms) kernel_ms[i] = -1.f;
                l = net.layers[i];
            }
        } else if (forward_conv_shortcut_pair(net, i) || forward_conv_yolo_pair(net, i) ||
                   forward_conv_pool_pair(net, i)) {
            hip_event_record(ev[i + 1]);
            ++i;
            if (kernel_ms) kernel_ms[i] = -1.f;
            l = net.layers[i];
        } else {
            l.forward_gpu(l, net);
        }
        if (kernel_ms) {
            if (timed && conv_profile_pending()) { /* another kernel served the layer */
                conv_profile_next(0, 0);
                timed = 0;
            }
            kernel_ms[first] = timed ? 0.f : -1.f; /* 0 = to be read after the pass */
        }
        net.input_gpu = l.output_gpu;
        hip_event_record(ev[i + 1]);
    }
    total = hip_event_elapsed_ms(ev[0], ev[net.n]);
    if (layer_ms)
        for (i = 0; i < net.n; ++i) layer_ms[i] = hip_event_elapsed_ms(ev[i], ev[i + 1]);
    if (kernel_ms)
        for (i = 0; i < net.n; ++i)
            if (kernel_ms[i] == 0.f) kernel_ms[i] = hip_event_elapsed_ms(ks[i], ke[i]);
    return total;
}

float forward_network_profiled(network *netp, float *layer_ms)
{
    return forward_network_profiled_kernels(netp, layer_ms, 0);
}

/* src/network.c:1123-1127 */
void pull_network_output(network *net)
{
    layer l = get_network_output_layer(net);
    hip_pull_array(l.output_gpu, l.output, (size_t)l.outputs * l.batch);
}

/* What the host reads after a forward: the yolo heads (the reference pulls them inside
 * forward_yolo_layer_gpu, src/yolo_layer.c:359-361) and the output layer (src/network.c:786). */
void network_pull_outputs(network *netp)
{
    network net = *netp;
    int i;
    for (i = 0; i < net.n - 1; ++i) {
        layer l = net.layers[i];
        if (l.type == YOLO) hip_pull_array(l.output_gpu, l.output, (size_t)l.batch * l.outputs);
    }
    pull_network_output(netp);
}

/* src/network.c:762-788 */
void forward_network_gpu(network *netp)
{
    DN_NEED_DEVICE("forward_network_gpu");
    network net = *netp;
    int i;
    /* a batch submitted with network_predict_submit is still being computed or copied out of the very
     * buffers this pass would write */
    if (network_predict_in_flight(netp))
        dn_fatal("forward_network_gpu: batches submitted with network_predict_submit are in flight; collect them first");
    hip_set_device(net.gpu_index);
    hip_push_array(net.input_gpu, net.input, (size_t)net.inputs * net.batch);
    forward_network_device(netp);
    (void)i;
    network_pull_outputs(netp);
}

/* src/network.c:188-211 */
void forward_network(network *net)
{
    if (net->gpu_index < 0) dn_fatal("forward_network: this library has no CPU path (gpu_index < 0)");
    forward_network_gpu(net);
}

/* src/network.c:497-508 */
float *network_predict(network *net, float *input)
{
    DN_NEED_DEVICE("network_predict");
    network orig = *net;
    float *out;
    net->input = input;
    net->truth = 0;
    net->train = 0;
    net->delta = 0;
    forward_network(net);
    out = net->output;
    *net = orig;
    return out;
}

/* src/network.c:53-63 */
network *load_network(char *cfg, char *weights, int clear)
{
    network *net = parse_network_cfg(cfg);
    if (weights && weights[0] != 0) load_weights(net, weights);
    if (clear) *net->seen = 0;
    return net;
}

/* ---- additions ---------------------------------------------------------------------------- */
float *layer_output_host(network *net, int i)
{
    layer *l;
    if (i < 0 || i >= net->n) dn_fatal("layer_output_host: layer index out of range");
    l = &net->layers[i];
    /* a dropout layer's output is the buffer of the layer before it (src/parser.c:829-836) */
    if (l->type == DROPOUT && i > 0) return layer_output_host(net, i - 1);
    if (xnor_map_skipped(net, i))
        dn_fatal("layer_output_host: in lean mode (network_set_fusion(2)) this convolution's map is not written; "
                 "only the maxpool behind it is");
    if (!l->output) {
        /* sized for the batch the network was built with: set_batch_network may come back up to it */
        const int cap = net->max_batch > l->batch ? net->max_batch : l->batch;
        l->output = (float *)dn_calloc((size_t)l->outputs * cap, sizeof(float));
        if (i == net->n - 1) net->output = l->output;
    }
    hip_pull_array(l->output_gpu, l->output, (size_t)l->outputs * l->batch);
    return l->output;
}

int *layer_indexes_host(network *net, int i)
{
    layer *l;
    if (i < 0 || i >= net->n) dn_fatal("layer_indexes_host: layer index out of range");
    l = &net->layers[i];
    if (l->type != MAXPOOL || !l->indexes_gpu) dn_fatal("layer_indexes_host: layer has no indexes");
    if (i > 0 && xnor_map_skipped(net, i - 1))
        dn_fatal("layer_indexes_host: in lean mode (network_set_fusion(2)) the map this layer pools is not written");
    if (!l->indexes)
        l->indexes = (int *)dn_calloc((size_t)l->outputs * (net->max_batch > l->batch ? net->max_batch : l->batch), sizeof(int));
    /* the forward pass leaves the argmax out (only the backward pass reads it): compute it now from
     * the layer's input, which is still resident (nothing is recycled between layers) */
    forward_maxpool_gpu(i ? net->layers[i - 1].output_gpu : net->input_gpu, l->output_gpu, l->indexes_gpu,
                        l->batch, l->c, l->h, l->w, l->size, l->stride, l->pad);
    hip_pull_int_array(l->indexes_gpu, l->indexes, (size_t)l->outputs * l->batch);
    return l->indexes;
}

void network_set_conv(network *net, int i, const float *weights, const float *biases, const float *scales,
                      const float *rolling_mean, const float *rolling_variance)
{
    layer l;
    if (i >= 0 && i < net->n && net->layers[i].type == LOCAL) { /* weights[nweights], biases[outputs] */
        l = net->layers[i];
        if (weights) memcpy(l.weights, weights, sizeof(float) * (size_t)l.nweights);
        if (biases) memcpy(l.biases, biases, sizeof(float) * (size_t)l.outputs);
        push_local_layer(l);
        return;
    }
    if (i >= 0 && i < net->n && net->layers[i].type == BATCHNORM) { /* c values each; no weights */
        l = net->layers[i];
        if (biases) memcpy(l.biases, biases, sizeof(float) * (size_t)l.c);
        if (scales) memcpy(l.scales, scales, sizeof(float) * (size_t)l.c);
        if (rolling_mean) memcpy(l.rolling_mean, rolling_mean, sizeof(float) * (size_t)l.c);
        if (rolling_variance) memcpy(l.rolling_variance, rolling_variance, sizeof(float) * (size_t)l.c);
        push_batchnorm_layer(l);
        hip_push_array(l.biases_gpu, l.biases, (size_t)l.c);
        return;
    }
    if (i < 0 || i >= net->n || (net->layers[i].type != CONVOLUTIONAL && net->layers[i].type != CONNECTED))
        dn_fatal("network_set_conv: not a convolutional, connected, batchnorm or local layer");
    l = net->layers[i];
    if (weights) memcpy(l.weights, weights, sizeof(float) * (size_t)l.nweights);
    if (biases) memcpy(l.biases, biases, sizeof(float) * (size_t)l.n);
    if (l.batch_normalize) {
        if (scales) memcpy(l.scales, scales, sizeof(float) * (size_t)l.n);
        if (rolling_mean) memcpy(l.rolling_mean, rolling_mean, sizeof(float) * (size_t)l.n);
        if (rolling_variance) memcpy(l.rolling_variance, rolling_variance, sizeof(float) * (size_t)l.n);
    }
    push_convolutional_layer(l);
}

int network_num_layers(network *net) { return net->n; }
float *network_input_gpu(network *net) { return net->input_gpu; }

void network_info(network *net, int *iv)
{
    iv[0] = net->n;
    iv[1] = net->batch;
    iv[2] = net->h;
    iv[3] = net->w;
    iv[4] = net->c;
    iv[5] = net->inputs;
    iv[6] = net->outputs;
}

void network_layer_info(network *net, int i, int *iv, float *fv)
{
    layer l;
    int k = 0;
    if (i < 0 || i >= net->n) dn_fatal("network_layer_info: layer index out of range");
    l = net->layers[i];
    iv[k++] = (int)l.type;
    iv[k++] = l.batch;
    iv[k++] = l.h;
    iv[k++] = l.w;
    iv[k++] = l.c;
    iv[k++] = l.out_h;
    iv[k++] = l.out_w;
    iv[k++] = l.out_c;
    iv[k++] = l.n;
    iv[k++] = l.size;
    iv[k++] = l.stride;
    iv[k++] = l.pad;
    iv[k++] = l.groups;
    iv[k++] = l.batch_normalize;
    iv[k++] = (int)l.activation;
    iv[k++] = l.binary;
    iv[k++] = l.xnor;
    iv[k++] = l.index;
    iv[k++] = l.inputs;
    iv[k++] = l.outputs;
    iv[k++] = l.nweights;
    iv[k++] = l.classes;
    iv[k++] = l.total;
    iv[k++] = l.reverse;
    iv[k++] = (int)(l.workspace_size / sizeof(float));
    iv[k++] = l.nbiases;
    iv[k++] = l.truths;
    iv[k++] = l.max_boxes;
    fv[0] = l.alpha;
    fv[1] = l.beta;
    fv[2] = l.scale;
    fv[3] = l.temperature;
}

int network_route_inputs(network *net, int i, int *layers, int *sizes, int cap)
{
    layer l;
    int j;
    if (i < 0 || i >= net->n) dn_fatal("network_route_inputs: layer index out of range");
    l = net->layers[i];
    if (l.type != ROUTE) return 0;
    for (j = 0; j < l.n && j < cap; ++j) {
        layers[j] = l.input_layers[j];
        sizes[j] = l.input_sizes[j];
    }
    return l.n;
}

/* numops of the reference (examples/darknet.c:81-114): the convolutional and connected terms */
double network_conv_flops(network *net)
{
    double ops = 0;
    int i;
    for (i = 0; i < net->n; ++i) {
        layer l = net->layers[i];
        if (l.type == CONVOLUTIONAL)
            ops += 2.0 * l.n * l.size * l.size * (l.c / l.groups) * l.out_h * l.out_w;
        else if (l.type == CONNECTED)
            ops += 2.0 * l.inputs * l.outputs;
    }
    return ops;
}
