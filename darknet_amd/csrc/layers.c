/*
 * layers.c - constructors and forward_gpu adapters of the layer types on the inference path.
 *
 * A constructor fixes the geometry exactly as the reference's make_*_layer does and allocates
 * the device buffers the forward needs; the adapter spells the by-value `layer` / `network`
 * out into the plain-pointer entry points of darknet_hip.h.  No layer has a CPU forward.
 */
#include <math.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include "host.h"

int dn_verbose = 1;

void network_set_verbose(int on) { dn_verbose = on; }

/* ---- convolutional: src/convolutional_layer.c:176-328 ------------------------------------- */
layer make_convolutional_layer(int batch, int h, int w, int c, int n, int groups, int size, int stride,
                               int padding, ACTIVATION activation, int batch_normalize, int binary,
                               int xnor, int adam)
{
    layer l;
    size_t packed;
    int i;
    (void)adam;
    memset(&l, 0, sizeof l);
    if (groups < 1) groups = 1;
    if (c % groups || n % groups) dn_fatal("convolutional layer: groups must divide channels and filters");
    l.type = CONVOLUTIONAL;
    l.groups = groups;
    l.h = h;
    l.w = w;
    l.c = c;
    l.n = n;
    l.binary = binary;
    l.xnor = xnor;
    l.batch = batch;
    l.stride = stride;
    l.size = size;
    l.pad = padding;
    l.batch_normalize = batch_normalize;
    l.activation = activation;
    l.nweights = c / groups * n * size * size;
    l.nbiases = n;
    l.out_h = (h + 2 * padding - size) / stride + 1; /* :66-74 */
    l.out_w = (w + 2 * padding - size) / stride + 1;
    l.out_c = n;
    l.outputs = l.out_h * l.out_w * l.out_c;
    l.inputs = l.w * l.h * l.c;
    if (l.out_h <= 0 || l.out_w <= 0) dn_fatal("convolutional layer: empty output");

    /* Host parameters start as the reference leaves them apart from the random draw: biases 0,
     * scales 1, rolling statistics 0 (:198, :237-248).  Weights start at zero; callers load a
     * weights file or write them through network_set_conv. */
    l.weights = (float *)dn_calloc((size_t)l.nweights, sizeof(float));
    l.biases = (float *)dn_calloc((size_t)n, sizeof(float));
    if (batch_normalize) {
        l.scales = (float *)dn_calloc((size_t)n, sizeof(float));
        for (i = 0; i < n; ++i) l.scales[i] = 1;
        l.rolling_mean = (float *)dn_calloc((size_t)n, sizeof(float));
        l.rolling_variance = (float *)dn_calloc((size_t)n, sizeof(float));
    }

    l.forward_gpu = forward_convolutional_layer_gpu;
    if (gpu_index < 0) dn_fatal("this library has no CPU path: gpu_index must name a device");
    l.weights_gpu = hip_make_array(l.weights, (size_t)l.nweights);
    l.biases_gpu = hip_make_array(l.biases, (size_t)n);
    l.output_gpu = hip_make_array(0, (size_t)batch * l.outputs);
    if (batch_normalize) {
        l.scales_gpu = hip_make_array(l.scales, (size_t)n);
        l.rolling_mean_gpu = hip_make_array(l.rolling_mean, (size_t)n);
        l.rolling_variance_gpu = hip_make_array(l.rolling_variance, (size_t)n);
    }
    if (xnor) {
        if (groups != 1) dn_fatal("convolutional layer: xnor with groups is not supported");
        l.xnor_wbits_gpu = (unsigned *)hip_make_int_array(0, xnor_weight_words(n, c, size));
        l.xnor_xbits_gpu = (unsigned *)hip_make_int_array(0, xnor_input_words(batch, c, h, w));
        l.xnor_wmean_gpu = hip_make_array(0, (size_t)n);
    } else {
        packed = conv_packed_floats(n, c, groups, size);
        if (packed) {
            l.weights_packed_gpu = hip_make_array(0, packed);
            conv_pack_weights_gpu(l.weights_gpu, l.weights_packed_gpu, n, c, groups, size);
        }
    }
    /* what the reference would ask of net->workspace for its im2col buffer (:118) */
    l.workspace_size = (size_t)l.out_h * l.out_w * size * size * (c / groups) * sizeof(float);

    if (dn_verbose)
        fprintf(stderr, "conv  %5d %2d x%2d /%2d  %4d x%4d x%4d   ->  %4d x%4d x%4d  %5.3f BFLOPs\n", n, size,
                size, stride, w, h, c, l.out_w, l.out_h, l.out_c,
                (2.0 * l.n * l.size * l.size * l.c / l.groups * l.out_h * l.out_w) / 1000000000.);
    return l;
}

void forward_convolutional_layer_gpu(layer l, network net)
{
    if (l.xnor) {
        forward_convolutional_xnor_gpu(net.input_gpu, l.weights_gpu, l.xnor_wbits_gpu, l.xnor_wmean_gpu,
                                       l.xnor_xbits_gpu, l.biases_gpu, l.scales_gpu, l.rolling_mean_gpu,
                                       l.rolling_variance_gpu, l.output_gpu, l.batch, l.c, l.h, l.w, l.n,
                                       l.size, l.stride, l.pad, l.batch_normalize, (int)l.activation);
        return;
    }
    forward_convolutional_gpu(net.input_gpu, l.weights_gpu, l.weights_packed_gpu, l.biases_gpu, l.scales_gpu,
                              l.rolling_mean_gpu, l.rolling_variance_gpu, l.output_gpu, l.batch, l.c, l.h,
                              l.w, l.n, l.groups, l.size, l.stride, l.pad, l.batch_normalize,
                              (int)l.activation);
}

/* Host -> device for every parameter vector, then the MFMA repack (the reference's
 * push_convolutional_layer, src/convolutional_kernels.cu:286-297, is where a weights file load
 * ends, src/parser.c:1210-1214). */
void push_convolutional_layer(layer l)
{
    hip_push_array(l.weights_gpu, l.weights, (size_t)l.nweights);
    hip_push_array(l.biases_gpu, l.biases, (size_t)l.n);
    if (l.batch_normalize) {
        hip_push_array(l.scales_gpu, l.scales, (size_t)l.n);
        hip_push_array(l.rolling_mean_gpu, l.rolling_mean, (size_t)l.n);
        hip_push_array(l.rolling_variance_gpu, l.rolling_variance, (size_t)l.n);
    }
    if (l.weights_packed_gpu)
        conv_pack_weights_gpu(l.weights_gpu, l.weights_packed_gpu, l.n, l.c, l.groups, l.size);
}

void pull_convolutional_layer(layer l)
{
    hip_pull_array(l.weights_gpu, l.weights, (size_t)l.nweights);
    hip_pull_array(l.biases_gpu, l.biases, (size_t)l.n);
    if (l.batch_normalize) {
        hip_pull_array(l.scales_gpu, l.scales, (size_t)l.n);
        hip_pull_array(l.rolling_mean_gpu, l.rolling_mean, (size_t)l.n);
        hip_pull_array(l.rolling_variance_gpu, l.rolling_variance, (size_t)l.n);
    }
}

/* ---- maxpool: src/maxpool_layer.c:21-52 ---------------------------------------------------- */
layer make_maxpool_layer(int batch, int h, int w, int c, int size, int stride, int padding)
{
    layer l;
    memset(&l, 0, sizeof l);
    l.type = MAXPOOL;
    l.batch = batch;
    l.h = h;
    l.w = w;
    l.c = c;
    l.pad = padding;
    l.out_w = (w + padding - size) / stride + 1;
    l.out_h = (h + padding - size) / stride + 1;
    l.out_c = c;
    l.outputs = l.out_h * l.out_w * l.out_c;
    l.inputs = h * w * c;
    l.size = size;
    l.stride = stride;
    l.forward_gpu = forward_maxpool_layer_gpu;
    l.indexes_gpu = hip_make_int_array(0, (size_t)l.outputs * batch);
    l.output_gpu = hip_make_array(0, (size_t)l.outputs * batch);
    if (dn_verbose)
        fprintf(stderr, "max          %d x %d / %d  %4d x%4d x%4d   ->  %4d x%4d x%4d\n", size, size, stride, w,
                h, c, l.out_w, l.out_h, l.out_c);
    return l;
}

void forward_maxpool_layer_gpu(layer l, network net)
{
    /* indexes feed only the backward pass; inference writes them when asked to train-compatible
     * behaviour is wanted (net.train) or a caller reads them through layer_indexes_host. */
    forward_maxpool_gpu(net.input_gpu, l.output_gpu, l.indexes_gpu, l.batch, l.c, l.h, l.w, l.size, l.stride,
                        l.pad);
}

/* ---- route: src/route_layer.c:7-38 --------------------------------------------------------- */
layer make_route_layer(int batch, int n, int *input_layers, int *input_sizes)
{
    layer l;
    int i, outputs = 0;
    memset(&l, 0, sizeof l);
    if (dn_verbose) fprintf(stderr, "route ");
    l.type = ROUTE;
    l.batch = batch;
    l.n = n;
    l.input_layers = input_layers;
    l.input_sizes = input_sizes;
    for (i = 0; i < n; ++i) {
        if (dn_verbose) fprintf(stderr, " %d", input_layers[i]);
        outputs += input_sizes[i];
    }
    if (dn_verbose) fprintf(stderr, "\n");
    l.outputs = outputs;
    l.inputs = outputs;
    l.forward_gpu = forward_route_layer_gpu;
    l.output_gpu = hip_make_array(0, (size_t)outputs * batch);
    return l;
}

void forward_route_layer_gpu(layer l, network net)
{
    const float *srcs[8];
    int i;
    if (l.n > 8) dn_fatal("route layer: more than 8 sources");
    for (i = 0; i < l.n; ++i) srcs[i] = net.layers[l.input_layers[i]].output_gpu;
    forward_route_gpu(srcs, l.input_sizes, l.n, l.output_gpu, l.batch);
}

/* ---- shortcut: src/shortcut_layer.c:9-39.  (w2,h2,c2) is the `from` layer's output. -------- */
layer make_shortcut_layer(int batch, int index, int w, int h, int c, int w2, int h2, int c2)
{
    layer l;
    memset(&l, 0, sizeof l);
    if (dn_verbose)
        fprintf(stderr, "res  %3d                %4d x%4d x%4d   ->  %4d x%4d x%4d\n", index, w2, h2, c2, w, h, c);
    l.type = SHORTCUT;
    l.batch = batch;
    l.w = w2;
    l.h = h2;
    l.c = c2;
    l.out_w = w;
    l.out_h = h;
    l.out_c = c;
    l.outputs = w * h * c;
    l.inputs = l.outputs;
    l.index = index;
    l.forward_gpu = forward_shortcut_layer_gpu;
    l.output_gpu = hip_make_array(0, (size_t)l.outputs * batch);
    return l;
}

void forward_shortcut_layer_gpu(layer l, network net)
{
    forward_shortcut_gpu(net.input_gpu, net.layers[l.index].output_gpu, l.output_gpu, l.batch, l.w, l.h, l.c,
                         l.out_w, l.out_h, l.out_c, l.alpha, l.beta, (int)l.activation);
}

/* ---- upsample: src/upsample_layer.c:7-43 --------------------------------------------------- */
layer make_upsample_layer(int batch, int w, int h, int c, int stride)
{
    layer l;
    memset(&l, 0, sizeof l);
    l.type = UPSAMPLE;
    l.batch = batch;
    l.w = w;
    l.h = h;
    l.c = c;
    l.out_w = w * stride;
    l.out_h = h * stride;
    l.out_c = c;
    if (stride < 0) {
        stride = -stride;
        l.reverse = 1;
        l.out_w = w / stride;
        l.out_h = h / stride;
    }
    l.stride = stride;
    l.outputs = l.out_w * l.out_h * l.out_c;
    l.inputs = l.w * l.h * l.c;
    l.forward_gpu = forward_upsample_layer_gpu;
    l.output_gpu = hip_make_array(0, (size_t)l.outputs * batch);
    if (dn_verbose) {
        if (l.reverse)
            fprintf(stderr, "downsample         %2dx  %4d x%4d x%4d   ->  %4d x%4d x%4d\n", stride, w, h, c,
                    l.out_w, l.out_h, l.out_c);
        else
            fprintf(stderr, "upsample           %2dx  %4d x%4d x%4d   ->  %4d x%4d x%4d\n", stride, w, h, c,
                    l.out_w, l.out_h, l.out_c);
    }
    return l;
}

void forward_upsample_layer_gpu(layer l, network net)
{
    if (l.reverse) dn_fatal("upsample layer: the reverse (downsample) direction is not built");
    upsample_gpu(net.input_gpu, l.w, l.h, l.c, l.batch, l.stride, 1, l.scale, l.output_gpu);
}

/* ---- yolo: src/yolo_layer.c:13-61.  biases hold the anchors (default .5). ------------------ */
layer make_yolo_layer(int batch, int w, int h, int n, int total, int *mask, int classes)
{
    layer l;
    int i;
    memset(&l, 0, sizeof l);
    l.type = YOLO;
    l.n = n;
    l.total = total;
    l.batch = batch;
    l.h = h;
    l.w = w;
    l.c = n * (classes + 4 + 1);
    l.out_w = l.w;
    l.out_h = l.h;
    l.out_c = l.c;
    l.classes = classes;
    l.biases = (float *)dn_calloc((size_t)total * 2, sizeof(float));
    if (mask) {
        l.mask = mask;
    } else {
        l.mask = (int *)dn_calloc((size_t)n, sizeof(int));
        for (i = 0; i < n; ++i) l.mask[i] = i;
    }
    l.outputs = h * w * n * (classes + 4 + 1);
    l.inputs = l.outputs;
    l.truths = 90 * (4 + 1);
    l.output = (float *)dn_calloc((size_t)batch * l.outputs, sizeof(float));
    for (i = 0; i < total * 2; ++i) l.biases[i] = .5f;
    l.forward_gpu = forward_yolo_layer_gpu;
    l.output_gpu = hip_make_array(0, (size_t)batch * l.outputs);
    if (dn_verbose) fprintf(stderr, "yolo\n");
    return l;
}

/* The host copy of a yolo head's output is refreshed by forward_network_gpu once the whole
 * forward has been queued, not here, so the device is not drained in the middle of the network
 * (the reference pulls at this point, src/yolo_layer.c:359-361; the host sees the same data
 * when network_predict returns). */
void forward_yolo_layer_gpu(layer l, network net)
{
    forward_yolo_gpu(net.input_gpu, l.output_gpu, l.batch, l.w, l.h, l.n, l.classes);
}

/* ---- avgpool: src/avgpool_layer.c:5-33 ------------------------------------------------------ */
layer make_avgpool_layer(int batch, int w, int h, int c)
{
    layer l;
    memset(&l, 0, sizeof l);
    if (dn_verbose) fprintf(stderr, "avg                     %4d x%4d x%4d   ->  %4d\n", w, h, c, c);
    l.type = AVGPOOL;
    l.batch = batch;
    l.h = h;
    l.w = w;
    l.c = c;
    l.out_w = 1;
    l.out_h = 1;
    l.out_c = c;
    l.outputs = l.out_c;
    l.inputs = h * w * c;
    l.forward_gpu = forward_avgpool_layer_gpu;
    l.output_gpu = hip_make_array(0, (size_t)l.outputs * batch);
    return l;
}

void forward_avgpool_layer_gpu(layer l, network net)
{
    forward_avgpool_gpu(net.input_gpu, l.output_gpu, l.batch, l.c, l.h, l.w);
}

/* ---- softmax: src/softmax_layer.c:11-37 (no tree, no spatial mode) -------------------------- */
layer make_softmax_layer(int batch, int inputs, int groups)
{
    layer l;
    memset(&l, 0, sizeof l);
    if (groups < 1 || inputs % groups) dn_fatal("softmax layer: groups must divide inputs");
    if (dn_verbose) fprintf(stderr, "softmax                                        %4d\n", inputs);
    l.type = SOFTMAX;
    l.batch = batch;
    l.groups = groups;
    l.inputs = inputs;
    l.outputs = inputs;
    l.forward_gpu = forward_softmax_layer_gpu;
    l.output_gpu = hip_make_array(0, (size_t)inputs * batch);
    return l;
}

void forward_softmax_layer_gpu(layer l, network net)
{
    softmax_gpu(net.input_gpu, l.inputs / l.groups, l.batch, l.inputs, l.groups, l.inputs / l.groups, 1,
                l.temperature, l.output_gpu);
}

/* ---- src/layer.c:6-97 ----------------------------------------------------------------------- */
void free_layer(layer l)
{
    free(l.mask);
    free(l.input_layers);
    free(l.input_sizes);
    free(l.biases);
    free(l.scales);
    free(l.weights);
    free(l.rolling_mean);
    free(l.rolling_variance);
    free(l.output);
    free(l.indexes);
    if (l.indexes_gpu) hip_free((float *)l.indexes_gpu);
    if (l.weights_gpu) hip_free(l.weights_gpu);
    if (l.biases_gpu) hip_free(l.biases_gpu);
    if (l.scales_gpu) hip_free(l.scales_gpu);
    if (l.rolling_mean_gpu) hip_free(l.rolling_mean_gpu);
    if (l.rolling_variance_gpu) hip_free(l.rolling_variance_gpu);
    if (l.output_gpu) hip_free(l.output_gpu);
    if (l.binary_weights_gpu) hip_free(l.binary_weights_gpu);
    if (l.binary_input_gpu) hip_free(l.binary_input_gpu);
    if (l.weights_packed_gpu) hip_free(l.weights_packed_gpu);
    if (l.xnor_wbits_gpu) hip_free((float *)l.xnor_wbits_gpu);
    if (l.xnor_xbits_gpu) hip_free((float *)l.xnor_xbits_gpu);
    if (l.xnor_wmean_gpu) hip_free(l.xnor_wmean_gpu);
}
