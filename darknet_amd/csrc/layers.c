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
    /* The reference hands a 1x1 layer's image to the GEMM as it lies, whatever stride and padding say
     * (src/convolutional_layer.c:468-469): with stride 2 it multiplies the first out_h*out_w floats
     * of every channel block instead of the strided pixels, with padding it reads past the image.
     * No cfg in the tree asks for that, and there is no meaningful result to be identical to, so the
     * geometry is refused where the network is built rather than at its first forward. */
    if (size == 1 && (stride != 1 || padding != 0))
        dn_fatal("convolutional layer: a 1x1 kernel needs stride 1 and no padding (the reference's result for "
                 "anything else is a misread image, src/convolutional_layer.c:468-469)");
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
        xnor_pack_weights_gpu(l.weights_gpu, l.xnor_wbits_gpu, l.xnor_wmean_gpu, n, c, size);
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
        /* sign bits and mean|w| were written when the weights last changed (push_convolutional_layer) */
        forward_convolutional_xnor_packed_gpu(net.input_gpu, l.xnor_wbits_gpu, l.xnor_wmean_gpu,
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
    if (l.xnor_wbits_gpu) xnor_pack_weights_gpu(l.weights_gpu, l.xnor_wbits_gpu, l.xnor_wmean_gpu, l.n, l.c, l.size);
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
    /* the argmax indexes feed only the backward pass: inference leaves them out (a quarter of the
     * layer's write traffic); layer_indexes_host() computes them on demand */
    forward_maxpool_gpu(net.input_gpu, l.output_gpu, net.train ? l.indexes_gpu : 0, l.batch, l.c, l.h, l.w, l.size,
                        l.stride, l.pad);
}

/* ---- route: src/route_layer.c:7-38 --------------------------------------------------------- */
static layer route_layer_without_output(int batch, int n, int *input_layers, int *input_sizes)
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
    return l;
}

layer make_route_layer(int batch, int n, int *input_layers, int *input_sizes)
{
    layer l = route_layer_without_output(batch, n, input_layers, input_sizes);
    l.output_gpu = hip_make_array(0, (size_t)l.outputs * batch);
    return l;
}

/* A route of one source as a view of that source's device buffer: what the reference copies
 * (src/route_layer.c:74-87) is already there.  The buffer stays the source's: free_layer leaves it. */
layer make_route_view(int batch, int input_layer, int input_size, float *source_output_gpu)
{
    int *layers = (int *)dn_calloc(1, sizeof(int)), *sizes = (int *)dn_calloc(1, sizeof(int));
    layer l;
    layers[0] = input_layer;
    sizes[0] = input_size;
    l = route_layer_without_output(batch, 1, layers, sizes);
    l.output_gpu = source_output_gpu;
    l.output_gpu_is_view = 1;
    return l;
}

void forward_route_layer_gpu(layer l, network net)
{
    const float *srcs[8];
    int i;
    if (l.n > 8) dn_fatal("route layer: more than 8 sources");
    for (i = 0; i < l.n; ++i) srcs[i] = net.layers[l.input_layers[i]].output_gpu;
    if (l.output_gpu_is_view) return; /* its one source's buffer is its output (make_route_view) */
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
    l.output = hip_host_alloc((size_t)batch * l.outputs); /* pinned: network_predict pulls it every call */
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
/* ---- connected: src/connected_layer.c:14-110.  out[b][o] = sum_k in[b][k]*w[o][k] is the 1x1
 * convolution of a 1x1 image with `inputs` channels, so the layer runs on the convolution
 * kernel (M = outputs, K = inputs, N = batch) with the same batch-norm / bias / activation
 * tail (forward_connected_layer :150-167: gemm, forward_batchnorm_layer or add_bias, activate). */
layer make_connected_layer(int batch, int inputs, int outputs, ACTIVATION activation, int batch_normalize,
                           int adam)
{
    layer l;
    size_t packed;
    int i;
    (void)adam;
    memset(&l, 0, sizeof l);
    l.type = CONNECTED;
    l.inputs = inputs;
    l.outputs = outputs;
    l.batch = batch;
    l.batch_normalize = batch_normalize;
    l.h = 1;
    l.w = 1;
    l.c = inputs;
    l.out_h = 1;
    l.out_w = 1;
    l.out_c = outputs;
    l.n = outputs;
    l.size = 1;
    l.stride = 1;
    l.groups = 1;
    l.activation = activation;
    l.nweights = inputs * outputs;
    l.nbiases = outputs;
    if ((long)inputs * outputs >= (1L << 31)) dn_fatal("connected layer: too many weights");
    l.weights = (float *)dn_calloc((size_t)l.nweights, sizeof(float));
    l.biases = (float *)dn_calloc((size_t)outputs, sizeof(float));
    l.forward_gpu = forward_connected_layer_gpu;
    if (gpu_index < 0) dn_fatal("this library has no CPU path: gpu_index must name a device");
    l.weights_gpu = hip_make_array(l.weights, (size_t)l.nweights);
    l.biases_gpu = hip_make_array(l.biases, (size_t)outputs);
    l.output_gpu = hip_make_array(0, (size_t)batch * outputs);
    if (batch_normalize) {
        l.scales = (float *)dn_calloc((size_t)outputs, sizeof(float));
        for (i = 0; i < outputs; ++i) l.scales[i] = 1;
        l.rolling_mean = (float *)dn_calloc((size_t)outputs, sizeof(float));
        l.rolling_variance = (float *)dn_calloc((size_t)outputs, sizeof(float));
        l.scales_gpu = hip_make_array(l.scales, (size_t)outputs);
        l.rolling_mean_gpu = hip_make_array(l.rolling_mean, (size_t)outputs);
        l.rolling_variance_gpu = hip_make_array(l.rolling_variance, (size_t)outputs);
    }
    packed = conv_packed_floats(outputs, inputs, 1, 1);
    if (packed) {
        l.weights_packed_gpu = hip_make_array(0, packed);
        conv_pack_weights_gpu(l.weights_gpu, l.weights_packed_gpu, outputs, inputs, 1, 1);
    }
    if (dn_verbose) fprintf(stderr, "connected                            %4d  ->  %4d\n", inputs, outputs);
    return l;
}

void forward_connected_layer_gpu(layer l, network net)
{
    /* small batches are bound by one pass over the weights: the streaming kernel does that pass at
     * twice the rate of the tiled one; from 17 images on the matrix cores win */
    if (!l.batch_normalize && l.batch <= 16) {
        forward_connected_stream_gpu(net.input_gpu, l.weights_gpu, l.biases_gpu, l.output_gpu, l.batch, l.inputs,
                                     l.outputs, (int)l.activation);
        return;
    }
    forward_convolutional_gpu(net.input_gpu, l.weights_gpu, l.weights_packed_gpu, l.biases_gpu, l.scales_gpu,
                              l.rolling_mean_gpu, l.rolling_variance_gpu, l.output_gpu, l.batch, l.inputs, 1, 1,
                              l.outputs, 1, 1, 1, 0, l.batch_normalize, (int)l.activation);
}

void push_connected_layer(layer l) { push_convolutional_layer(l); }
void pull_connected_layer(layer l) { pull_convolutional_layer(l); }

/* ---- dropout: src/dropout_layer.c:7-27.  At inference the layer does nothing
 * (forward_dropout_layer :38-41); its output IS the previous layer's output, which the cfg
 * parser wires up as src/parser.c:829-836 does. --------------------------------------------- */
/* ---- batchnorm as a layer of its own: src/batchnorm_layer.c:6-67, inference forward :189-235 - */
layer make_batchnorm_layer(int batch, int w, int h, int c)
{
    layer l;
    int i;
    memset(&l, 0, sizeof l);
    if (batch <= 0 || w <= 0 || h <= 0 || c <= 0) dn_fatal("batchnorm layer: bad geometry");
    l.type = BATCHNORM;
    l.batch = batch;
    l.h = l.out_h = h;
    l.w = l.out_w = w;
    l.c = l.out_c = c;
    l.inputs = w * h * c;
    l.outputs = l.inputs;
    l.scales = (float *)dn_calloc((size_t)c, sizeof(float));
    l.biases = (float *)dn_calloc((size_t)c, sizeof(float));
    for (i = 0; i < c; ++i) l.scales[i] = 1;
    l.rolling_mean = (float *)dn_calloc((size_t)c, sizeof(float));
    l.rolling_variance = (float *)dn_calloc((size_t)c, sizeof(float));
    l.forward_gpu = forward_batchnorm_layer_gpu;
    if (gpu_index < 0) dn_fatal("this library has no CPU path: gpu_index must name a device");
    l.output_gpu = hip_make_array(0, (size_t)batch * l.outputs);
    l.biases_gpu = hip_make_array(l.biases, (size_t)c);
    l.scales_gpu = hip_make_array(l.scales, (size_t)c);
    l.rolling_mean_gpu = hip_make_array(l.rolling_mean, (size_t)c);
    l.rolling_variance_gpu = hip_make_array(l.rolling_variance, (size_t)c);
    if (dn_verbose) fprintf(stderr, "Batch Normalization Layer: %d x %d x %d image\n", w, h, c);
    return l;
}

/* The inference branch: copy, normalize with the rolling statistics, scale, bias - one pass. */
void forward_batchnorm_layer_gpu(layer l, network net)
{
    if (net.train) dn_fatal("forward_batchnorm_layer_gpu: training (batch statistics) is not served");
    forward_batchnorm_gpu(net.input_gpu, l.output_gpu, l.scales_gpu, l.biases_gpu, l.rolling_mean_gpu,
                          l.rolling_variance_gpu, l.batch, l.out_c, l.out_h * l.out_w);
}

/* src/batchnorm_layer.c:176-187: the three vectors a weights file holds for this layer (the biases
 * are not part of it, src/parser.c:979-990,1122-1133) */
void pull_batchnorm_layer(layer l)
{
    hip_pull_array(l.scales_gpu, l.scales, (size_t)l.c);
    hip_pull_array(l.rolling_mean_gpu, l.rolling_mean, (size_t)l.c);
    hip_pull_array(l.rolling_variance_gpu, l.rolling_variance, (size_t)l.c);
}

void push_batchnorm_layer(layer l)
{
    hip_push_array(l.scales_gpu, l.scales, (size_t)l.c);
    hip_push_array(l.rolling_mean_gpu, l.rolling_mean, (size_t)l.c);
    hip_push_array(l.rolling_variance_gpu, l.rolling_variance, (size_t)l.c);
}

layer make_dropout_layer(int batch, int inputs, float probability)
{
    layer l;
    memset(&l, 0, sizeof l);
    l.type = DROPOUT;
    l.probability = probability;
    l.inputs = inputs;
    l.outputs = inputs;
    l.batch = batch;
    l.scale = (float)(1. / (1. - probability));
    l.forward_gpu = forward_dropout_layer_gpu;
    if (dn_verbose) fprintf(stderr, "dropout       p = %.2f               %4d  ->  %4d\n", probability, inputs, inputs);
    return l;
}

void forward_dropout_layer_gpu(layer l, network net)
{
    (void)l;
    (void)net;
}

/* ---- reorg: src/reorg_layer.c:8-58, forward :88-107 ---------------------------------------- */
layer make_reorg_layer(int batch, int w, int h, int c, int stride, int reverse, int flatten, int extra)
{
    layer l;
    memset(&l, 0, sizeof l);
    l.type = REORG;
    l.batch = batch;
    l.stride = stride;
    l.extra = extra;
    l.h = h;
    l.w = w;
    l.c = c;
    l.flatten = flatten;
    if (stride < 1) dn_fatal("reorg layer: stride must be at least 1");
    if (reverse) {
        l.out_w = w * stride;
        l.out_h = h * stride;
        l.out_c = c / (stride * stride);
    } else {
        l.out_w = w / stride;
        l.out_h = h / stride;
        l.out_c = c * (stride * stride);
    }
    l.reverse = reverse;
    l.outputs = l.out_h * l.out_w * l.out_c;
    l.inputs = h * w * c;
    if (l.extra) {
        l.out_w = l.out_h = l.out_c = 0;
        l.outputs = l.inputs + l.extra;
    }
    if (!extra && !flatten && l.outputs != l.inputs)
        dn_fatal("reorg layer: stride must divide width and height (and stride*stride the channels when reversed)");
    if (dn_verbose) {
        if (extra) fprintf(stderr, "reorg              %4d   ->  %4d\n", l.inputs, l.outputs);
        else fprintf(stderr, "reorg              /%2d  %4d x%4d x%4d   ->  %4d x%4d x%4d\n", stride, w, h, c, l.out_w,
                     l.out_h, l.out_c);
    }
    l.forward_gpu = forward_reorg_layer_gpu;
    l.output_gpu = hip_make_array(0, (size_t)l.outputs * batch); /* zero: the `extra` tail stays 0 */
    return l;
}

void forward_reorg_layer_gpu(layer l, network net)
{
    int i;
    if (l.flatten) {
        flatten_gpu(net.input_gpu, l.w * l.h, l.c, l.batch, l.reverse ? 0 : 1, l.output_gpu);
    } else if (l.extra) {
        for (i = 0; i < l.batch; ++i)
            copy_gpu_offset(l.inputs, net.input_gpu, i * l.inputs, 1, l.output_gpu, i * l.outputs, 1);
    } else if (l.reverse) {
        reorg_gpu(net.input_gpu, l.w, l.h, l.c, l.batch, l.stride, 1, l.output_gpu);
    } else {
        reorg_gpu(net.input_gpu, l.w, l.h, l.c, l.batch, l.stride, 0, l.output_gpu);
    }
}

/* ---- crop: src/crop_layer.c:18-51; inference takes the centred window ---------------------- */
layer make_crop_layer(int batch, int h, int w, int c, int crop_height, int crop_width, int flip, float angle,
                      float saturation, float exposure)
{
    layer l;
    (void)angle;
    (void)saturation;
    (void)exposure;
    memset(&l, 0, sizeof l);
    if (dn_verbose) fprintf(stderr, "Crop Layer: %d x %d -> %d x %d x %d image\n", h, w, crop_height, crop_width, c);
    if (crop_height > h || crop_width > w || crop_height < 1 || crop_width < 1)
        dn_fatal("crop layer: the window must fit inside the input");
    l.type = CROP;
    l.batch = batch;
    l.h = h;
    l.w = w;
    l.c = c;
    l.scale = (float)crop_height / h;
    l.flip = flip;
    l.out_w = crop_width;
    l.out_h = crop_height;
    l.out_c = c;
    l.inputs = l.w * l.h * l.c;
    l.outputs = l.out_w * l.out_h * l.out_c;
    l.forward_gpu = forward_crop_layer_gpu;
    l.output_gpu = hip_make_array(0, (size_t)l.outputs * batch);
    return l;
}

void forward_crop_layer_gpu(layer l, network net)
{
    forward_crop_gpu(net.input_gpu, l.output_gpu, l.batch, l.c, l.h, l.w, l.out_h, l.out_w, l.noadjust);
}

/* ---- cost: src/cost_layer.c:40-63.  Without a truth the forward returns at once (:79); the
 * layer only has to exist so that cfgs ending in [cost] parse, and is skipped when the
 * network's output layer is looked up (src/network.c:689-697). ------------------------------- */
layer make_cost_layer(int batch, int inputs, int cost_type, float scale)
{
    layer l;
    (void)cost_type;
    memset(&l, 0, sizeof l);
    if (dn_verbose) fprintf(stderr, "cost                                           %4d\n", inputs);
    l.type = COST;
    l.scale = scale;
    l.batch = batch;
    l.inputs = inputs;
    l.outputs = inputs;
    l.forward_gpu = forward_cost_layer_gpu;
    l.output_gpu = hip_make_array(0, (size_t)inputs * batch);
    return l;
}

void forward_cost_layer_gpu(layer l, network net)
{
    (void)l;
    (void)net;
}

/* ---- region (yolov2 head): src/region_layer.c:13-56.  biases hold the n anchors in cell
 * units (default .5). --------------------------------------------------------------------------- */
layer make_region_layer(int batch, int w, int h, int n, int classes, int coords)
{
    layer l;
    int i;
    memset(&l, 0, sizeof l);
    if (coords != 4) dn_fatal("region layer: coords must be 4 (forward_region_gpu and region_decode_gpu serve nothing else)");
    l.type = REGION;
    l.n = n;
    l.batch = batch;
    l.h = h;
    l.w = w;
    l.c = n * (classes + coords + 1);
    l.out_w = l.w;
    l.out_h = l.h;
    l.out_c = l.c;
    l.classes = classes;
    l.coords = coords;
    l.biases = (float *)dn_calloc((size_t)n * 2, sizeof(float));
    l.outputs = h * w * n * (classes + coords + 1);
    l.inputs = l.outputs;
    l.truths = 30 * (l.coords + 1);
    l.output = hip_host_alloc((size_t)batch * l.outputs);
    for (i = 0; i < n * 2; ++i) l.biases[i] = .5f;
    l.forward_gpu = forward_region_layer_gpu;
    l.output_gpu = hip_make_array(0, (size_t)batch * l.outputs);
    if (dn_verbose) fprintf(stderr, "detection\n");
    return l;
}

void forward_region_layer_gpu(layer l, network net)
{
    forward_region_gpu(net.input_gpu, l.output_gpu, l.batch, l.w, l.h, l.n, l.classes, l.coords, l.background,
                       l.softmax);
}

/* ---- local (yolov1): src/local_layer.c:26-89.  One weight matrix per output location, one bias
 * per output element; the reference's random initial weights are left to the weights file. ----- */
layer make_local_layer(int batch, int h, int w, int c, int n, int size, int stride, int pad, ACTIVATION activation)
{
    layer l;
    long locations, nweights;
    memset(&l, 0, sizeof l);
    l.type = LOCAL;
    l.h = h;
    l.w = w;
    l.c = c;
    l.n = n;
    l.batch = batch;
    l.stride = stride;
    l.size = size;
    l.pad = pad;
    if (size < 1 || stride < 1 || n < 1 || pad < 0) dn_fatal("local layer: bad size, stride, pad or filters");
    if ((pad ? 1 : size) > h || (pad ? 1 : size) > w) dn_fatal("local layer: kernel larger than its input");
    l.out_h = (h - (pad ? 1 : size)) / stride + 1; /* src/local_layer.c:10-24 */
    l.out_w = (w - (pad ? 1 : size)) / stride + 1;
    if ((h + 2 * pad - size) / stride + 1 != l.out_h || (w + 2 * pad - size) / stride + 1 != l.out_w)
        dn_fatal("local layer: pad and size give im2col a different output size than the layer's");
    l.out_c = n;
    l.outputs = l.out_h * l.out_w * l.out_c;
    l.inputs = l.w * l.h * l.c;
    l.activation = activation;
    locations = (long)l.out_h * l.out_w;
    nweights = (long)c * n * size * size * locations;
    if (nweights >= (1L << 31)) dn_fatal("local layer: too many weights");
    l.nweights = (int)nweights;
    l.nbiases = l.outputs;
    l.weights = (float *)dn_calloc((size_t)nweights, sizeof(float));
    l.biases = (float *)dn_calloc((size_t)l.outputs, sizeof(float));
    l.workspace_size = (size_t)l.out_h * l.out_w * size * size * c; /* as src/local_layer.c:63 sets it; unused here */
    l.forward_gpu = forward_local_layer_gpu;
    if (gpu_index < 0) dn_fatal("this library has no CPU path: gpu_index must name a device");
    l.weights_gpu = hip_make_array(l.weights, (size_t)nweights);
    l.biases_gpu = hip_make_array(l.biases, (size_t)l.outputs);
    l.output_gpu = hip_make_array(0, (size_t)batch * l.outputs);
    if (dn_verbose)
        fprintf(stderr, "Local Layer: %d x %d x %d image, %d filters -> %d x %d x %d image\n", h, w, c, n, l.out_h,
                l.out_w, n);
    return l;
}

void forward_local_layer_gpu(layer l, network net)
{
    forward_local_gpu(net.input_gpu, l.weights_gpu, l.biases_gpu, l.output_gpu, l.batch, l.c, l.h, l.w, l.n, l.size,
                      l.stride, l.pad, (int)l.activation);
}

void push_local_layer(layer l)
{
    hip_push_array(l.weights_gpu, l.weights, (size_t)l.nweights);
    hip_push_array(l.biases_gpu, l.biases, (size_t)l.outputs);
}

void pull_local_layer(layer l)
{
    hip_pull_array(l.weights_gpu, l.weights, (size_t)l.nweights);
    hip_pull_array(l.biases_gpu, l.biases, (size_t)l.outputs);
}

/* ---- detection (yolov1 head): src/detection_layer.c:14-48.  At inference the layer is a copy
 * of its input, with a softmax over each cell's class scores when `softmax` is set (:50-66; the
 * reference's GPU forward :256-262 only copies, its CPU forward is followed here). -------------- */
layer make_detection_layer(int batch, int inputs, int n, int side, int classes, int coords, int rescore)
{
    layer l;
    memset(&l, 0, sizeof l);
    l.type = DETECTION;
    l.n = n;
    l.batch = batch;
    l.inputs = inputs;
    l.classes = classes;
    l.coords = coords;
    l.rescore = rescore;
    l.side = side;
    l.w = side;
    l.h = side;
    if (side < 1 || n < 1 || classes < 0 || (long)side * side * ((long)(1 + coords) * n + classes) != inputs)
        dn_fatal("detection layer: the layer before it must output side*side*((1+coords)*num+classes) values");
    l.outputs = l.inputs;
    l.truths = l.side * l.side * (1 + l.coords + l.classes);
    l.output = hip_host_alloc((size_t)batch * l.outputs);
    l.forward_gpu = forward_detection_layer_gpu;
    l.output_gpu = hip_make_array(0, (size_t)batch * l.outputs);
    if (dn_verbose) fprintf(stderr, "Detection Layer\n");
    return l;
}

void forward_detection_layer_gpu(layer l, network net)
{
    copy_gpu(l.batch * l.inputs, net.input_gpu, 1, l.output_gpu, 1);
    if (l.softmax) /* per image and cell, over the classes at the head of the vector */
        softmax_gpu(net.input_gpu, l.classes, l.batch, l.inputs, l.side * l.side, l.classes, 1, 1.f, l.output_gpu);
}

void free_layer(layer l)
{
    if (l.type == DROPOUT) return; /* its buffers belong to the layer before it (src/layer.c:8-14) */
    free(l.mask);
    free(l.input_layers);
    free(l.input_sizes);
    free(l.biases);
    free(l.scales);
    free(l.weights);
    free(l.rolling_mean);
    free(l.rolling_variance);
    hip_host_free(l.output);
    free(l.indexes);
    if (l.indexes_gpu) hip_free((float *)l.indexes_gpu);
    if (l.weights_gpu) hip_free(l.weights_gpu);
    if (l.biases_gpu) hip_free(l.biases_gpu);
    if (l.scales_gpu) hip_free(l.scales_gpu);
    if (l.rolling_mean_gpu) hip_free(l.rolling_mean_gpu);
    if (l.rolling_variance_gpu) hip_free(l.rolling_variance_gpu);
    if (l.output_gpu && !l.output_gpu_is_view) hip_free(l.output_gpu);
    if (l.binary_weights_gpu) hip_free(l.binary_weights_gpu);
    if (l.binary_input_gpu) hip_free(l.binary_input_gpu);
    if (l.weights_packed_gpu) hip_free(l.weights_packed_gpu);
    if (l.xnor_wbits_gpu) hip_free((float *)l.xnor_wbits_gpu);
    if (l.xnor_xbits_gpu) hip_free((float *)l.xnor_xbits_gpu);
    if (l.xnor_wmean_gpu) hip_free(l.xnor_wmean_gpu);
}
