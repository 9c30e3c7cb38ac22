/*
 * Test infrastructure only.  A thin driver around the *compiled reference* (CPU build of
 * pjreddie/darknet, linked from oracle/_ref/libdarknet_ref*.so).  It is compiled against the
 * reference's own public header, found through -I at build time, so the struct layouts are the
 * reference's; nothing from the reference is copied here.  It flattens what the tests need out
 * of `network` / `layer` (include/darknet.h:115-422, :430-496 of the reference) into plain int
 * and float arrays so Python can read them without mirroring those structs.
 */
#include "darknet.h"
#include <string.h>

/* Built a second time with -DGPU against the reference tree as bound to the HIP library
 * (oracle/Makefile, target ref_hip): the same calls then drive the reference's own
 * parse_network_cfg / network_predict / forward_network_gpu over the adapters, parameters are
 * pushed to the device after they are written and layer outputs are pulled before they are read. */
#ifdef GPU
#include "convolutional_layer.h"
#include "batchnorm_layer.h"
void refh_set_gpu(int n) { cuda_set_device(n); }
int refh_is_gpu_build(void) { return 1; }
#else
int refh_is_gpu_build(void) { return 0; }
#endif

enum { REFH_NI = 28, REFH_NF = 4 };

network *refh_load(char *cfg)
{
    return parse_network_cfg(cfg);
}

void refh_free(network *net)
{
    free_network(net);
}

int refh_nlayers(network *net) { return net->n; }

void refh_net_info(network *net, int *iv)
{
    iv[0] = net->n;
    iv[1] = net->batch;
    iv[2] = net->h;
    iv[3] = net->w;
    iv[4] = net->c;
    iv[5] = net->inputs;
    iv[6] = net->outputs;
    iv[7] = (int)(net->layers[net->n - 1].type);
}

void refh_layer_info(network *net, int i, int *iv, float *fv)
{
    layer l = net->layers[i];
    int k = 0;
    iv[k++] = (int)l.type;          /* 0 */
    iv[k++] = l.batch;              /* 1 */
    iv[k++] = l.h;                  /* 2 */
    iv[k++] = l.w;                  /* 3 */
    iv[k++] = l.c;                  /* 4 */
    iv[k++] = l.out_h;              /* 5 */
    iv[k++] = l.out_w;              /* 6 */
    iv[k++] = l.out_c;              /* 7 */
    iv[k++] = l.n;                  /* 8 */
    iv[k++] = l.size;               /* 9 */
    iv[k++] = l.stride;             /* 10 */
    iv[k++] = l.pad;                /* 11 */
    iv[k++] = l.groups;             /* 12 */
    iv[k++] = l.batch_normalize;    /* 13 */
    iv[k++] = (int)l.activation;    /* 14 */
    iv[k++] = l.binary;             /* 15 */
    iv[k++] = l.xnor;               /* 16 */
    iv[k++] = l.index;              /* 17 */
    iv[k++] = l.inputs;             /* 18 */
    iv[k++] = l.outputs;            /* 19 */
    iv[k++] = l.nweights;           /* 20 */
    iv[k++] = l.classes;            /* 21 */
    iv[k++] = l.total;              /* 22 */
    iv[k++] = l.reverse;            /* 23 */
    iv[k++] = (int)(l.workspace_size / sizeof(float)); /* 24 */
    iv[k++] = l.nbiases;            /* 25 */
    iv[k++] = l.truths;             /* 26 */
    iv[k++] = l.max_boxes;          /* 27 */
    fv[0] = l.alpha;
    fv[1] = l.beta;
    fv[2] = l.scale;
    fv[3] = l.temperature;
}

int refh_route_inputs(network *net, int i, int *layers, int *sizes, int cap)
{
    layer l = net->layers[i];
    int j;
    for (j = 0; j < l.n && j < cap; ++j) {
        layers[j] = l.input_layers[j];
        sizes[j] = l.input_sizes[j];
    }
    return l.n;
}

int refh_yolo_mask(network *net, int i, int *mask, int cap, float *anchors, int acap)
{
    layer l = net->layers[i];
    int j;
    for (j = 0; j < l.n && j < cap; ++j) mask[j] = l.mask[j];
    for (j = 0; j < 2 * l.total && j < acap; ++j) anchors[j] = l.biases[j];
    return l.n;
}

/* Overwrite a convolutional layer's parameters; NULL leaves a vector as it is. */
void refh_set_conv(network *net, int i, const float *weights, const float *biases,
                   const float *scales, const float *mean, const float *variance)
{
    layer l = net->layers[i];
    if (weights) memcpy(l.weights, weights, sizeof(float) * (size_t)l.nweights);
    if (biases) memcpy(l.biases, biases, sizeof(float) * (size_t)l.n);
    if (l.batch_normalize) {
        if (scales) memcpy(l.scales, scales, sizeof(float) * (size_t)l.n);
        if (mean) memcpy(l.rolling_mean, mean, sizeof(float) * (size_t)l.n);
        if (variance) memcpy(l.rolling_variance, variance, sizeof(float) * (size_t)l.n);
    }
#ifdef GPU
    push_convolutional_layer(l);
#endif
}

/* The same for a [batchnorm] layer: c values per vector, no weights (src/batchnorm_layer.c:20-33). */
void refh_set_batchnorm(network *net, int i, const float *biases, const float *scales, const float *mean,
                        const float *variance)
{
    layer l = net->layers[i];
    if (biases) memcpy(l.biases, biases, sizeof(float) * (size_t)l.c);
    if (scales) memcpy(l.scales, scales, sizeof(float) * (size_t)l.c);
    if (mean) memcpy(l.rolling_mean, mean, sizeof(float) * (size_t)l.c);
    if (variance) memcpy(l.rolling_variance, variance, sizeof(float) * (size_t)l.c);
#ifdef GPU
    push_batchnorm_layer(l);
#endif
}

/* The same for a connected layer (its parameter vectors are sized by outputs / inputs). */
void refh_set_connected(network *net, int i, const float *weights, const float *biases,
                        const float *scales, const float *mean, const float *variance)
{
    layer l = net->layers[i];
    if (weights) memcpy(l.weights, weights, sizeof(float) * (size_t)l.inputs * l.outputs);
    if (biases) memcpy(l.biases, biases, sizeof(float) * (size_t)l.outputs);
    if (l.batch_normalize) {
        if (scales) memcpy(l.scales, scales, sizeof(float) * (size_t)l.outputs);
        if (mean) memcpy(l.rolling_mean, mean, sizeof(float) * (size_t)l.outputs);
        if (variance) memcpy(l.rolling_variance, variance, sizeof(float) * (size_t)l.outputs);
    }
}

/* The same for a local layer: weights[locations*n*size*size*c], biases[outputs]
 * (src/local_layer.c:48-52; the layer does not fill in nweights). */
void refh_set_local(network *net, int i, const float *weights, const float *biases)
{
    layer l = net->layers[i];
    size_t nw = (size_t)l.c * l.n * l.size * l.size * l.out_h * l.out_w;
    if (weights) memcpy(l.weights, weights, sizeof(float) * nw);
    if (biases) memcpy(l.biases, biases, sizeof(float) * (size_t)l.outputs);
}

float *refh_predict(network *net, float *input)
{
    return network_predict(net, input);
}

float *refh_layer_output(network *net, int i)
{
    layer l = net->layers[i];
#ifdef GPU
    if (l.output_gpu && l.output) cuda_pull_array(l.output_gpu, l.output, (size_t)l.outputs * l.batch);
#endif
    return l.output;
}

int *refh_layer_indexes(network *net, int i)
{
    layer l = net->layers[i];
#ifdef GPU
    if (l.indexes_gpu && l.indexes) hip_pull_int_array(l.indexes_gpu, l.indexes, (size_t)l.outputs * l.batch);
#endif
    return l.indexes;
}
float *refh_layer_weights(network *net, int i) { return net->layers[i].weights; }
float *refh_layer_binary_weights(network *net, int i) { return net->layers[i].binary_weights; }
float *refh_layer_binary_input(network *net, int i) { return net->layers[i].binary_input; }

/* Run one layer's CPU forward on a caller-supplied input (used to inject an input into a
 * single XNOR layer, where end-to-end comparison is ill-posed). */
void refh_forward_layer(network *net, int i, float *input)
{
    network copy = *net;
    layer l = net->layers[i];
    copy.input = input;
    copy.train = 0;
    copy.truth = 0;
    copy.index = i;
    l.forward(l, copy);
}

/* get_network_boxes (src/network.c:563) on the outputs of the last refh_predict, optionally
 * followed by do_nms_sort (src/box.c:58), flattened to rows of 5 + classes floats:
 * x, y, w, h, objectness, prob[classes].  Returns the number of detections (rows beyond `cap`
 * are not written).  The reference leaves the array sorted by the last class after NMS; callers
 * compare order-free. */
int refh_get_boxes(network *net, int w, int h, float thresh, int relative, float nms, float *rows, int cap)
{
    int n = 0, i, j;
    layer l = net->layers[net->n - 1];
    detection *dets = get_network_boxes(net, w, h, thresh, .5f, 0, relative, &n);
    if (nms > 0) do_nms_sort(dets, n, l.classes, nms);
    for (i = 0; i < n && i < cap; ++i) {
        float *r = rows + (size_t)i * (5 + l.classes);
        r[0] = dets[i].bbox.x;
        r[1] = dets[i].bbox.y;
        r[2] = dets[i].bbox.w;
        r[3] = dets[i].bbox.h;
        r[4] = dets[i].objectness;
        for (j = 0; j < l.classes; ++j) r[5 + j] = dets[i].prob[j];
    }
    free_detections(dets, n);
    return n;
}

/* Overwrite a yolo layer's host output (so that decode and NMS can be driven with chosen
 * tensors without running a network that produces them). */
void refh_set_output(network *net, int i, const float *values)
{
    layer l = net->layers[i];
    memcpy(l.output, values, sizeof(float) * (size_t)l.outputs * l.batch);
}

/* resize_image / letterbox_image (src/image.c:1199, :812) on a caller's [c][h][w] array */
void refh_resize_image(float *data, int w, int h, int c, int ow, int oh, float *out)
{
    image im = {w, h, c, data};
    image r = resize_image(im, ow, oh);
    memcpy(out, r.data, sizeof(float) * (size_t)ow * oh * c);
    free_image(r);
}

void refh_letterbox_image(float *data, int w, int h, int c, int bw, int bh, float *out)
{
    image im = {w, h, c, data};
    image r = letterbox_image(im, bw, bh);
    memcpy(out, r.data, sizeof(float) * (size_t)bw * bh * c);
    free_image(r);
}

