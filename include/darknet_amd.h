/*
 * darknet_amd.h - the layer / network API of the darknet forward path, on top of the device
 * layer in darknet_hip.h.
 *
 * This header mirrors the part of the reference's public header that inference uses
 * (include/darknet.h of pjreddie/darknet): the ACTIVATION and LAYER_TYPE enums in the same
 * order, `layer` and `network` with the reference's field names, the constructors the cfg parser
 * calls, and parse_network_cfg / network_predict / forward_network with their reference
 * signatures.  Both structs are passed BY VALUE to every forward function, as in the
 * reference (include/darknet.h:119-124).  Only the GPU dispatch exists: `forward` (the CPU
 * pointer) is always NULL and forward_network() ends the process if gpu_index < 0 - this library
 * has no CPU path to fall back to.
 *
 * LAYOUT: `layer` and `network` here hold the members inference uses, under the reference's names
 * and types, but NOT at the reference's offsets and not all of them (the reference's structs carry
 * some three hundred training, recurrent and cuDNN members, and their size depends on its GPU /
 * CUDNN macros, include/darknet.h:334-421).  Both structs travel by value through this API, so an
 * object file compiled against the reference's include/darknet.h cannot exchange layer / network
 * objects with this library: a program either compiles against THIS header (same source text:
 * same names, same calls), or keeps the reference's own host files and structs and binds the
 * plain-pointer device layer of darknet_hip.h, whose signatures carry no struct at all.
 *
 * Training-only members (delta, updates, x, x_norm, adam state, cost) are not allocated:
 * inference never reads them and at batch 64 they would triple the footprint.
 *
 * Citations: reference file:line each declaration stands in for.
 */
#ifndef DARKNET_AMD_H
#define DARKNET_AMD_H

#include <stddef.h>
#include <stdio.h>

#include "darknet_hip.h"

#ifdef __cplusplus
extern "C" {
#endif

/* include/darknet.h:48-50 */
typedef enum {
    LOGISTIC, RELU, RELIE, LINEAR, RAMP, TANH, PLSE, LEAKY, ELU, LOGGY, STAIR, HARDTAN, LHTAN, SELU
} ACTIVATION;

/* include/darknet.h:60-91 */
typedef enum {
    CONVOLUTIONAL, DECONVOLUTIONAL, CONNECTED, MAXPOOL, SOFTMAX, DETECTION, DROPOUT, CROP, ROUTE,
    COST, NORMALIZATION, AVGPOOL, LOCAL, SHORTCUT, ACTIVE, RNN, GRU, LSTM, CRNN, BATCHNORM, NETWORK,
    XNOR, REGION, YOLO, ISEG, REORG, UPSAMPLE, LOGXENT, L2NORM, BLANK
} LAYER_TYPE;

struct network;
typedef struct network network;
struct layer;
typedef struct layer layer;

/* include/darknet.h:115-422, inference subset */
struct layer {
    LAYER_TYPE type;
    ACTIVATION activation;
    void (*forward)(struct layer, struct network);     /* always NULL here */
    void (*forward_gpu)(struct layer, struct network);
    int batch_normalize;
    int batch;
    int flipped;
    int inputs;
    int outputs;
    int nweights;
    int nbiases;
    int truths;
    int h, w, c;
    int out_h, out_w, out_c;
    int n;
    int max_boxes;
    int groups;
    int size;
    int stride;
    int reverse;
    int pad;
    int index;
    int binary;
    int xnor;
    int truth;
    int classes;
    int total;
    int noloss;
    int dontload;
    int dontloadscales;
    int numload;
    int onlyforward;
    int *mask;
    float alpha;
    float beta;
    float scale;
    float temperature;
    float jitter;
    float ignore_thresh;
    float truth_thresh;
    int random;
    int coords;        /* region, detection */
    int background;
    int softmax;
    int side;          /* detection */
    int sqrt;
    int rescore;
    int flatten;       /* reorg */
    int extra;
    int noadjust;      /* crop */
    int flip;
    float probability; /* dropout */
    float shift;

    int *input_layers;
    int *input_sizes;

    /* host copies: parameters always; output only where the host reads it (yolo heads and the
     * last layer), see layer_output_host() for the rest */
    float *biases;
    float *scales;
    float *weights;
    float *rolling_mean;
    float *rolling_variance;
    float *output;
    int *indexes;

    size_t workspace_size;

    /* device buffers (include/darknet.h:334-421) */
    int *indexes_gpu;
    float *weights_gpu;
    float *biases_gpu;
    float *scales_gpu;
    float *rolling_mean_gpu;
    float *rolling_variance_gpu;
    float *output_gpu;
    float *binary_weights_gpu;
    float *binary_input_gpu;

    /* additions of this library */
    float *weights_packed_gpu; /* MFMA layout of weights_gpu; refreshed by push_convolutional_layer */
    int output_gpu_is_view;    /* output_gpu belongs to another layer (a one-source route): free_layer leaves it */
    unsigned *xnor_wbits_gpu;  /* xnor layers: packed sign(w), packed sign(x), mean|w| per filter */
    unsigned *xnor_xbits_gpu;
    float *xnor_wmean_gpu;
};

/* include/darknet.h:430-496, inference subset */
typedef struct network {
    int n;
    int batch;
    size_t *seen;
    int subdivisions;
    layer *layers;
    float *output;
    int time_steps;
    int inputs;
    int outputs;
    int truths;
    int h, w, c;
    int gpu_index;
    float *input;
    float *truth;
    float *delta;
    float *workspace;
    int train;
    int index;
    float *input_gpu;
    float *truth_gpu;
    float *delta_gpu;
    float *output_gpu;

    /* additions of this library: device row buffer of the detection decode; the batch the buffers
     * were allocated for (set_batch_network may go down and come back up to it) */
    float *det_rows_gpu;
    int *det_count_gpu;
    int det_max_rows;
    int max_batch;
    void *pipeline;   /* state of network_predict_submit / _collect, made on first use */
} network;

/* include/darknet.h:515-526 */
typedef struct {
    float x, y, w, h;
} box;

typedef struct detection {
    box bbox;
    int classes;
    float *prob;
    float *mask;
    float objectness;
    int sort_class;
} detection;

/* ---- cfg parsing (src/parser.c:742-889; list/option helpers src/list.c, src/option_list.c) */
network *parse_network_cfg(char *filename);
network *load_network(char *cfg, char *weights, int clear);          /* src/network.c:53-63 */
void load_weights(network *net, char *filename);                      /* src/parser.c:1308 */
void load_weights_upto(network *net, char *filename, int start, int cutoff); /* src/parser.c:1218 */
void save_weights(network *net, char *filename);                      /* src/parser.c:1081 */
void save_weights_upto(network *net, char *filename, int cutoff);     /* src/parser.c:1007 */
ACTIVATION get_activation(char *s);                                   /* src/activations.c:44 */
char *get_activation_string(ACTIVATION a);                            /* src/activations.c:8 */
char *get_layer_string(LAYER_TYPE a);                                 /* src/network.c:110 */

/* ---- layer constructors, reference signatures -------------------------------------------- */
layer make_convolutional_layer(int batch, int h, int w, int c, int n, int groups, int size,
                               int stride, int padding, ACTIVATION activation,
                               int batch_normalize, int binary, int xnor,
                               int adam);                 /* src/convolutional_layer.c:176 */
layer make_maxpool_layer(int batch, int h, int w, int c, int size, int stride,
                         int padding);                    /* src/maxpool_layer.c:21 */
layer make_route_layer(int batch, int n, int *input_layers, int *input_sizes); /* src/route_layer.c:7 */
layer make_shortcut_layer(int batch, int index, int w, int h, int c, int w2, int h2,
                          int c2);                        /* src/shortcut_layer.c:9 */
layer make_upsample_layer(int batch, int w, int h, int c, int stride); /* src/upsample_layer.c:7 */
layer make_yolo_layer(int batch, int w, int h, int n, int total, int *mask,
                      int classes);                       /* src/yolo_layer.c:13 */
layer make_avgpool_layer(int batch, int w, int h, int c); /* src/avgpool_layer.c:5 */
layer make_connected_layer(int batch, int inputs, int outputs, ACTIVATION activation,
                           int batch_normalize, int adam); /* src/connected_layer.c:14 */
layer make_dropout_layer(int batch, int inputs, float probability); /* src/dropout_layer.c:7 */
layer make_batchnorm_layer(int batch, int w, int h, int c);          /* src/batchnorm_layer.c:6 */
layer make_reorg_layer(int batch, int w, int h, int c, int stride, int reverse, int flatten,
                       int extra);                        /* src/reorg_layer.c:8 */
layer make_crop_layer(int batch, int h, int w, int c, int crop_height, int crop_width, int flip,
                      float angle, float saturation, float exposure); /* src/crop_layer.c:18 */
layer make_cost_layer(int batch, int inputs, int cost_type, float scale); /* src/cost_layer.c:40 */
layer make_region_layer(int batch, int w, int h, int n, int classes, int coords); /* src/region_layer.c:13 */
layer make_softmax_layer(int batch, int inputs, int groups); /* src/softmax_layer.c:11 */
layer make_local_layer(int batch, int h, int w, int c, int n, int size, int stride, int pad,
                       ACTIVATION activation);                 /* src/local_layer.c:26 */
layer make_detection_layer(int batch, int inputs, int n, int side, int classes, int coords,
                           int rescore);                       /* src/detection_layer.c:14 */
void free_layer(layer l);                                 /* src/layer.c:6 */

/* ---- per-layer GPU forwards, the function-pointer targets (include/darknet.h:122) -------- */
void forward_convolutional_layer_gpu(layer l, network net); /* src/convolutional_kernels.cu:73 */
void forward_maxpool_layer_gpu(layer l, network net);       /* src/maxpool_layer_kernels.cu:87 */
void forward_route_layer_gpu(layer l, network net);         /* src/route_layer.c:105 */
void forward_shortcut_layer_gpu(layer l, network net);      /* src/shortcut_layer.c:77 */
void forward_upsample_layer_gpu(layer l, network net);      /* src/upsample_layer.c:88 */
void forward_yolo_layer_gpu(layer l, network net);          /* src/yolo_layer.c:347 */
void forward_avgpool_layer_gpu(layer l, network net);       /* src/avgpool_layer_kernels.cu:46 */
void forward_softmax_layer_gpu(layer l, network net);       /* src/softmax_layer.c:71 */
void forward_connected_layer_gpu(layer l, network net);     /* src/connected_layer.c:286 */
void forward_dropout_layer_gpu(layer l, network net);       /* src/dropout_layer_kernels.cu:17 (inference: nothing) */
void forward_batchnorm_layer_gpu(layer l, network net);     /* src/batchnorm_layer.c:189 (src/batchnorm_layer.h:13; inference branch) */
void push_batchnorm_layer(layer l);                         /* src/batchnorm_layer.c:182 (src/batchnorm_layer.h:16) */
void pull_batchnorm_layer(layer l);                         /* src/batchnorm_layer.c:176 (src/batchnorm_layer.h:15) */
void forward_reorg_layer_gpu(layer l, network net);         /* src/reorg_layer.c:149 */
void forward_crop_layer_gpu(layer l, network net);          /* src/crop_layer_kernels.cu:183 */
void forward_cost_layer_gpu(layer l, network net);          /* src/cost_layer.c:120 (no truth: nothing) */
void forward_region_layer_gpu(layer l, network net);        /* src/region_layer.c:439 */
void forward_local_layer_gpu(layer l, network net);         /* src/local_layer.c:186 */
void forward_detection_layer_gpu(layer l, network net);     /* src/detection_layer.c:256 (inference) */
void push_local_layer(layer l);                             /* src/local_layer.c:286 */
void pull_local_layer(layer l);                             /* src/local_layer.c:278 */
void push_connected_layer(layer l);                         /* src/connected_layer.c:268 */
void pull_connected_layer(layer l);                         /* src/connected_layer.c:254 */
void push_convolutional_layer(layer l);                     /* src/convolutional_kernels.cu:286 */
void pull_convolutional_layer(layer l);                     /* src/convolutional_kernels.cu:270 */

/* ---- network runtime ---------------------------------------------------------------------- */
network *make_network(int n);                               /* src/network.c:177 */
void free_network(network *net);                            /* src/network.c:699 */
void forward_network(network *net);                         /* src/network.c:188 */
void forward_network_gpu(network *net);                     /* src/network.c:762 */
float *network_predict(network *net, float *input);         /* src/network.c:497 */
void set_batch_network(network *net, int b);                /* src/network.c:339 (1 .. the batch the cfg was parsed with) */
layer get_network_output_layer(network *net);               /* src/network.c:689 */
float *network_output(network *net);                        /* src/network.c:755 */
void pull_network_output(network *net);                     /* src/network.c:1123 */
int network_width(network *net);                            /* src/network.c:674 */
int network_height(network *net);                           /* src/network.c:675 */

/* network_predict in two halves (no counterpart in the reference, whose network_predict uploads,
 * computes and downloads one after the other, src/network.c:497-508, :766, :786, src/yolo_layer.c:360).
 * Up to two batches are in flight: while batch n computes, the input of batch n+1 is uploaded and the
 * outputs of batch n-1 are downloaded on two copy streams of their own.
 *   network_predict_submit   takes `input` (net->inputs * net->batch floats; copied before the call
 *                            returns unless it lies in hip_host_alloc memory, which must then stay
 *                            untouched until that batch is collected) and queues upload, forward
 *                            and download; ends the process if two batches are already in flight
 *   network_predict_collect  waits for the oldest batch in flight and returns the host copy of the
 *                            output layer, what network_predict returns, same bits
 *   network_collected_output the host copy of layer i (a yolo head or the output layer) of the
 *                            batch collected last
 * The pointers stay valid until the next network_predict_submit.  Between a submit and its collect
 * the device buffers of the network belong to the pipeline: no network_predict, set_batch_network or
 * detection call on the same network in between.  One host thread per network, as everywhere. */
void network_predict_submit(network *net, float *input);
float *network_predict_collect(network *net);
float *network_collected_output(network *net, int i);
int network_predict_in_flight(network *net);

/* ---- input side: include/darknet.h:508-513 and src/image.c / src/network.c:579 ------------- */
typedef struct {
    int w;
    int h;
    int c;
    float *data;
} image;
image make_image(int w, int h, int c);                     /* src/image.c:743 */
image make_empty_image(int w, int h, int c);               /* src/image.c:734 */
void free_image(image m);                                  /* src/image.c:1368 */
image resize_image(image im, int w, int h);                /* src/image.c:1199 */
image letterbox_image(image im, int w, int h);             /* src/image.c:812 */
float *network_predict_image(network *net, image im);      /* src/network.c:579 */
/* additions: letterbox `im` straight into image slot b of the device input (one upload of the
 * frame at its own size through a pinned staging buffer, no host-side resize); and the host
 * pulls network_predict ends with (yolo heads + output layer) on their own */
void network_letterbox_input(network *net, int b, image im);
void network_pull_outputs(network *net);

/* ---- detections (yolo, region and yolov1 detection heads) ---- */
int num_detections(network *net, float thresh);                       /* src/network.c:510 */
detection *make_network_boxes(network *net, float thresh, int *num);  /* src/network.c:526 */
void fill_network_boxes(network *net, int w, int h, float thresh, float hier, int *map, int relative,
                        detection *dets);                             /* src/network.c:543 */
detection *get_network_boxes(network *net, int w, int h, float thresh, float hier, int *map,
                             int relative, int *num);                 /* src/network.c:563 */
void free_detections(detection *dets, int n);                         /* src/network.c:570 */
void do_nms_sort(detection *dets, int total, int classes, float thresh); /* src/box.c:58 */
/* additions: the same for image b of the batch (the reference reads image 0 only), with the
 * suppression done on the device before the rows are copied back when nms > 0; and the decode
 * alone, leaving the rows in net->det_rows_gpu and returning their number */
detection *get_network_boxes_image(network *net, int b, int w, int h, float thresh, int relative,
                                   float nms, int *num);
int network_decode_image_gpu(network *net, int b, int w, int h, float thresh, int relative);

/* ---- additions (no reference twin) --------------------------------------------------------
 * forward_network_device: the layer loop alone, on whatever net->input_gpu holds; no host<->
 * device copies, returns without synchronising.  This is what the benchmark times.
 * layer_output_host: pulls layer i's output into a host buffer owned by the layer.
 * network_set_verbose: 0 silences the per-layer table the constructors print to stderr. */
void forward_network_device(network *net);
/* forward_network_device with a HIP event after every layer: fills layer_ms[net->n] (may be
 * NULL) and returns the whole pass in milliseconds; synchronises before returning. */
float forward_network_profiled(network *net, float *layer_ms);
/* the same, plus kernel_ms[net->n]: the duration of each convolutional / connected layer's main
 * kernel alone, from events attached to its dispatch (-1 where there is none) */
float forward_network_profiled_kernels(network *net, float *layer_ms, float *kernel_ms);
/* 1 (default): forward_network_device runs a convolution and the same-geometry shortcut right
 * after it as one pass (forward_convolutional_shortcut_gpu), likewise a convolution and the yolo
 * head it feeds (forward_convolutional_yolo_gpu), a first layer or an xnor convolution and the 2x2
 * stride-2 maxpool behind it (forward_convolutional_maxpool_gpu, forward_convolutional_xnor_fused_gpu),
 * and the layer in front of an xnor convolution writes the sign bits that convolution reads;
 * 0: layer by layer as src/network.c:773-785 does.  Every layer's output buffer is written in both
 * modes and holds the same bits.
 * 2 (lean): as 1, except that the map of a convolution which nothing but the maxpool fused behind
 * it reads is not written: its output buffer is stale, layer_output_host() refuses it. */
void network_set_fusion(int on);
/* At the present fusion level: whether layer i runs inside the kernel of the convolution in front
 * of it (no launch of its own), and whether layer i's own output is left unwritten (lean mode). */
int network_layer_runs_fused(network *net, int i);
int network_layer_output_skipped(network *net, int i);
float *layer_output_host(network *net, int i);
int *layer_indexes_host(network *net, int i);
void network_set_verbose(int on);
/* Overwrites layer i's parameters (host and device copies); NULL leaves a vector as it is.
 * Convolutional: weights[nweights], biases/scales/mean/variance[n]; connected: the same with
 * n = outputs; local: weights[nweights], biases[outputs] (the other three are ignored); batchnorm:
 * biases/scales/mean/variance[c] (weights ignored). */
void network_set_conv(network *net, int i, const float *weights, const float *biases,
                      const float *scales, const float *rolling_mean,
                      const float *rolling_variance);
/* Flat read-out of a layer for FFI callers that do not mirror the struct: iv receives
 * type, batch, h, w, c, out_h, out_w, out_c, n, size, stride, pad, groups, batch_normalize,
 * activation, binary, xnor, index, inputs, outputs, nweights, classes, total, reverse,
 * workspace_floats, nbiases, truths, max_boxes (28 ints); fv alpha, beta, scale, temperature. */
void network_layer_info(network *net, int i, int *iv, float *fv);
int network_route_inputs(network *net, int i, int *layers, int *sizes, int cap);
int network_num_layers(network *net);
float *network_input_gpu(network *net); /* device buffer forward_network_device reads */
void network_info(network *net, int *iv); /* n, batch, h, w, c, inputs, outputs */
double network_conv_flops(network *net);   /* per image, the reference's count (examples/darknet.c:88) */

#ifdef __cplusplus
}
#endif
#endif
