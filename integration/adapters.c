/*
 * adapters.c - what a pjreddie/darknet tree adds to run its inference forward pass on
 * libdarknet_hip.so while keeping its own host files, structs and driver loop.
 *
 * It is compiled INSIDE that tree (against the tree's include/darknet.h and src/ headers, with -DGPU)
 * and takes the place of the host functions that lived in the tree's CUDA translation units:
 *
 *   src/convolutional_kernels.cu:73-135   forward_convolutional_layer_gpu
 *   src/convolutional_kernels.cu:273-297  pull_convolutional_layer, push_convolutional_layer
 *   src/maxpool_layer_kernels.cu:87-97    forward_maxpool_layer_gpu
 *   src/avgpool_layer_kernels.cu:46-52    forward_avgpool_layer_gpu
 *   src/crop_layer_kernels.cu:183-204     forward_crop_layer_gpu (inference)
 *   src/dropout_layer_kernels.cu:17-31    forward_dropout_layer_gpu (inference: nothing)
 *
 * Every other forward_*_layer_gpu of the tree (route, shortcut, upsample, yolo, region, reorg,
 * softmax, batchnorm, cost, detection: they live in .c files) stays as it is and reaches the device
 * through the helpers the library exports under the tree's own names (fill_gpu, copy_gpu,
 * activate_array_gpu, shortcut_gpu, upsample_gpu, softmax_gpu, normalize_gpu, scale_bias_gpu,
 * add_bias_gpu, reorg_gpu, flatten_gpu, cuda_*).
 *
 * The by-value `layer` / `network` of the tree are only spelled out into pointers and sizes here.
 * The tree's `layer` has no member for the MFMA-packed weights, so the copy is kept by the
 * library, keyed by the address of weights_gpu (conv_packed_cached_gpu); the scratch of an xnor
 * layer is kept in a small table below, keyed the same way.
 *
 * Device symbols that only training reaches (backward_*, update_*, the BLAS-1 and loss kernels,
 * gemm_gpu) are in training_stubs.c.
 */
#include "darknet.h"
#include "cuda.h"
#include "convolutional_layer.h"
#include "maxpool_layer.h"
#include "avgpool_layer.h"
#include "crop_layer.h"
#include "dropout_layer.h"

#include <stdio.h>
#include <stdlib.h>

static void adapters_fatal(const char *what)
{
    fprintf(stderr, "darknet-hip adapters: %s\n", what);
    exit(-1);
}

/* ---- scratch of xnor layers ------------------------------------------------------------------
 * Sign bits of the weights and of the current input, and mean|w| per filter.  All of it is
 * rewritten by every forward, so an entry can never be stale; it is re-made when a layer of
 * another geometry turns up at the same weights address. */
typedef struct {
    const float *weights;
    unsigned *wbits, *xbits;
    float *wmean;
    size_t wwords, xwords;
    int n;
} xnor_scratch;

static xnor_scratch *xnor_table = 0;
static int xnor_count = 0, xnor_cap = 0;

static xnor_scratch *xnor_scratch_for(layer l)
{
    const size_t wwords = xnor_weight_words(l.n, l.c, l.size);
    const size_t xwords = xnor_input_words(l.batch, l.c, l.h, l.w);
    xnor_scratch *s = 0;
    int i;
    for (i = 0; i < xnor_count; ++i)
        if (xnor_table[i].weights == l.weights_gpu) s = &xnor_table[i];
    if (s && s->wwords == wwords && s->xwords >= xwords && s->n == l.n) return s;
    if (s) {
        cuda_free((float *)s->wbits);
        cuda_free((float *)s->xbits);
        cuda_free(s->wmean);
    } else {
        if (xnor_count == xnor_cap) {
            xnor_cap = xnor_cap ? 2 * xnor_cap : 32;
            xnor_table = realloc(xnor_table, sizeof(*xnor_table) * (size_t)xnor_cap);
            if (!xnor_table) adapters_fatal("out of host memory");
        }
        s = &xnor_table[xnor_count++];
    }
    s->weights = l.weights_gpu;
    s->wwords = wwords;
    s->xwords = xwords;
    s->n = l.n;
    s->wbits = (unsigned *)cuda_make_int_array(0, wwords);
    s->xbits = (unsigned *)cuda_make_int_array(0, xwords);
    s->wmean = cuda_make_array(0, (size_t)l.n);
    return s;
}

/* ---- convolution ------------------------------------------------------------------------------
 * One call instead of fill_gpu + (im2col_gpu + gemm_gpu) per image and group + the batch-norm /
 * bias / activation passes.  Results follow the tree's CPU forward (src/convolutional_layer.c:445-485):
 * `binary` alone changes nothing there (only `xnor` binarises, :451-456), and so here. */
void forward_convolutional_layer_gpu(convolutional_layer l, network net)
{
    if (net.train) adapters_fatal("forward_convolutional_layer_gpu: training is not served (net.train != 0)");
    if (l.xnor) {
        xnor_scratch *s;
        if (l.groups != 1) adapters_fatal("forward_convolutional_layer_gpu: xnor with groups is not served");
        s = xnor_scratch_for(l);
        forward_convolutional_xnor_gpu(net.input_gpu, l.weights_gpu, s->wbits, s->wmean, s->xbits, l.biases_gpu,
                                       l.scales_gpu, l.rolling_mean_gpu, l.rolling_variance_gpu, l.output_gpu,
                                       l.batch, l.c, l.h, l.w, l.n, l.size, l.stride, l.pad, l.batch_normalize,
                                       (int)l.activation);
        return;
    }
    forward_convolutional_gpu(net.input_gpu, l.weights_gpu,
                              conv_packed_cached_gpu(l.weights_gpu, l.n, l.c, l.groups, l.size), l.biases_gpu,
                              l.scales_gpu, l.rolling_mean_gpu, l.rolling_variance_gpu, l.output_gpu, l.batch,
                              l.c, l.h, l.w, l.n, l.groups, l.size, l.stride, l.pad, l.batch_normalize,
                              (int)l.activation);
}

/* The tree calls this at the end of load_convolutional_weights (src/parser.c:1210-1214) and from
 * its weight-sharing code; cuda_push_array on weights_gpu already drops the library's packed copy
 * of them, so the next forward repacks. */
void push_convolutional_layer(convolutional_layer l)
{
    cuda_push_array(l.weights_gpu, l.weights, l.nweights);
    cuda_push_array(l.biases_gpu, l.biases, l.n);
    if (l.weight_updates_gpu) cuda_push_array(l.weight_updates_gpu, l.weight_updates, l.nweights);
    if (l.bias_updates_gpu) cuda_push_array(l.bias_updates_gpu, l.bias_updates, l.n);
    if (l.batch_normalize) {
        cuda_push_array(l.scales_gpu, l.scales, l.n);
        cuda_push_array(l.rolling_mean_gpu, l.rolling_mean, l.n);
        cuda_push_array(l.rolling_variance_gpu, l.rolling_variance, l.n);
    }
}

void pull_convolutional_layer(convolutional_layer l)
{
    cuda_pull_array(l.weights_gpu, l.weights, l.nweights);
    cuda_pull_array(l.biases_gpu, l.biases, l.n);
    if (l.weight_updates_gpu) cuda_pull_array(l.weight_updates_gpu, l.weight_updates, l.nweights);
    if (l.bias_updates_gpu) cuda_pull_array(l.bias_updates_gpu, l.bias_updates, l.n);
    if (l.batch_normalize) {
        cuda_pull_array(l.scales_gpu, l.scales, l.n);
        cuda_pull_array(l.rolling_mean_gpu, l.rolling_mean, l.n);
        cuda_pull_array(l.rolling_variance_gpu, l.rolling_variance, l.n);
    }
}

/* ---- pooling ------------------------------------------------------------------------------- */
void forward_maxpool_layer_gpu(maxpool_layer l, network net)
{
    forward_maxpool_gpu(net.input_gpu, l.output_gpu, l.indexes_gpu, l.batch, l.c, l.h, l.w, l.size, l.stride,
                        l.pad);
}

void forward_avgpool_layer_gpu(avgpool_layer l, network net)
{
    forward_avgpool_gpu(net.input_gpu, l.output_gpu, l.batch, l.c, l.h, l.w);
}

/* ---- crop, dropout: inference only --------------------------------------------------------- */
void forward_crop_layer_gpu(crop_layer l, network net)
{
    if (net.train) adapters_fatal("forward_crop_layer_gpu: training-time augmentation is not served");
    forward_crop_gpu(net.input_gpu, l.output_gpu, l.batch, l.c, l.h, l.w, l.out_h, l.out_w, l.noadjust);
}

void forward_dropout_layer_gpu(dropout_layer l, network net)
{
    (void)l;
    if (net.train) adapters_fatal("forward_dropout_layer_gpu: training is not served");
}
