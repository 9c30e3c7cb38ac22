/*
 * weights_io.c - darknet `.weights` files for the layer types on the inference path.
 *
 * Format (src/parser.c:1007-1079 save_weights_upto, :1218-1306 load_weights_upto): three ints
 * major, minor, revision; then `seen` as size_t when major*10+minor >= 2 (and both < 1000),
 * else as int; then, per layer in order, for a convolutional layer: biases[n]; if
 * batch_normalize (and not dontloadscales) scales[n], rolling_mean[n], rolling_variance[n];
 * weights[nweights] (src/parser.c:958-977, :1164-1215); for a connected layer: biases[outputs],
 * weights[outputs*inputs], then the batch-norm vectors (:991-1005, :1098-1120); for a local
 * layer: biases[outputs], weights[locations*n*size*size*c] (:1066-1077, :1292-1302).  Other layer
 * types on this path carry no parameters.  A load ends in push_convolutional_layer, which also refreshes the packed copy
 * the MFMA kernel reads.
 */
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include "host.h"

static void file_error(const char *s)
{
    fprintf(stderr, "Couldn't open file: %s\n", s);
    exit(0);
}

static void read_floats(float *dst, size_t n, FILE *fp, const char *what)
{
    if (fread(dst, sizeof(float), n, fp) != n) {
        char buf[160];
        snprintf(buf, sizeof buf, "weights file ends inside %s", what);
        dn_fatal(buf);
    }
}

/* In-place transpose of a rows x cols matrix (src/parser.c:1110-1122), used by `flipped`. */
static void transpose_matrix(float *a, int rows, int cols)
{
    float *t = (float *)dn_calloc((size_t)rows * cols, sizeof(float));
    int x, y;
    for (x = 0; x < rows; ++x)
        for (y = 0; y < cols; ++y) t[y * rows + x] = a[x * cols + y];
    memcpy(a, t, sizeof(float) * (size_t)rows * cols);
    free(t);
}

static void load_convolutional_weights(layer l, FILE *fp)
{
    /* numload: the file holds only the first `numload` filters (src/parser.c:1166).  The reference
     * shrinks its by-value copy's n for the whole function; here only the reads and the transpose
     * see the smaller count, the push runs on the layer as built, whose packed copy is laid out for
     * all n filters. */
    const int n = l.numload ? l.numload : l.n;
    const int num = l.c / l.groups * n * l.size * l.size;
    if (n < 0 || n > l.n) dn_fatal("convolutional layer: numload exceeds the number of filters");
    read_floats(l.biases, (size_t)n, fp, "convolutional biases");
    if (l.batch_normalize && !l.dontloadscales) {
        read_floats(l.scales, (size_t)n, fp, "convolutional scales");
        read_floats(l.rolling_mean, (size_t)n, fp, "convolutional rolling_mean");
        read_floats(l.rolling_variance, (size_t)n, fp, "convolutional rolling_variance");
    }
    read_floats(l.weights, (size_t)num, fp, "convolutional weights");
    if (l.flipped) transpose_matrix(l.weights, l.c * l.size * l.size, n);
    push_convolutional_layer(l);
}

/* src/parser.c:1098-1120: biases, weights (transposed when the file says so), then the
 * batch-norm vectors - note the order differs from the convolutional layer's */
static void load_connected_weights(layer l, FILE *fp, int transpose)
{
    read_floats(l.biases, (size_t)l.outputs, fp, "connected biases");
    read_floats(l.weights, (size_t)l.outputs * l.inputs, fp, "connected weights");
    if (transpose) transpose_matrix(l.weights, l.inputs, l.outputs);
    if (l.batch_normalize && !l.dontloadscales) {
        read_floats(l.scales, (size_t)l.outputs, fp, "connected scales");
        read_floats(l.rolling_mean, (size_t)l.outputs, fp, "connected rolling_mean");
        read_floats(l.rolling_variance, (size_t)l.outputs, fp, "connected rolling_variance");
    }
    push_connected_layer(l);
}

void load_weights_upto(network *net, char *filename, int start, int cutoff)
{
    FILE *fp;
    int major, minor, revision, i, transpose;
    hip_set_device(net->gpu_index);
    if (dn_verbose) fprintf(stderr, "Loading weights from %s...", filename);
    fp = fopen(filename, "rb");
    if (!fp) file_error(filename);
    if (fread(&major, sizeof(int), 1, fp) != 1 || fread(&minor, sizeof(int), 1, fp) != 1 ||
        fread(&revision, sizeof(int), 1, fp) != 1)
        dn_fatal("weights file is shorter than its header");
    if ((major * 10 + minor) >= 2 && major < 1000 && minor < 1000) {
        if (fread(net->seen, sizeof(size_t), 1, fp) != 1) dn_fatal("weights file is shorter than its header");
    } else {
        int iseen = 0;
        if (fread(&iseen, sizeof(int), 1, fp) != 1) dn_fatal("weights file is shorter than its header");
        *net->seen = (size_t)iseen;
    }
    transpose = (major > 1000) || (minor > 1000); /* src/parser.c:1246 */
    for (i = start; i < net->n && i < cutoff; ++i) {
        layer l = net->layers[i];
        if (l.dontload) continue;
        if (l.type == CONVOLUTIONAL) load_convolutional_weights(l, fp);
        if (l.type == CONNECTED) load_connected_weights(l, fp, transpose);
        if (l.type == BATCHNORM) { /* src/parser.c:1122-1133 */
            read_floats(l.scales, (size_t)l.c, fp, "batchnorm scales");
            read_floats(l.rolling_mean, (size_t)l.c, fp, "batchnorm rolling_mean");
            read_floats(l.rolling_variance, (size_t)l.c, fp, "batchnorm rolling_variance");
            push_batchnorm_layer(l);
        }
        if (l.type == LOCAL) { /* src/parser.c:1292-1302 */
            read_floats(l.biases, (size_t)l.outputs, fp, "local biases");
            read_floats(l.weights, (size_t)l.nweights, fp, "local weights");
            push_local_layer(l);
        }
    }
    if (dn_verbose) fprintf(stderr, "Done!\n");
    fclose(fp);
}

void load_weights(network *net, char *filename)
{
    load_weights_upto(net, filename, 0, net->n);
}

void save_weights_upto(network *net, char *filename, int cutoff)
{
    FILE *fp;
    int major = 0, minor = 2, revision = 0, i;
    hip_set_device(net->gpu_index);
    if (dn_verbose) fprintf(stderr, "Saving weights to %s\n", filename);
    fp = fopen(filename, "wb");
    if (!fp) file_error(filename);
    fwrite(&major, sizeof(int), 1, fp);
    fwrite(&minor, sizeof(int), 1, fp);
    fwrite(&revision, sizeof(int), 1, fp);
    fwrite(net->seen, sizeof(size_t), 1, fp);
    for (i = 0; i < net->n && i < cutoff; ++i) {
        layer l = net->layers[i];
        if (l.type == CONNECTED) { /* src/parser.c:991-1005 */
            pull_connected_layer(l);
            fwrite(l.biases, sizeof(float), (size_t)l.outputs, fp);
            fwrite(l.weights, sizeof(float), (size_t)l.outputs * l.inputs, fp);
            if (l.batch_normalize) {
                fwrite(l.scales, sizeof(float), (size_t)l.outputs, fp);
                fwrite(l.rolling_mean, sizeof(float), (size_t)l.outputs, fp);
                fwrite(l.rolling_variance, sizeof(float), (size_t)l.outputs, fp);
            }
            continue;
        }
        if (l.type == BATCHNORM) { /* src/parser.c:979-990 */
            pull_batchnorm_layer(l);
            fwrite(l.scales, sizeof(float), (size_t)l.c, fp);
            fwrite(l.rolling_mean, sizeof(float), (size_t)l.c, fp);
            fwrite(l.rolling_variance, sizeof(float), (size_t)l.c, fp);
            continue;
        }
        if (l.type == LOCAL) { /* src/parser.c:1066-1077 */
            pull_local_layer(l);
            fwrite(l.biases, sizeof(float), (size_t)l.outputs, fp);
            fwrite(l.weights, sizeof(float), (size_t)l.nweights, fp);
            continue;
        }
        if (l.type != CONVOLUTIONAL) continue;
        pull_convolutional_layer(l);
        fwrite(l.biases, sizeof(float), (size_t)l.n, fp);
        if (l.batch_normalize) {
            fwrite(l.scales, sizeof(float), (size_t)l.n, fp);
            fwrite(l.rolling_mean, sizeof(float), (size_t)l.n, fp);
            fwrite(l.rolling_variance, sizeof(float), (size_t)l.n, fp);
        }
        fwrite(l.weights, sizeof(float), (size_t)l.nweights, fp);
    }
    fclose(fp);
}

void save_weights(network *net, char *filename)
{
    save_weights_upto(net, filename, net->n);
}
