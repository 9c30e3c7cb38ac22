/*
 * TEST INFRASTRUCTURE, NOT PRODUCT CODE (see oracle.h).
 *
 * CPU restatement of darknet's inference forward path.  Each function names the reference
 * lines whose behaviour it restates; paths are relative to the reference tree.  The arithmetic
 * is spelled out with explicit float/double conversions where the reference relies on C's
 * implicit promotions, because those promotions decide the last bit of the result.
 *
 * Build: `make -C oracle oracle` (strict -O2 -ffp-contract=off for parity work, and an
 * -Ofast -fopenmp twin that is only ever timed).
 */
#include "oracle.h"

#include <float.h>
#include <math.h>
#include <stdlib.h>
#include <string.h>

/* ---- im2col: src/im2col.c:3-12 (pixel fetch with zero outside), :16-39 (unroll) -------- */
void orc_im2col(const float *im, int channels, int height, int width,
                int ksize, int stride, int pad, float *col)
{
    const int oh = (height + 2 * pad - ksize) / stride + 1;
    const int ow = (width + 2 * pad - ksize) / stride + 1;
    const int rows = channels * ksize * ksize;
    for (int r = 0; r < rows; ++r) {
        const int kx = r % ksize;
        const int ky = (r / ksize) % ksize;
        const int ch = r / (ksize * ksize);
        float *dst = col + (long)r * oh * ow;
        for (int oy = 0; oy < oh; ++oy) {
            const int iy = oy * stride + ky - pad;
            for (int ox = 0; ox < ow; ++ox) {
                const int ix = ox * stride + kx - pad;
                float v = 0.f;
                if (iy >= 0 && ix >= 0 && iy < height && ix < width)
                    v = im[ix + width * (iy + height * ch)];
                dst[oy * ow + ox] = v;
            }
        }
    }
}

/* ---- gemm_nn: src/gemm.c:74-89.  C += (alpha*A[i][k]) * B[k][:] with k as the outer loop,
 * accumulated into C in memory in that order; rows are the only parallel axis (:80). -------- */
void orc_gemm_nn(int M, int N, int K, float alpha, const float *A, int lda,
                 const float *B, int ldb, float *C, int ldc)
{
#pragma omp parallel for
    for (int i = 0; i < M; ++i) {
        float *crow = C + (long)i * ldc;
        for (int k = 0; k < K; ++k) {
            const float a = alpha * A[(long)i * lda + k];
            const float *brow = B + (long)k * ldb;
            for (int j = 0; j < N; ++j) crow[j] += a * brow[j];
        }
    }
}

/* ---- normalize_cpu: src/blas.c:147-158.  sqrt is taken in double, the 1e-6f epsilon is
 * added outside the root, and the float numerator is divided in double. ------------------- */
void orc_normalize(float *x, const float *mean, const float *variance,
                   int batch, int filters, int spatial)
{
    for (int b = 0; b < batch; ++b)
        for (int f = 0; f < filters; ++f) {
            const double denom = sqrt((double)variance[f]) + (double).000001f;
            float *p = x + ((long)b * filters + f) * spatial;
            for (int i = 0; i < spatial; ++i) {
                const float num = p[i] - mean[f];
                p[i] = (float)((double)num / denom);
            }
        }
}

/* ---- scale_bias / add_bias: src/convolutional_layer.c:423-433, :411-421 ----------------- */
void orc_scale_bias(float *x, const float *scales, int batch, int n, int size)
{
    for (int b = 0; b < batch; ++b)
        for (int f = 0; f < n; ++f) {
            float *p = x + ((long)b * n + f) * size;
            for (int i = 0; i < size; ++i) p[i] *= scales[f];
        }
}

void orc_add_bias(float *x, const float *biases, int batch, int n, int size)
{
    for (int b = 0; b < batch; ++b)
        for (int f = 0; f < n; ++f) {
            float *p = x + ((long)b * n + f) * size;
            for (int i = 0; i < size; ++i) p[i] += biases[f];
        }
}

/* ---- activations: src/activations.h:18-52 (scalar forms), src/activations.c:65-106
 * (dispatch + array loop).  Literals such as .1 are doubles in the reference, so the product is
 * formed in double and rounded to float on return. --------------------------------------- */
static float act_one(float x, int a)
{
    const double xd = (double)x;
    switch (a) {
    case 0: /* logistic */ return (float)(1. / (1. + exp((double)(-x))));
    case 1: /* relu */ return x * (float)(x > 0);
    case 2: /* relie */ return (x > 0) ? x : (float)(.01 * xd);
    case 3: /* linear */ return x;
    case 4: /* ramp */ return (float)((double)(x * (float)(x > 0)) + .1 * xd);
    case 5: /* tanh */ {
        const double e = exp((double)(2 * x));
        return (float)((e - 1) / (e + 1));
    }
    case 6: /* plse */
        if (x < -4) return (float)(.01 * (double)(x + 4));
        if (x > 4) return (float)(.01 * (double)(x - 4) + 1);
        return (float)(.125 * xd + .5);
    case 7: /* leaky */ return (x > 0) ? x : (float)(.1 * xd);
    case 8: /* elu */ return (float)((double)((float)(x >= 0) * x) + (x < 0) * (exp(xd) - 1));
    case 9: /* loggy */ return (float)(2. / (1. + exp((double)(-x))) - 1);
    case 10: /* stair */ {
        const int n = (int)floor(xd);
        if (n % 2 == 0) return (float)floor(xd / 2.);
        return (float)((double)(x - n) + floor(xd / 2.));
    }
    case 11: /* hardtan */
        if (x < -1) return -1;
        if (x > 1) return 1;
        return x;
    case 12: /* lhtan */
        if (x < 0) return (float)(.001 * xd);
        if (x > 1) return (float)(.001 * (double)(x - 1) + 1);
        return x;
    case 13: /* selu */
        return (float)((x >= 0) * 1.0507 * xd + (x < 0) * 1.0507 * 1.6732 * (exp(xd) - 1));
    default: return 0;
    }
}

void orc_activate_array(float *x, long n, int activation)
{
    for (long i = 0; i < n; ++i) x[i] = act_one(x[i], activation);
}

/* ---- binarize_weights: src/convolutional_layer.c:28-41.  Sequential sum of |w| carried in
 * a float (each partial sum rounded), mean = sum/size, zero maps to -mean. ----------------- */
void orc_binarize_weights(const float *weights, int n, int size, float *binary)
{
    for (int f = 0; f < n; ++f) {
        const float *w = weights + (long)f * size;
        float mean = 0;
        for (int i = 0; i < size; ++i) mean = (float)((double)mean + fabs((double)w[i]));
        mean = mean / size;
        for (int i = 0; i < size; ++i) binary[(long)f * size + i] = (w[i] > 0) ? mean : -mean;
    }
}

/* ---- binarize_cpu: src/convolutional_layer.c:43-49.  0, -0 and NaN all map to -1. -------- */
void orc_binarize_input(const float *input, long n, float *binary)
{
    for (long i = 0; i < n; ++i) binary[i] = (input[i] > 0) ? 1.f : -1.f;
}

/* ---- forward_convolutional_layer: src/convolutional_layer.c:445-485, with the inference
 * branch of forward_batchnorm_layer (src/batchnorm_layer.c:135-155) as its tail.  A 1x1 kernel
 * feeds the image to the GEMM directly, whatever the stride (:468-469). ------------------- */
void orc_conv_forward(const float *input, const float *weights, const float *biases,
                      const float *scales, const float *rolling_mean,
                      const float *rolling_variance, float *output, float *workspace,
                      float *binary_weights, float *binary_input,
                      int batch, int c, int h, int w, int n, int groups, int size, int stride,
                      int pad, int batch_normalize, int activation, int xnor)
{
    const int out_h = (h + 2 * pad - size) / stride + 1;
    const int out_w = (w + 2 * pad - size) / stride + 1;
    const long outputs = (long)out_h * out_w * n;
    const int cg = c / groups;
    const long nweights = (long)cg * n * size * size;

    memset(output, 0, sizeof(float) * (size_t)(outputs * batch));

    if (xnor) {
        orc_binarize_weights(weights, n, cg * size * size, binary_weights);
        weights = binary_weights;
        orc_binarize_input(input, (long)c * h * w * batch, binary_input);
        input = binary_input;
    }

    const int M = n / groups;
    const int K = size * size * cg;
    const int N = out_w * out_h;
    for (int b = 0; b < batch; ++b)
        for (int g = 0; g < groups; ++g) {
            const float *A = weights + g * (nweights / groups);
            const float *im = input + ((long)b * groups + g) * cg * h * w;
            float *C = output + ((long)b * groups + g) * N * M;
            const float *B = im;
            if (size != 1) {
                orc_im2col(im, cg, h, w, size, stride, pad, workspace);
                B = workspace;
            }
            orc_gemm_nn(M, N, K, 1.f, A, K, B, N, C, N);
        }

    if (batch_normalize) {
        orc_normalize(output, rolling_mean, rolling_variance, batch, n, out_h * out_w);
        orc_scale_bias(output, scales, batch, n, out_h * out_w);
        orc_add_bias(output, biases, batch, n, out_h * out_w);
    } else {
        orc_add_bias(output, biases, batch, n, out_h * out_w);
    }
    orc_activate_array(output, outputs * batch, activation);
}

static double act_one_f64(double x, int a)
{
    switch (a) {
    case 0: return 1. / (1. + exp(-x));
    case 1: return x > 0 ? x : 0;
    case 2: return x > 0 ? x : .01 * x;
    case 3: return x;
    case 4: return (x > 0 ? x : 0) + .1 * x;
    case 5: return tanh(x);
    case 7: return x > 0 ? x : .1 * x;
    case 8: return x >= 0 ? x : exp(x) - 1;
    case 9: return 2. / (1. + exp(-x)) - 1;
    default: return (double)act_one((float)x, a);
    }
}

/* Referee (no reference counterpart by design): cross-correlation, NCHW, zero padding, groups,
 * as the definition reads, in double. */
void orc_conv_forward_f64(const float *input, const float *weights, const float *biases,
                          const float *scales, const float *rolling_mean,
                          const float *rolling_variance, double *output,
                          int batch, int c, int h, int w, int n, int groups, int size,
                          int stride, int pad, int batch_normalize, int activation)
{
    const int out_h = (h + 2 * pad - size) / stride + 1;
    const int out_w = (w + 2 * pad - size) / stride + 1;
    const int cg = c / groups;
    const int ng = n / groups;
    /* A 1x1 kernel in the reference ignores stride and pad (it multiplies the raw image), which
     * is only shape-consistent when stride==1 and pad==0; the referee keeps to that case. */
#pragma omp parallel for collapse(2)
    for (int b = 0; b < batch; ++b)
        for (int f = 0; f < n; ++f) {
            const int g = f / ng;
            double denom = 1, mean = 0, sc = 1;
            if (batch_normalize) {
                denom = sqrt((double)rolling_variance[f]) + (double).000001f;
                mean = rolling_mean[f];
                sc = scales[f];
            }
            for (int oy = 0; oy < out_h; ++oy)
                for (int ox = 0; ox < out_w; ++ox) {
                    double acc = 0;
                    for (int ci = 0; ci < cg; ++ci)
                        for (int ky = 0; ky < size; ++ky) {
                            const int iy = oy * stride + ky - pad;
                            if (iy < 0 || iy >= h) continue;
                            for (int kx = 0; kx < size; ++kx) {
                                const int ix = ox * stride + kx - pad;
                                if (ix < 0 || ix >= w) continue;
                                acc += (double)weights[((long)(f * cg + ci) * size + ky) * size + kx] *
                                       (double)input[(((long)b * c + g * cg + ci) * h + iy) * w + ix];
                            }
                        }
                    if (batch_normalize) acc = (acc - mean) / denom * sc;
                    acc += biases[f];
                    output[(((long)b * n + f) * out_h + oy) * out_w + ox] = act_one_f64(acc, activation);
                }
        }
}

/* ---- forward_maxpool_layer: src/maxpool_layer.c:79-114.  Window origin is (-pad)/2 in C
 * integer division; cells outside the image count as -FLT_MAX; the first strict maximum in
 * row-major window order wins and its flat input index is recorded (-1 if none). ----------- */
void orc_maxpool(const float *input, float *output, int *indexes, int batch, int c, int h,
                 int w, int size, int stride, int pad)
{
    const int off = -pad / 2;
    const int oh = (h + pad - size) / stride + 1;
    const int ow = (w + pad - size) / stride + 1;
    for (int b = 0; b < batch; ++b)
        for (int k = 0; k < c; ++k)
            for (int oy = 0; oy < oh; ++oy)
                for (int ox = 0; ox < ow; ++ox) {
                    float best = -FLT_MAX;
                    int best_i = -1;
                    for (int dy = 0; dy < size; ++dy)
                        for (int dx = 0; dx < size; ++dx) {
                            const int iy = off + oy * stride + dy;
                            const int ix = off + ox * stride + dx;
                            const int idx = ix + w * (iy + h * (k + b * c));
                            const int inside = iy >= 0 && iy < h && ix >= 0 && ix < w;
                            const float v = inside ? input[idx] : -FLT_MAX;
                            if (v > best) {
                                best = v;
                                best_i = idx;
                            }
                        }
                    const long o = ox + (long)ow * (oy + (long)oh * (k + (long)c * b));
                    output[o] = best;
                    indexes[o] = best_i;
                }
}

/* ---- forward_upsample_layer (non-reverse): src/upsample_layer.c:68-76 -> upsample_cpu
 * src/blas.c:334-349.  Nearest neighbour, every output written once as scale*in. ----------- */
void orc_upsample(const float *input, float *output, int batch, int c, int h, int w,
                  int stride, float scale)
{
    const int oh = h * stride, ow = w * stride;
    for (int b = 0; b < batch; ++b)
        for (int k = 0; k < c; ++k) {
            const float *src = input + ((long)b * c + k) * h * w;
            float *dst = output + ((long)b * c + k) * oh * ow;
            for (int y = 0; y < oh; ++y)
                for (int x = 0; x < ow; ++x) dst[(long)y * ow + x] = scale * src[(y / stride) * w + x / stride];
        }
}

/* ---- shortcut_cpu: src/blas.c:68-92 (called from src/shortcut_layer.c:62-67 after the layer
 * input was copied into out).  (w1,h1,c1) is the `add` tensor, (w2,h2,c2) is out. ---------- */
void orc_shortcut(int batch, int w1, int h1, int c1, const float *add, int w2, int h2, int c2,
                  float s1, float s2, float *out)
{
    int stride = w1 / w2;
    int sample = w2 / w1;
    if (stride < 1) stride = 1;
    if (sample < 1) sample = 1;
    const int mw = w1 < w2 ? w1 : w2;
    const int mh = h1 < h2 ? h1 : h2;
    const int mc = c1 < c2 ? c1 : c2;
    for (int b = 0; b < batch; ++b)
        for (int k = 0; k < mc; ++k)
            for (int j = 0; j < mh; ++j)
                for (int i = 0; i < mw; ++i) {
                    const long o = i * sample + (long)w2 * (j * sample + (long)h2 * (k + (long)c2 * b));
                    const long a = i * stride + (long)w1 * (j * stride + (long)h1 * (k + (long)c1 * b));
                    out[o] = s1 * out[o] + s2 * add[a];
                }
}

/* ---- forward_route_layer: src/route_layer.c:74-87, one source at a time: image j of the
 * source lands at dst + dst_offset + j*dst_stride. ---------------------------------------- */
void orc_route_copy(const float *src, int src_size, float *dst, int dst_stride, int dst_offset,
                    int batch)
{
    for (int j = 0; j < batch; ++j)
        memcpy(dst + dst_offset + (long)j * dst_stride, src + (long)j * src_size,
               sizeof(float) * (size_t)src_size);
}

/* ---- forward_yolo_layer, inference part of the CPU build: src/yolo_layer.c:132-148 with
 * entry_index :125-130.  Layout [b][anchor][entry][h][w]; entries 0,1 and 4..4+classes get the
 * logistic, entries 2,3 stay raw. ---------------------------------------------------------- */
void orc_yolo(const float *input, float *output, int batch, int w, int h, int n_anchors,
              int classes)
{
    const long plane = (long)w * h;
    const long per_anchor = plane * (4 + classes + 1);
    const long outputs = per_anchor * n_anchors;
    memcpy(output, input, sizeof(float) * (size_t)(outputs * batch));
    for (int b = 0; b < batch; ++b)
        for (int a = 0; a < n_anchors; ++a) {
            float *base = output + b * outputs + a * per_anchor;
            orc_activate_array(base, 2 * plane, 0);
            orc_activate_array(base + 4 * plane, (1 + classes) * plane, 0);
        }
}

/* ---- forward_avgpool_layer: src/avgpool_layer.c:40-55.  Sequential float sum, then divided
 * by the int h*w converted to float. ------------------------------------------------------ */
void orc_avgpool(const float *input, float *output, int batch, int c, int h, int w)
{
    const int area = h * w;
    for (int b = 0; b < batch; ++b)
        for (int k = 0; k < c; ++k) {
            const float *p = input + ((long)b * c + k) * area;
            float s = 0;
            for (int i = 0; i < area; ++i) s += p[i];
            output[k + b * c] = s / area;
        }
}

/* ---- softmax / softmax_cpu: src/blas.c:305-321, :324-332 (called from
 * src/softmax_layer.c:39-57 with n=inputs/groups, batch_offset=inputs, group_offset=n,
 * stride=1).  The exponent's argument is formed in float, exp itself runs in double. ------- */
static void softmax_one(const float *in, int n, float temp, int stride, float *out)
{
    float sum = 0;
    float largest = -FLT_MAX;
    for (int i = 0; i < n; ++i)
        if (in[i * stride] > largest) largest = in[i * stride];
    for (int i = 0; i < n; ++i) {
        const float arg = in[i * stride] / temp - largest / temp;
        const float e = (float)exp((double)arg);
        sum += e;
        out[i * stride] = e;
    }
    for (int i = 0; i < n; ++i) out[i * stride] /= sum;
}

void orc_softmax(const float *input, int n, int batch, int batch_offset, int groups,
                 int group_offset, int stride, float temp, float *output)
{
    for (int b = 0; b < batch; ++b)
        for (int g = 0; g < groups; ++g)
            softmax_one(input + b * batch_offset + g * group_offset, n, temp, stride,
                        output + b * batch_offset + g * group_offset);
}

/* ---- detections out of one yolo head: get_yolo_detections src/yolo_layer.c:316-343 for image
 * 0 of `pred` ([anchor][entry][lh][lw]), with get_yolo_box :83-91 and correct_yolo_boxes
 * :247-273.  Rows of (5 + classes) floats: x, y, w, h, objectness, prob[classes].  Returns the
 * number of rows written (the caller sizes `rows` for lw*lh*n). ---------------------------- */
int orc_yolo_detections(const float *pred, int lw, int lh, int n, int classes, const float *biases,
                        const int *mask, int netw, int neth, int w, int h, int relative, float thresh,
                        float *rows)
{
    const int cells = lw * lh;
    const int entries = 5 + classes;
    int count = 0;
    for (int i = 0; i < cells; ++i) {
        const int row = i / lw;
        const int col = i % lw;
        for (int a = 0; a < n; ++a) {
            const float *p = pred + (long)a * cells * entries + i;
            const float objectness = p[4L * cells];
            if (objectness <= thresh) continue;
            float *r = rows + (long)count * entries;
            /* get_yolo_box: stride = lw*lh */
            r[0] = (col + p[0]) / lw;
            r[1] = (row + p[1L * cells]) / lh;
            r[2] = exp(p[2L * cells]) * biases[2 * mask[a]] / netw;
            r[3] = exp(p[3L * cells]) * biases[2 * mask[a] + 1] / neth;
            r[4] = objectness;
            for (int j = 0; j < classes; ++j) {
                const float prob = objectness * p[(long)(5 + j) * cells];
                r[5 + j] = (prob > thresh) ? prob : 0;
            }
            ++count;
        }
    }
    /* correct_yolo_boxes */
    int new_w = 0, new_h = 0;
    if (((float)netw / w) < ((float)neth / h)) {
        new_w = netw;
        new_h = (h * netw) / w;
    } else {
        new_h = neth;
        new_w = (w * neth) / h;
    }
    for (int i = 0; i < count; ++i) {
        float *r = rows + (long)i * entries;
        float bx = r[0], by = r[1], bw = r[2], bh = r[3];
        bx = (bx - (netw - new_w) / 2. / netw) / ((float)new_w / netw);
        by = (by - (neth - new_h) / 2. / neth) / ((float)new_h / neth);
        bw *= (float)netw / new_w;
        bh *= (float)neth / new_h;
        if (!relative) {
            bx *= w;
            bw *= w;
            by *= h;
            bh *= h;
        }
        r[0] = bx;
        r[1] = by;
        r[2] = bw;
        r[3] = bh;
    }
    return count;
}

/* box_iou: src/box.c:111-155 */
static float orc_overlap(float x1, float w1, float x2, float w2)
{
    float l1 = x1 - w1 / 2;
    float l2 = x2 - w2 / 2;
    float left = l1 > l2 ? l1 : l2;
    float r1 = x1 + w1 / 2;
    float r2 = x2 + w2 / 2;
    float right = r1 < r2 ? r1 : r2;
    return right - left;
}

float orc_box_iou(const float *a, const float *b)
{
    float w = orc_overlap(a[0], a[2], b[0], b[2]);
    float h = orc_overlap(a[1], a[3], b[1], b[3]);
    float inter = (w < 0 || h < 0) ? 0 : w * h;
    float uni = a[2] * a[3] + b[2] * b[3] - inter;
    return inter / uni;
}

/* do_nms_sort: src/box.c:58-89, on rows that stay in place (the reference reorders its array;
 * here an index permutation is sorted instead, which suppresses the same pairs).  Ties in the
 * sort keep the lower row first. */
struct orc_nms_key {
    float p;
    int i;
};

static int orc_nms_cmp(const void *pa, const void *pb)
{
    const struct orc_nms_key *a = (const struct orc_nms_key *)pa, *b = (const struct orc_nms_key *)pb;
    float diff = a->p - b->p; /* nms_comparator src/box.c:5-21: descending probability */
    if (diff < 0) return 1;
    if (diff > 0) return -1;
    return a->i - b->i;
}

void orc_nms_sort(float *rows, int total, int classes, float thresh)
{
    const int entries = 5 + classes;
    struct orc_nms_key *keys = (struct orc_nms_key *)calloc((size_t)(total > 0 ? total : 1), sizeof *keys);
    for (int k = 0; k < classes; ++k) {
        int n = 0;
        for (int i = 0; i < total; ++i) {
            if (rows[(long)i * entries + 4] == 0) continue; /* objectness 0: dropped up front (:62-71) */
            keys[n].p = rows[(long)i * entries + 5 + k];
            keys[n].i = i;
            ++n;
        }
        qsort(keys, (size_t)n, sizeof *keys, orc_nms_cmp);
        for (int i = 0; i < n; ++i) {
            float *a = rows + (long)keys[i].i * entries;
            if (a[5 + k] == 0) continue;
            for (int j = i + 1; j < n; ++j) {
                float *b = rows + (long)keys[j].i * entries;
                if (orc_box_iou(a, b) > thresh) b[5 + k] = 0;
            }
        }
    }
    free(keys);
}

/* ---- forward_connected_layer: src/connected_layer.c:150-167.  gemm(0,1,...) = gemm_nt
 * (src/gemm.c:91-107): a register sum over k per output, added to the zero-filled output; then
 * forward_batchnorm_layer (out_c = outputs, 1x1 spatial) or add_bias, then the activation. --- */
void orc_connected_forward(const float *input, const float *weights, const float *biases,
                           const float *scales, const float *rolling_mean,
                           const float *rolling_variance, float *output, int batch, int inputs,
                           int outputs, int batch_normalize, int activation)
{
    memset(output, 0, sizeof(float) * (size_t)batch * outputs);
#pragma omp parallel for
    for (int i = 0; i < batch; ++i)
        for (int j = 0; j < outputs; ++j) {
            float sum = 0;
            for (int k = 0; k < inputs; ++k) sum += 1.f * input[(long)i * inputs + k] * weights[(long)j * inputs + k];
            output[(long)i * outputs + j] += sum;
        }
    if (batch_normalize) {
        orc_normalize(output, rolling_mean, rolling_variance, batch, outputs, 1);
        orc_scale_bias(output, scales, batch, outputs, 1);
        orc_add_bias(output, biases, batch, outputs, 1);
    } else {
        orc_add_bias(output, biases, batch, outputs, 1);
    }
    orc_activate_array(output, (long)outputs * batch, activation);
}

/* ---- reorg_cpu: src/blas.c:9-30 ------------------------------------------------------------ */
void orc_reorg(const float *x, int w, int h, int c, int batch, int stride, int forward, float *out)
{
    const int out_c = c / (stride * stride);
    for (int b = 0; b < batch; ++b)
        for (int k = 0; k < c; ++k)
            for (int j = 0; j < h; ++j)
                for (int i = 0; i < w; ++i) {
                    const long in_index = i + (long)w * (j + (long)h * (k + (long)c * b));
                    const int c2 = k % out_c;
                    const int offset = k / out_c;
                    const int w2 = i * stride + offset % stride;
                    const int h2 = j * stride + offset / stride;
                    const long out_index = w2 + (long)w * stride * (h2 + (long)h * stride * (c2 + (long)out_c * b));
                    if (forward) out[out_index] = x[in_index];
                    else out[in_index] = x[out_index];
                }
}

/* ---- flatten: src/blas.c:32-49 (out of place here) ----------------------------------------- */
void orc_flatten(const float *x, int size, int layers, int batch, int forward, float *out)
{
    for (int b = 0; b < batch; ++b)
        for (int c = 0; c < layers; ++c)
            for (int i = 0; i < size; ++i) {
                const long i1 = (long)b * layers * size + (long)c * size + i;
                const long i2 = (long)b * layers * size + (long)i * layers + c;
                if (forward) out[i2] = x[i1];
                else out[i1] = x[i2];
            }
}

/* ---- forward_crop_layer with net.train == 0: src/crop_layer.c:67-103 ----------------------- */
void orc_crop(const float *input, float *output, int batch, int c, int h, int w, int out_h, int out_w,
              int noadjust)
{
    const int dh = (h - out_h) / 2, dw = (w - out_w) / 2;
    float scale = 2, trans = -1;
    long count = 0;
    if (noadjust) {
        scale = 1;
        trans = 0;
    }
    for (int b = 0; b < batch; ++b)
        for (int k = 0; k < c; ++k)
            for (int i = 0; i < out_h; ++i)
                for (int j = 0; j < out_w; ++j) {
                    const long index = (j + dw) + (long)w * ((i + dh) + (long)h * (k + (long)c * b));
                    output[count++] = input[index] * scale + trans;
                }
}

/* ---- resize_image: src/image.c:1199-1241.  Horizontal pass into `part`, vertical pass from it;
 * images are [c][h][w]. ---------------------------------------------------------------------- */
void orc_resize_image(const float *im, int imw, int imh, int imc, float *resized, int w, int h)
{
    float *part = (float *)calloc((size_t)w * imh * imc, sizeof(float));
    const float w_scale = (float)(imw - 1) / (w - 1);
    const float h_scale = (float)(imh - 1) / (h - 1);
    for (int k = 0; k < imc; ++k)
        for (int r = 0; r < imh; ++r)
            for (int c = 0; c < w; ++c) {
                float val = 0;
                if (c == w - 1 || imw == 1) {
                    val = im[(long)k * imh * imw + (long)r * imw + imw - 1];
                } else {
                    float sx = c * w_scale;
                    int ix = (int)sx;
                    float dx = sx - ix;
                    val = (1 - dx) * im[(long)k * imh * imw + (long)r * imw + ix] +
                          dx * im[(long)k * imh * imw + (long)r * imw + ix + 1];
                }
                part[(long)k * imh * w + (long)r * w + c] = val;
            }
    for (int k = 0; k < imc; ++k)
        for (int r = 0; r < h; ++r) {
            float sy = r * h_scale;
            int iy = (int)sy;
            float dy = sy - iy;
            for (int c = 0; c < w; ++c)
                resized[(long)k * h * w + (long)r * w + c] = (1 - dy) * part[(long)k * imh * w + (long)iy * w + c];
            if (r == h - 1 || imh == 1) continue;
            for (int c = 0; c < w; ++c)
                resized[(long)k * h * w + (long)r * w + c] += dy * part[(long)k * imh * w + (long)(iy + 1) * w + c];
        }
    free(part);
}

/* ---- letterbox_image: src/image.c:812-831 with fill_image(.5) and embed_image :428-439 ----- */
void orc_letterbox_image(const float *im, int imw, int imh, int imc, float *boxed, int w, int h)
{
    int new_w = imw, new_h = imh;
    if (((float)w / imw) < ((float)h / imh)) {
        new_w = w;
        new_h = (imh * w) / imw;
    } else {
        new_h = h;
        new_w = (imw * h) / imh;
    }
    float *resized = (float *)calloc((size_t)new_w * new_h * imc, sizeof(float));
    orc_resize_image(im, imw, imh, imc, resized, new_w, new_h);
    for (long i = 0; i < (long)w * h * imc; ++i) boxed[i] = .5;
    const int dx = (w - new_w) / 2, dy = (h - new_h) / 2;
    for (int k = 0; k < imc; ++k)
        for (int y = 0; y < new_h; ++y)
            for (int x = 0; x < new_w; ++x) {
                const int X = dx + x, Y = dy + y;
                if (X < 0 || Y < 0 || X >= w || Y >= h) continue;
                boxed[(long)k * h * w + (long)Y * w + X] = resized[(long)k * new_h * new_w + (long)y * new_w + x];
            }
    free(resized);
}

/* ---- forward_region_layer, inference part of the CPU build: src/region_layer.c:158-184 with
 * entry_index :150-155 and softmax_cpu / softmax src/blas.c:305-332 (temp 1, stride w*h). ----- */
void orc_region(const float *input, float *output, int batch, int w, int h, int n_anchors, int classes,
                int coords, int background, int softmax)
{
    const long plane = (long)w * h;
    const long entries = coords + classes + 1;
    const long outputs = plane * entries * n_anchors;
    memcpy(output, input, sizeof(float) * (size_t)(outputs * batch));
    for (int b = 0; b < batch; ++b)
        for (int n = 0; n < n_anchors; ++n) {
            float *base = output + b * outputs + n * plane * entries;
            orc_activate_array(base, 2 * plane, 0);
            if (!background) orc_activate_array(base + coords * plane, plane, 0);
            if (!softmax) orc_activate_array(base + (coords + 1) * plane, classes * plane, 0);
        }
    if (softmax) {
        const long first = (coords + !background) * plane;
        const int cnt = classes + background;
        for (long g = 0; g < (long)batch * n_anchors; ++g)
            for (long cell = 0; cell < plane; ++cell) {
                const float *x = input + g * (outputs / n_anchors) + first + cell;
                float *y = output + g * (outputs / n_anchors) + first + cell;
                float sum = 0;
                float largest = -FLT_MAX;
                for (int i = 0; i < cnt; ++i)
                    if (x[i * plane] > largest) largest = x[i * plane];
                for (int i = 0; i < cnt; ++i) {
                    float e = exp(x[i * plane] / 1.f - largest / 1.f);
                    sum += e;
                    y[i * plane] = e;
                }
                for (int i = 0; i < cnt; ++i) y[i * plane] /= sum;
            }
    }
}

/* ---- get_region_detections: src/region_layer.c:364-437 (no tree, no map, coords 4) for image 0
 * of `pred`; writes all lw*lh*n rows, row anchor*lw*lh + cell. -------------------------------- */
int orc_region_detections(const float *pred, int lw, int lh, int n, int classes, int coords, int background,
                          const float *biases, int netw, int neth, int w, int h, int relative, float thresh,
                          float *rows)
{
    const int cells = lw * lh;
    const int entries = coords + classes + 1;
    const int out_entries = 5 + classes;
    for (int i = 0; i < cells; ++i) {
        const int row = i / lw;
        const int col = i % lw;
        for (int a = 0; a < n; ++a) {
            const int index = a * cells + i;
            float *r = rows + (long)index * out_entries;
            const float *p = pred + (long)a * cells * entries + i;
            for (int j = 0; j < classes; ++j) r[5 + j] = 0;
            const float scale = background ? 1 : p[(long)coords * cells];
            r[0] = (col + p[0]) / lw;
            r[1] = (row + p[1L * cells]) / lh;
            r[2] = exp(p[2L * cells]) * biases[2 * a] / lw;
            r[3] = exp(p[3L * cells]) * biases[2 * a + 1] / lh;
            r[4] = scale > thresh ? scale : 0;
            if (r[4]) {
                for (int j = 0; j < classes; ++j) {
                    const float prob = scale * p[(long)(coords + 1 + j) * cells];
                    r[5 + j] = (prob > thresh) ? prob : 0;
                }
            }
        }
    }
    /* correct_region_boxes :336-362 */
    int new_w = 0, new_h = 0;
    if (((float)netw / w) < ((float)neth / h)) {
        new_w = netw;
        new_h = (h * netw) / w;
    } else {
        new_h = neth;
        new_w = (w * neth) / h;
    }
    for (int i = 0; i < cells * n; ++i) {
        float *r = rows + (long)i * out_entries;
        float bx = r[0], by = r[1], bw = r[2], bh = r[3];
        bx = (bx - (netw - new_w) / 2. / netw) / ((float)new_w / netw);
        by = (by - (neth - new_h) / 2. / neth) / ((float)new_h / neth);
        bw *= (float)netw / new_w;
        bh *= (float)neth / new_h;
        if (!relative) {
            bx *= w;
            bw *= w;
            by *= h;
            bh *= h;
        }
        r[0] = bx;
        r[1] = by;
        r[2] = bw;
        r[3] = bh;
    }
    return cells * n;
}

/* ---- forward_local_layer: src/local_layer.c:91-120.  Output starts as the per-element biases
 * (:97-99); per image one im2col (pad is the pixel count here), then for every location j a
 * [n x K] by [K x 1] gemm on column j of the im2col buffer, accumulated into out[., j] in the
 * reference's k order (:101-117); then the activation.  Weights are location-major.
 * workspace: K * locations floats. -------------------------------------------------------------- */
void orc_local_forward(const float *input, const float *weights, const float *biases, float *output, int batch,
                       int c, int h, int w, int n, int size, int stride, int pad, int activation, float *workspace)
{
    const int out_h = (h - (pad ? 1 : size)) / stride + 1; /* local_out_height :10-16 */
    const int out_w = (w - (pad ? 1 : size)) / stride + 1;
    const int locations = out_h * out_w;
    const int K = size * size * c;
    const long outputs = (long)locations * n;
    for (int b = 0; b < batch; ++b) {
        float *out = output + b * outputs;
        for (long i = 0; i < outputs; ++i) out[i] = biases[i];
        orc_im2col(input + (long)b * c * h * w, c, h, w, size, stride, pad, workspace);
        for (int j = 0; j < locations; ++j)
            orc_gemm_nn(n, 1, K, 1.f, weights + (long)j * K * n, K, workspace + j, locations, out + j, locations);
    }
    orc_activate_array(output, outputs * batch, activation);
}

/* ---- forward_detection_layer at inference: src/detection_layer.c:50-66: a copy, then softmax
 * over each cell's classes when `softmax` is set. ---------------------------------------------- */
void orc_detection_forward(const float *input, float *output, int batch, int inputs, int side, int classes,
                           int softmax)
{
    memcpy(output, input, sizeof(float) * (size_t)inputs * batch);
    if (!softmax) return;
    for (int b = 0; b < batch; ++b)
        for (int i = 0; i < side * side; ++i) {
            const long o = (long)b * inputs + (long)i * classes;
            orc_softmax(output + o, classes, 1, 0, 1, 0, 1, 1.f, output + o);
        }
}

/* ---- get_detection_detections: src/detection_layer.c:225-252 on image 0 of `pred`; all
 * side*side*n rows, row cell*n + box: x, y, w, h, objectness (the box scale, whatever the
 * threshold), prob[classes]. -------------------------------------------------------------------- */
int orc_detection_detections(const float *pred, int side, int n, int classes, int sqrt_flag, int w, int h,
                             float thresh, float *rows)
{
    for (int i = 0; i < side * side; ++i) {
        const int row = i / side;
        const int col = i % side;
        for (int k = 0; k < n; ++k) {
            const int index = i * n + k;
            const int p_index = side * side * classes + i * n + k;
            const float scale = pred[p_index];
            const int box_index = side * side * (classes + n) + (i * n + k) * 4;
            float *r = rows + (long)index * (5 + classes);
            r[0] = (pred[box_index + 0] + col) / side * w;
            r[1] = (pred[box_index + 1] + row) / side * h;
            r[2] = pow(pred[box_index + 2], (sqrt_flag ? 2 : 1)) * w;
            r[3] = pow(pred[box_index + 3], (sqrt_flag ? 2 : 1)) * h;
            r[4] = scale;
            for (int j = 0; j < classes; ++j) {
                const float prob = scale * pred[i * classes + j];
                r[5 + j] = (prob > thresh) ? prob : 0;
            }
        }
    }
    return side * side * n;
}
