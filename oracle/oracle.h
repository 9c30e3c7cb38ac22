/*
 * TEST INFRASTRUCTURE, NOT PRODUCT CODE.
 *
 * CPU restatement of the inference forward path of pjreddie/darknet, written from the
 * reference's behaviour (file:line citations on every function in oracle.c).  It exists so that
 * the HIP library can be checked on a machine where the reference sources are absent.  Only
 * tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg may load it; the shipped
 * library never links, loads or calls anything in this directory.
 *
 * Every function here is pinned, in tests/test_oracle_*.py, against the compiled reference
 * (oracle/_ref, when built) and against independent mathematics (fp64 direct convolution,
 * torch CPU conv2d / max_pool2d / interpolate, closed forms, brute force on tiny inputs).
 *
 * Activation codes follow the reference enum order (include/darknet.h:48-50):
 * LOGISTIC 0, RELU 1, RELIE 2, LINEAR 3, RAMP 4, TANH 5, PLSE 6, LEAKY 7, ELU 8, LOGGY 9,
 * STAIR 10, HARDTAN 11, LHTAN 12, SELU 13.
 */
#ifndef DN_ORACLE_H
#define DN_ORACLE_H

#ifdef __cplusplus
extern "C" {
#endif

void orc_im2col(const float *im, int channels, int height, int width,
                int ksize, int stride, int pad, float *col);

void orc_gemm_nn(int M, int N, int K, float alpha, const float *A, int lda,
                 const float *B, int ldb, float *C, int ldc);

void orc_normalize(float *x, const float *mean, const float *variance,
                   int batch, int filters, int spatial);
void orc_scale_bias(float *x, const float *scales, int batch, int n, int size);
void orc_add_bias(float *x, const float *biases, int batch, int n, int size);
void orc_activate_array(float *x, long n, int activation);

void orc_binarize_weights(const float *weights, int n, int size, float *binary);
void orc_binarize_input(const float *input, long n, float *binary);

/* Whole convolutional layer forward.  `workspace` holds out_h*out_w*size*size*c/groups floats.
 * `binary_weights` (nweights) and `binary_input` (batch*c*h*w) are only touched when xnor!=0. */
void orc_conv_forward(const float *input, const float *weights, const float *biases,
                      const float *scales, const float *rolling_mean,
                      const float *rolling_variance, float *output, float *workspace,
                      float *binary_weights, float *binary_input,
                      int batch, int c, int h, int w, int n, int groups, int size, int stride,
                      int pad, int batch_normalize, int activation, int xnor);

/* Referee: the same layer as a direct 7-loop cross-correlation accumulated in double, with the
 * batch-norm / bias / activation tail evaluated in double.  Independent of im2col and gemm. */
void orc_conv_forward_f64(const float *input, const float *weights, const float *biases,
                          const float *scales, const float *rolling_mean,
                          const float *rolling_variance, double *output,
                          int batch, int c, int h, int w, int n, int groups, int size,
                          int stride, int pad, int batch_normalize, int activation);

void orc_maxpool(const float *input, float *output, int *indexes, int batch, int c, int h,
                 int w, int size, int stride, int pad);
void orc_upsample(const float *input, float *output, int batch, int c, int h, int w,
                  int stride, float scale);
/* out holds a copy of the layer input on entry (w2,h2,c2); add has geometry (w1,h1,c1). */
void orc_shortcut(int batch, int w1, int h1, int c1, const float *add, int w2, int h2, int c2,
                  float s1, float s2, float *out);
void orc_route_copy(const float *src, int src_size, float *dst, int dst_stride, int dst_offset,
                    int batch);
void orc_yolo(const float *input, float *output, int batch, int w, int h, int n_anchors,
              int classes);
void orc_avgpool(const float *input, float *output, int batch, int c, int h, int w);
void orc_softmax(const float *input, int n, int batch, int batch_offset, int groups,
                 int group_offset, int stride, float temp, float *output);

void orc_connected_forward(const float *input, const float *weights, const float *biases,
                           const float *scales, const float *rolling_mean,
                           const float *rolling_variance, float *output, int batch, int inputs,
                           int outputs, int batch_normalize, int activation);
void orc_reorg(const float *x, int w, int h, int c, int batch, int stride, int forward, float *out);
void orc_flatten(const float *x, int size, int layers, int batch, int forward, float *out);
void orc_crop(const float *input, float *output, int batch, int c, int h, int w, int out_h, int out_w,
              int noadjust);

void orc_resize_image(const float *im, int imw, int imh, int imc, float *resized, int w, int h);
void orc_letterbox_image(const float *im, int imw, int imh, int imc, float *boxed, int w, int h);

void orc_region(const float *input, float *output, int batch, int w, int h, int n_anchors, int classes,
                int coords, int background, int softmax);
int orc_region_detections(const float *pred, int lw, int lh, int n, int classes, int coords, int background,
                          const float *biases, int netw, int neth, int w, int h, int relative, float thresh,
                          float *rows);

void orc_local_forward(const float *input, const float *weights, const float *biases, float *output, int batch,
                       int c, int h, int w, int n, int size, int stride, int pad, int activation, float *workspace);
void orc_detection_forward(const float *input, float *output, int batch, int inputs, int side, int classes,
                           int softmax);
int orc_detection_detections(const float *pred, int side, int n, int classes, int sqrt_flag, int w, int h,
                             float thresh, float *rows);

/* detections (test infrastructure like everything here): see oracle.c */
int orc_yolo_detections(const float *pred, int lw, int lh, int n, int classes, const float *biases,
                        const int *mask, int netw, int neth, int w, int h, int relative, float thresh,
                        float *rows);
float orc_box_iou(const float *a, const float *b);
void orc_nms_sort(float *rows, int total, int classes, float thresh);

#ifdef __cplusplus
}
#endif
#endif
