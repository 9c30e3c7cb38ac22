/*
 * darknet_hip.h - device layer of the darknet forward path on AMD MI355X (gfx950).
 *
 * This is the C-ABI a darknet tree binds in place of src/cuda.c, the src/ *_kernels.cu files and cuBLAS:
 * plain pointers and sizes only.  Every pointer named *_gpu (and every `float *` argument of a
 * *_gpu function) is device memory obtained from hip_make_array / cuda_make_array.  All work is
 * issued on one stream (hip_get_stream(), the null stream unless changed) and is asynchronous
 * with respect to the host except the push/pull copies, as in the reference.
 *
 * Error convention is the reference's (src/cuda.c:27-49, src/utils.c:253-258): a failed HIP
 * call or an argument the kernels cannot honour prints a message to stderr and ends the
 * process with exit(-1).  There is no CPU fallback anywhere in this library.
 *
 * Citations name the reference interface each entry point replaces (paths relative to the
 * pjreddie/darknet tree).
 */
#ifndef DARKNET_HIP_H
#define DARKNET_HIP_H

#include <stddef.h>

#ifdef __cplusplus
extern "C" {
#endif

/* ACTIVATION codes, same order as the reference enum (include/darknet.h:48-50). */
enum {
    DN_LOGISTIC = 0, DN_RELU, DN_RELIE, DN_LINEAR, DN_RAMP, DN_TANH, DN_PLSE, DN_LEAKY, DN_ELU,
    DN_LOGGY, DN_STAIR, DN_HARDTAN, DN_LHTAN, DN_SELU
};

/* ------------------------------------------------------------------------------------------
 * Device shim: replaces src/cuda.c / src/cuda.h (and include/darknet.h:632-637).
 * The cuda_* spellings are exported as real symbols as well, so reference objects that call
 * them link unchanged.
 * ---------------------------------------------------------------------------------------- */
extern int gpu_index;                                   /* src/cuda.c:1 */
void   hip_set_device(int n);                           /* cuda_set_device      src/cuda.c:12  */
int    hip_get_device(void);                            /* cuda_get_device      src/cuda.c:19  */
void   hip_check_error(int status);                     /* check_error          src/cuda.c:27  */
float *hip_make_array(float *x, size_t n);              /* cuda_make_array      src/cuda.c:90  */
int   *hip_make_int_array(int *x, size_t n);            /* cuda_make_int_array  src/cuda.c:133 */
void   hip_free(float *x_gpu);                          /* cuda_free            src/cuda.c:147 */
void   hip_push_array(float *x_gpu, float *x, size_t n);/* cuda_push_array      src/cuda.c:153 */
void   hip_pull_array(float *x_gpu, float *x, size_t n);/* cuda_pull_array      src/cuda.c:160 */
float  hip_mag_array(float *x_gpu, size_t n);           /* cuda_mag_array       src/cuda.c:167 */
float  hip_compare(float *x_gpu, float *x, size_t n, char *s); /* cuda_compare  src/cuda.c:120 */
void   hip_random(float *x_gpu, size_t n);              /* cuda_random          src/cuda.c:106: n uniform floats in
                                                         * (0, 1]; the reference seeds with time(0), the stream here
                                                         * is a counter-based hash (dropout / crop at training time
                                                         * are its only readers; inference never calls it) */
void   hip_pull_int_array(int *x_gpu, int *x, size_t n);/* (maxpool indexes; no reference twin) */
void   hip_push_int_array(int *x_gpu, int *x, size_t n);/* (counters; no reference twin)        */
void   hip_synchronize(void);                           /* hipStreamSynchronize on the stream  */
/* Pinned host memory (zero-filled; no reference twin): hip_push_array / hip_pull_array move such a
 * buffer with one DMA at the link's rate instead of staging it through a host memcpy.  The library
 * uses it for the outputs network_predict returns; callers may use it for their input batches.
 * hip_host_free also accepts (and free()s) ordinary malloc'ed pointers. */
float *hip_host_alloc(size_t n);
void   hip_host_free(float *x);
/* Parse-only mode (no reference twin): after hip_set_parse_only(1) the cfg parser, the layer-table
 * queries and the weights-file reader/writer work on host memory alone, on a machine with or
 * without a GPU: nothing is allocated on or copied to a device (device pointers stay NULL).  It
 * computes nothing: network_predict, forward_network* and every other call that needs the device
 * print a message and exit(-1). */
void   hip_set_parse_only(int on);
int    hip_parse_only(void);
void  *hip_get_stream(void);                            /* hipStream_t the library launches on */
void   hip_set_stream(void *stream);                    /* 0 selects the null stream           */
const char *hip_device_name(void);

void   cuda_set_device(int n);
int    cuda_get_device(void);
float *cuda_make_array(float *x, size_t n);
int   *cuda_make_int_array(int *x, size_t n);
void   cuda_free(float *x_gpu);
void   cuda_push_array(float *x_gpu, float *x, size_t n);
void   cuda_pull_array(float *x_gpu, float *x, size_t n);
float  cuda_mag_array(float *x_gpu, size_t n);
float  cuda_compare(float *x_gpu, float *x, size_t n, char *s);
void   cuda_random(float *x_gpu, size_t n);

/* Event timing on the library's stream (used by the benchmark; no reference twin). */
void  *hip_event_create(void);
void   hip_event_record(void *ev);
float  hip_event_elapsed_ms(void *start, void *stop);   /* synchronises on `stop` */
void   hip_event_destroy(void *ev);

/* ------------------------------------------------------------------------------------------
 * Element-wise helpers with the reference's own names and argument order
 * (src/blas.h:51-102, src/activations.h:15, src/im2col.h:10; kernels in src/blas_kernels.cu,
 * src/activation_kernels.cu, src/im2col_kernels.cu).  Arithmetic follows the CPU forms the
 * parity contract names: normalize uses (x-mean)/(sqrt(var)+1e-6f) (src/blas.c:154), leaky and
 * logistic are evaluated in double (src/activations.h:32,39).
 * ---------------------------------------------------------------------------------------- */
void fill_gpu(int N, float ALPHA, float *X, int INCX);                       /* blas.h:100 */
void copy_gpu(int N, float *X, int INCX, float *Y, int INCY);                /* blas.h:53  */
void copy_gpu_offset(int N, float *X, int OFFX, int INCX, float *Y, int OFFY, int INCY); /* :54 */
#ifndef DARKNET_API  /* inside a darknet tree src/activations.h:15 declares it with the ACTIVATION enum */
void activate_array_gpu(float *x, int n, int activation);                    /* activations.h:15 */
#endif
void normalize_gpu(float *x, float *mean, float *variance, int batch, int filters, int spatial); /* blas.h:65 */
void scale_bias_gpu(float *output, float *scales, int batch, int n, int size);  /* blas.h:76 */
void add_bias_gpu(float *output, float *biases, int batch, int n, int size);    /* blas.h:79 */
void shortcut_gpu(int batch, int w1, int h1, int c1, float *add, int w2, int h2, int c2,
                  float s1, float s2, float *out);                           /* blas.h:75  */
void upsample_gpu(float *in, int w, int h, int c, int batch, int stride, int forward,
                  float scale, float *out);                                  /* blas.h:102 */
void softmax_gpu(float *input, int n, int batch, int batch_offset, int groups, int group_offset,
                 int stride, float temp, float *output);                     /* blas.h:96  */
void im2col_gpu(float *im, int channels, int height, int width, int ksize, int stride, int pad,
                float *data_col);                                            /* im2col.h:10 */
void binarize_gpu(float *x, int n, float *binary);            /* convolutional_kernels.cu:23; x>0 as on the CPU */
void binarize_weights_gpu(float *weights, int n, int size, float *binary); /* convolutional_kernels.cu:67 */

/* ------------------------------------------------------------------------------------------
 * Fused layer forwards.  Each replaces the body of the reference's forward_*_layer_gpu for
 * the inference case (net.train == 0); a darknet tree calls them from those functions with the
 * fields of `layer` / `network` spelled out.
 * ---------------------------------------------------------------------------------------- */

/* Convolution + batch-norm/bias + activation in one pass.
 * Replaces forward_convolutional_layer_gpu (src/convolutional_kernels.cu:73-135), i.e. the
 * fill_gpu / im2col_gpu / gemm_gpu(cublasSgemm) loop over batch x groups plus the
 * normalize/scale/add_bias/activate passes; CPU semantics of src/convolutional_layer.c:445-485.
 *   input   [batch][c][h][w]                  weights [n][c/groups][size][size]
 *   output  [batch][n][out_h][out_w],  out = (in + 2*pad - size)/stride + 1
 *   batch_normalize != 0: scales, rolling_mean, rolling_variance (n each) are read;
 *   otherwise they may be NULL.  biases (n) are always read.
 *   packed: NULL, or the buffer written by conv_pack_weights_gpu for these weights (skips the
 *   per-call repack; must be refreshed whenever the weights change).
 * A 1x1 kernel must come with stride 1 and pad 0 (the reference feeds the image straight to
 * the GEMM in that case, src/convolutional_layer.c:468-469; every cfg in the tree obeys it).
 * Results are deterministic run to run.  The order in which K is summed depends on how the launch
 * fills the chip, hence on the batch size: tiles of the last, partial round are cut along K and the
 * slices summed in slice order.  The same image therefore gives the same values at every batch size
 * only to rounding (measured <= 1e-5 of the layer's largest value, tests hold 2e-5), where the
 * reference's per-image GEMM gives the same bits.  conv_set_algo(3), or conv_set_ksplit(1, 0),
 * switches the cut off: then every output sums K in one fixed order and the bits no longer depend
 * on the batch size (tested).
 * Which kernel runs is decided by the geometry (conv_kernel_name_geometry names it): the implicit-GEMM
 * kernel on the fp32 matrix cores for nearly everything; kernels of their own for the first layers
 * of an image network (3x3 / 1 / pad 1 over 3 channels, or over 16 channels into up to 32 filters)
 * and for grouped 3x3 layers of 4 or 8 channels per group (vector ALU); a plain direct kernel for the
 * rest (groups that fit no tile scheme, 3x3 without padding on tap-blocked layers, one image beyond
 * 4 GiB).  `packed` is only read by the implicit-GEMM kernel. */
void forward_convolutional_gpu(const float *input, const float *weights, const float *packed,
                               const float *biases, const float *scales,
                               const float *rolling_mean, const float *rolling_variance,
                               float *output, int batch, int c, int h, int w, int n,
                               int groups, int size, int stride, int pad, int batch_normalize,
                               int activation);

/* Convolution layer followed by a same-geometry shortcut layer, in one pass: `output` receives
 * what forward_convolutional_gpu writes and `sum_output` what the shortcut layer after it would:
 *   sum_output[i] = shortcut_activation(alpha*output[i] + beta*add[i])
 * with add and sum_output of output's shape [batch][n][out_h][out_w].  Replaces the pair
 * forward_convolutional_layer_gpu (src/convolutional_kernels.cu:73-135) + forward_shortcut_layer_gpu
 * (src/shortcut_layer.c:77-83: copy_gpu, shortcut_gpu, activate_array_gpu) when the shortcut's
 * `from` layer has the convolution's output geometry, as in every darknet53 residual block; the
 * results equal those of the two separate calls bit for bit.  The residual is read and the sum
 * written in the convolution's epilogue, which saves the shortcut's own pass over memory.
 * sum_output must not alias output; add may be any other buffer. */
void forward_convolutional_shortcut_gpu(const float *input, const float *weights, const float *packed,
                                        const float *biases, const float *scales,
                                        const float *rolling_mean, const float *rolling_variance,
                                        float *output, int batch, int c, int h, int w, int n,
                                        int groups, int size, int stride, int pad, int batch_normalize,
                                        int activation, const float *add, float *sum_output, float alpha,
                                        float beta, int shortcut_activation);

/* Convolution layer followed by the yolo layer it feeds, in one pass: `output` receives what
 * forward_convolutional_gpu writes and `yolo_output` what forward_yolo_gpu would make of it
 * (src/yolo_layer.c:132-148: the copy, with the logistic on x, y, objectness and classes of every
 * anchor; n must be n_anchors * (5 + classes)).  Replaces the pair forward_convolutional_layer_gpu
 * + forward_yolo_layer_gpu of a detection head; both buffers hold the bits the two separate
 * calls write, and the head's own pass over memory disappears.  yolo_output must not alias output. */
void forward_convolutional_yolo_gpu(const float *input, const float *weights, const float *packed,
                                    const float *biases, const float *scales,
                                    const float *rolling_mean, const float *rolling_variance,
                                    float *output, int batch, int c, int h, int w, int n, int groups,
                                    int size, int stride, int pad, int batch_normalize, int activation,
                                    float *yolo_output, int n_anchors, int classes);

/* forward_convolutional_gpu for callers that cannot allocate device memory (code under stream
 * capture, tight serving loops, harnesses that forbid hipMalloc).  No counterpart in the
 * reference.  Same arguments and same result, bit for bit; the call itself makes no hipMalloc /
 * hipFree or any other allocating call: the K-split accumulators, the one buffer
 * forward_convolutional_gpu grows on demand, live in a fixed 64 MiB array inside the library's
 * code object (one copy per device, held until the process ends).
 *   - `packed` must be the buffer conv_pack_weights_gpu wrote wherever conv_packed_floats() != 0
 *     (the per-call repack would need a buffer);
 *   - conv_set_precision(1) is refused for 3x3 layers (that mode stages its input);
 *   - a geometry whose K-split needs more than 64 MiB is refused (none of the benchmark
 *     networks comes near: their largest need is 48 MB).
 * Returns 0, or -1 after a message on stderr when the call was refused; a refused call launches
 * nothing (one exception: a batch beyond the kernels' 32-bit offsets, 4 GiB of input, runs in
 * slices of whole images, and a slice can be refused after earlier ones ran) and drops a pending
 * conv_profile_next pair.  The address of the array is looked up once per device (hip_set_device does it;
 * otherwise the first call on that device, which should then precede any stream capture).
 * Every call on a device shares that device's array: calls that overlap on one device - two
 * streams, two host threads - race.  Calls on one stream are ordered and safe. */
int forward_convolutional_noalloc_gpu(const float *input, const float *weights, const float *packed,
                                      const float *biases, const float *scales,
                                      const float *rolling_mean, const float *rolling_variance,
                                      float *output, int batch, int c, int h, int w, int n,
                                      int groups, int size, int stride, int pad, int batch_normalize,
                                      int activation);

/* Weight repack for the MFMA kernel (the natural hook is push_convolutional_layer,
 * src/convolutional_kernels.cu:286-297).  conv_packed_floats() == 0 means the layer does not
 * use a packed copy (grouped convolutions outside the 32-filter block-diagonal scheme).  The
 * buffer holds the fp32 layout and, for layers the bf16-operand mode can serve, a bf16 copy
 * behind it (half as many bytes again), so conv_set_precision() needs no repacking. */
size_t conv_packed_floats(int n, int c, int groups, int size);
void conv_pack_weights_gpu(const float *weights, float *packed, int n, int c, int groups, int size);

/* The packed copy for binders whose `layer` struct has no member to keep it in (a darknet tree that
 * keeps the reference's include/darknet.h:115-422 as it is).  No counterpart in the reference.
 * conv_packed_cached_gpu returns the packed copy of the weights at device address `weights`, packing
 * them on the first call for that address and geometry; NULL when conv_packed_floats() == 0.  The
 * library owns the copy and drops it when those weights are freed through hip_free / cuda_free or
 * written through hip_push_array / cuda_push_array; a binder that writes the weights any other way
 * calls conv_packed_forget(weights) afterwards.  One host thread at a time, like the rest of the shim. */
const float *conv_packed_cached_gpu(const float *weights, int n, int c, int groups, int size);
void conv_packed_forget(const float *weights);
int conv_packed_cached_count(void);

/* Name of the kernel forward_convolutional_gpu launches for this geometry, as it appears in a
 * profiler trace (e.g. "conv_mfma_kernel<128,128,64,64,3>"); for reports only. */
const char *conv_kernel_name(int n, int c, int groups, int size);
/* The same for a layer of `columns` = batch*out_h*out_w output columns: the tile depends on the
 * number of columns (1x1 layers and layers of up to 64 filters run 64x64 tiles, 3x3 layers of 128 to
 * 256 channels and layers whose wide tiles would not fill the chip 128x64 tiles), and a launch that
 * does not fill the chip runs the variant whose K-order number carries +100 (e.g.
 * "conv_mfma_kernel<128,64,64,32,113>"). */
const char *conv_kernel_name_columns(int n, int c, int groups, int size, long columns);
/* The same for a layer whose whole geometry is known, decided by the very predicates the dispatch
 * uses; the only form that can name the first-layer kernel ("conv_patch_kernel<1,3>": 3 channels,
 * 3x3, stride 1, pad 1, up to 64 filters, image a multiple of 256 pixels and its width of 4) and
 * the direct kernel of geometries the MFMA kernels do not serve. */
const char *conv_kernel_name_geometry(int batch, int c, int h, int w, int n, int groups, int size,
                                      int stride, int pad);

/* Kernel timing for reports: the next forward_convolutional[_shortcut]_gpu call that runs on the
 * MFMA kernel attaches these two events (hip_event_create) to its main kernel's dispatch, so
 * hip_event_elapsed_ms(start, stop) is the kernel's own duration as a profiler reports it (the
 * K-split reduce pass and launch gaps excluded).  conv_profile_pending() != 0 afterwards means the
 * call took another kernel and the events were not recorded. */
void conv_profile_next(void *start_event, void *stop_event);
int conv_profile_pending(void);

/* Selects the convolution kernel: 0 = automatic (default), 1 = always the plain direct
 * kernel, 3 = MFMA kernel without the K-split of the last partial round of tiles.  The direct
 * kernel is the in-library cross-check of the MFMA kernel. */
void conv_set_algo(int algo);

/* Tuning hooks of the K-split (no counterpart in the reference).  When a layer's last round of
 * tiles would leave most of the chip idle, those tiles are cut along K into slices that a second
 * launch sums in slice order.
 *   split   0 = the cost model decides, n > 0 = n slices for every such tile (1 = none),
 *           -n (n = 2..32) = n slices for EVERY tile of the layer, not only the last round's
 *   tile_n  0 = automatic, 64 or 128 = column width of the tile of layers with more than 64 filters
 *           (64 also gives layers of 33..64 filters the 64x64 tile), 1 = 64x64 tiles for every layer */
void conv_set_ksplit(int split, int tile_n);

/* Tuning hook of the tile order (no counterpart in the reference).  The filter tiles of a layer are
 * cut into `bands` groups (1, 2, 4 or 8; halved until it divides the number of filter tiles); an
 * XCD's consecutive share of the tiles then reads 1/bands of the weights and bands/8 of the input
 * through its private L2.  0 = automatic: the count that minimises weights*8/bands + input*bands. */
void conv_set_bands(int bands);

/* Tuning hook of the first-layer kernel (3 or 16 input channels, 3x3; no counterpart in the reference).
 * Its 256-pixel tile is 2 rows x 128 columns, 4 x 64 or 8 x 32; waves_across = 4, 2 or 1 forces that
 * shape where its height divides the image's (the 2-row shape always applies), 0 = the shape that
 * wastes the fewest columns in the last tile of a row (default).  The outputs do not depend on the
 * shape. */
void conv_first_set_shape(int waves_across);

/* Operand precision of the tap-blocked MFMA convolution kernels (channels a multiple of 16, 1x1 or
 * 3x3 pad 1; grouped 32-filter tiles):
 *   0  fp32 (default; the reference's arithmetic on v_mfma_f32_32x32x2_f32);
 *   1  both operands rounded to bf16 (nearest even) inside the kernel, products and sums in fp32,
 *      epilogue unchanged: an opt-in speed/precision trade outside the parity bar;
 *   2  fp32 emulated on the bf16 matrix cores: each operand is the exact sum of three bf16 pieces,
 *      six piece-products per multiply-add summed in fp32 (the three dropped ones are below 2^-24
 *      relative).  Meets the fp32 parity bar; measured closer to the fp64 convolution than the
 *      fp32 CPU path is.
 * Layers served by other kernels (first layer, direct, xnor) stay fp32.  No counterpart in the
 * reference. */
void conv_set_precision(int precision);
int conv_get_precision(void);

/* XNOR convolution (xnor=1 layers): sign(x>0) inputs, sign(w>0)*mean|w| weights, zero padding,
 * computed as XOR + popcount on bit-packed operands, then the same batch-norm/bias/activation
 * tail.  Replaces the xnor branch of forward_convolutional_layer_gpu
 * (src/convolutional_kernels.cu:77-87) with the CPU semantics of
 * src/convolutional_layer.c:28-49,451-456.
 *   wbits  : scratch, xnor_weight_words(n,c,size) uint32 ([tap][slice][n padded to 16] sign bits, then the
 *            per-(filter, tap) popcounts);  wmean: scratch, n floats
 *   xbits  : scratch, xnor_input_words(batch,c,h,w) uint32 */
size_t xnor_weight_words(int n, int c, int size);
size_t xnor_input_words(int batch, int c, int h, int w);
void xnor_pack_weights_gpu(const float *weights, unsigned *wbits, float *wmean, int n, int c, int size);
void xnor_pack_input_gpu(const float *input, unsigned *xbits, int batch, int c, int h, int w);
void forward_convolutional_xnor_gpu(const float *input, const float *weights, unsigned *wbits,
                                    float *wmean, unsigned *xbits, const float *biases,
                                    const float *scales, const float *rolling_mean,
                                    const float *rolling_variance, float *output, int batch,
                                    int c, int h, int w, int n, int size, int stride, int pad,
                                    int batch_normalize, int activation);
/* The same with wbits / wmean already written by xnor_pack_weights_gpu for the current weights
 * (binarize_weights depends on the weights alone, so a caller that knows when they change - the
 * natural hook is push_convolutional_layer - packs once instead of on every forward). */
void forward_convolutional_xnor_packed_gpu(const float *input, const unsigned *wbits, const float *wmean,
                                           unsigned *xbits, const float *biases, const float *scales,
                                           const float *rolling_mean, const float *rolling_variance,
                                           float *output, int batch, int c, int h, int w, int n, int size,
                                           int stride, int pad, int batch_normalize, int activation);

/* A first layer and the 2x2 stride-2 maxpool layer behind it in one pass (no counterpart in the
 * reference): forward_convolutional_gpu (src/convolutional_kernels.cu:73-135) for a 3x3 / stride 1 /
 * pad 1 convolution of 3 channels into up to 64 filters, or of 16 channels into up to 32 (the second
 * convolution of the tiny networks), over an image of even height and a width that is a multiple of
 * 8, plus forward_maxpool_layer_gpu (src/maxpool_layer_kernels.cu:87-99; size 2, stride 2, padding 0
 * or 1) on its output.  forward_convolutional_gpu runs such a layer on the same kernel without the
 * pooled outputs, so the map is the same bits either way.
 *   output       the convolution's map [batch][n][h][w], or NULL: then only the pooled map is written
 *   pool_output  [batch][n][h/2][w/2]
 *   next_xbits   NULL, or where to write the sign bits (x > 0) of pool_output for an xnor convolution
 *                that reads it, in the layout of xnor_pack_input_gpu: xnor_input_words(batch, n, h/2, w/2)
 * Every buffer written holds the bits of the separate calls.  conv_maxpool_fusable() says whether a
 * geometry and activation are served; anything else ends the process. */
int conv_maxpool_fusable(int batch, int c, int h, int w, int n, int groups, int size, int stride, int pad,
                         int activation);
void forward_convolutional_maxpool_gpu(const float *input, const float *weights, const float *biases,
                                       const float *scales, const float *rolling_mean,
                                       const float *rolling_variance, float *output, float *pool_output,
                                       unsigned *next_xbits, int batch, int c, int h, int w, int n, int groups,
                                       int size, int stride, int pad, int batch_normalize, int activation);

/* forward_convolutional_xnor_packed_gpu with what the layers around an xnor convolution otherwise do
 * in passes of their own (no counterpart in the reference):
 *   xbits_ready != 0  xbits already holds the sign bits of the input (the layer that produced the
 *                     input wrote them through its own next_xbits); `input` is then not read
 *   pool_output       NULL, or the output of the 2x2 stride-2 maxpool layer behind this one
 *                     (src/maxpool_layer.c:79-114 with size 2, stride 2, padding 0 or 1), written from
 *                     the same pass: [batch][n][out_h/2][out_w/2].  Needs size 3, stride 1, pad 1 and
 *                     an even out_h, out_w.  `output` may then be NULL: the convolution's own map is
 *                     not written
 *   next_xbits        NULL, or where to write the sign bits (x > 0) of pool_output - of `output` when
 *                     there is no pool_output - in the layout xnor_pack_input_gpu gives that tensor:
 *                     xnor_input_words(batch, n, its height, its width) words
 * Every buffer written holds the bits the separate calls (forward_convolutional_xnor_packed_gpu,
 * forward_maxpool_gpu, xnor_pack_input_gpu) would write. */
void forward_convolutional_xnor_fused_gpu(const float *input, const unsigned *wbits, const float *wmean,
                                          unsigned *xbits, int xbits_ready, const float *biases,
                                          const float *scales, const float *rolling_mean,
                                          const float *rolling_variance, float *output, float *pool_output,
                                          unsigned *next_xbits, int batch, int c, int h, int w, int n, int size,
                                          int stride, int pad, int batch_normalize, int activation);

/* forward_maxpool_layer_gpu (src/maxpool_layer_kernels.cu:87-99), CPU semantics of
 * src/maxpool_layer.c:79-114: window origin (-pad)/2, outside = -FLT_MAX, first maximum wins.
 * indexes may be NULL (inference never reads them). */
void forward_maxpool_gpu(const float *input, float *output, int *indexes, int batch, int c,
                         int h, int w, int size, int stride, int pad);

/* forward_route_layer_gpu (src/route_layer.c:105-118): all sources concatenated per image in
 * one launch.  srcs[i] holds batch x sizes[i] floats; output is batch x sum(sizes). */
void forward_route_gpu(const float *const *srcs, const int *sizes, int nsrc, float *output,
                       int batch);

/* forward_shortcut_layer_gpu (src/shortcut_layer.c:77-82): out = act(s1*in + s2*add) over the
 * overlapping region, act(in) elsewhere; one pass instead of copy + shortcut + activate.
 * (w1,h1,c1) describe add, (w2,h2,c2) describe in/out, as in shortcut_cpu (src/blas.c:68). */
void forward_shortcut_gpu(const float *in, const float *add, float *out, int batch, int w1,
                          int h1, int c1, int w2, int h2, int c2, float s1, float s2,
                          int activation);

/* forward_yolo_layer_gpu, inference part (src/yolo_layer.c:347-361 on the GPU; the CPU form
 * src/yolo_layer.c:132-148 defines the result): copy + logistic on x,y,objectness,classes.  The
 * logistic is evaluated in single precision (correctly rounded expf, hardware reciprocal): within
 * 3e-7 absolute of the reference's double evaluation, which made this kernel compute-bound. */
void forward_yolo_gpu(const float *input, float *output, int batch, int w, int h, int n_anchors,
                      int classes);

/* forward_region_layer_gpu, inference part (src/region_layer.c:439-485 on the GPU; the CPU form
 * :158-184 defines the result): copy, logistic on x, y, on objectness unless `background`, and
 * on the classes unless `softmax`, in which case softmax_cpu runs over the classes (+background)
 * of every (image, anchor, cell) with stride w*h.  Layout [b][anchor][coords+1+classes][h][w]. */
void forward_region_gpu(const float *input, float *output, int batch, int w, int h, int n_anchors,
                        int classes, int coords, int background, int softmax);

/* forward_local_layer_gpu (src/local_layer.c:186-215; the CPU form :91-120 defines the result):
 * a convolution with one [n][size*size*c] weight matrix per output location (location-major) and
 * one bias per output element, then the activation.  `pad` is the number of zero pixels on each
 * side, as the reference hands it to im2col, not a flag.  Output [b][n][out_h][out_w] with
 * out_h = (h - (pad ? 1 : size))/stride + 1 (src/local_layer.c:10-24); geometries for which im2col
 * would produce a different count end the process. */
void forward_local_gpu(const float *input, const float *weights, const float *biases, float *output,
                       int batch, int c, int h, int w, int n, int size, int stride, int pad,
                       int activation);

/* forward_local_gpu gathers its patches into a library-owned device buffer of batch * out_h * out_w *
 * size*size*c floats, grown on demand and kept; beyond this budget (default 2^28 floats = 1 GiB) a
 * batch runs in slices of images, with the same result.  No counterpart in the reference, which
 * keeps one image's im2col in net.workspace. */
void local_set_patch_budget(long floats);

/* forward_connected_layer_gpu without batch-norm (src/connected_layer.c:286-303; the CPU form
 * :140-167 defines the result) as one streaming pass over the weights [outputs][inputs]: the form
 * for small batches, where the layer is bound by reading its weights once.  Any batch is accepted;
 * above 16 images the weights are read once per 16. */
void forward_connected_stream_gpu(const float *input, const float *weights, const float *biases,
                                  float *output, int batch, int inputs, int outputs, int activation);

/* forward_batchnorm_layer_gpu at inference (src/batchnorm_layer.c:189-235 with net.train == 0; CPU form
 * :135-155): output = ((input - rolling_mean) / (sqrt(rolling_variance) + 1e-6f)) * scales + biases per
 * channel, each step rounded to float as the reference's copy / normalize / scale_bias / add_bias passes
 * round it, in one pass.  input and output are [batch][c][spatial]; they may be the same buffer. */
void forward_batchnorm_gpu(const float *input, float *output, const float *scales, const float *biases,
                           const float *rolling_mean, const float *rolling_variance, int batch, int c,
                           int spatial);

/* forward_avgpool_layer_gpu (src/avgpool_layer_kernels.cu:46-54). */
void forward_avgpool_gpu(const float *input, float *output, int batch, int c, int h, int w);

/* reorg_gpu / flatten_gpu (src/blas.h:73-74, CPU forms src/blas.c:9-49): the index permutations
 * of the reorg layer.  (w,h,c) describe the tensor whose flat index the loop walks; `forward`
 * != 0 scatters x[walk] to out[permuted], 0 gathers out[walk] = x[permuted]; flatten_gpu writes
 * to `out` instead of permuting in place.  forward_crop_gpu: forward_crop_layer at inference
 * (src/crop_layer.c:67-103 with net.train == 0): centred window, value*2-1 unless noadjust. */
void reorg_gpu(float *x, int w, int h, int c, int batch, int stride, int forward, float *out);
void flatten_gpu(float *x, int spatial, int layers, int batch, int forward, float *out);
void forward_crop_gpu(const float *input, float *output, int batch, int c, int h, int w, int out_h,
                      int out_w, int noadjust);

/* ------------------------------------------------------------------------------------------
 * Input side.  Images are [c][h][w] floats as the reference's `image` (include/darknet.h:508).
 * ---------------------------------------------------------------------------------------- */

/* resize_image (src/image.c:1199-1241): the reference's two-pass bilinear filter, bit for bit
 * (the horizontal pass's float intermediate is recomputed, not stored).  letterbox_image
 * (src/image.c:812-831): the image resized to fit box_w x box_h with its aspect kept, centred
 * on a .5 background (fill_image, embed_image :428-439).  All pointers are device pointers. */
void resize_image_gpu(const float *im, int w, int h, int c, float *out, int out_w, int out_h);
void letterbox_image_gpu(const float *im, int w, int h, int c, float *boxed, int box_w, int box_h);

/* ------------------------------------------------------------------------------------------
 * Detections: the step right after the forward pass.  A detection is a row of (5 + classes)
 * floats in device memory: x, y, w, h, objectness, prob[classes].
 * ---------------------------------------------------------------------------------------- */

/* Thresholded decode of ONE yolo head of ONE image, appended to `rows`.  Replaces
 * yolo_num_detections + get_yolo_detections (src/yolo_layer.c:275-343) with get_yolo_box
 * (:83-91) and correct_yolo_boxes (:247-273): a cell/anchor whose objectness exceeds `thresh`
 * becomes a row, prob[j] = objectness*class_j if that exceeds `thresh`, else 0; rows keep the
 * reference's order (cells row-major, anchors inside a cell).
 *   layer_output  device, the image's slab of the yolo layer output [n][5+classes][lh][lw]
 *   anchors       HOST, 2*n floats: biases[2*mask[i]], biases[2*mask[i]+1]  (n <= 16)
 *   netw,neth     network input size; w,h the original image size; relative as the reference
 *   rows,max_rows device row buffer and its capacity in rows
 *   count         device int: rows already present; incremented by the rows this head adds even
 *                 past max_rows (nothing is written past it), so the caller can tell overflow */
void yolo_decode_gpu(const float *layer_output, int lw, int lh, int n, int classes,
                     const float *anchors, int netw, int neth, int w, int h, int relative,
                     float thresh, float *rows, int max_rows, int *count);

/* The same for ONE region head (yolov2), get_region_detections src/region_layer.c:364-437 with
 * get_region_box :76-84 and correct_region_boxes :336-362: all lw*lh*n rows are written, row
 * anchor*lw*lh + cell after the `*count` rows already there (the reference returns every anchor
 * of every cell; objectness at or below `thresh` is stored as 0 and leaves the probabilities
 * 0); anchors: HOST, the layer's 2*n biases, in cell units.  coords must be 4. */
void region_decode_gpu(const float *layer_output, int lw, int lh, int n, int classes, int coords,
                       int background, const float *anchors, int netw, int neth, int w, int h,
                       int relative, float thresh, float *rows, int max_rows, int *count);

/* The same for the yolov1 detection layer, get_detection_detections src/detection_layer.c:225-252:
 * all side*side*n rows are written, row cell*n + box after the `*count` rows already there; the
 * objectness column holds the box's scale whatever the threshold, the class columns
 * scale*probability where that exceeds `thresh`, else 0.  layer_output is one image of the
 * layer: [cells][classes] probabilities, [cells][n] scales, [cells][n][4] boxes; the box is scaled
 * to w x h as given (no letterbox correction, as in the reference). */
void detection_decode_gpu(const float *layer_output, int side, int n, int classes, int sqrt, int w,
                          int h, float thresh, float *rows, int max_rows, int *count);

/* do_nms_sort (src/box.c:58-89) on device rows, in place: per class, in descending
 * probability (ties: lower row first), a row zeroes that class's probability in every later row
 * whose box_iou (src/box.c:152-155) with it exceeds `thresh`.  Rows keep their positions. */
void nms_sort_gpu(float *rows, int total, int classes, float thresh);

#ifdef __cplusplus
}
#endif
#endif
