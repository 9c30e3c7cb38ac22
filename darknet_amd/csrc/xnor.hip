/*
 * xnor.hip - XNOR-net convolution (xnor=1 layers) as XOR + popcount on bit-packed operands.
 *
 * Reference semantics (CPU build): the weights of filter f become sign(w>0) * mean_f with
 * mean_f = (sequential float sum of |w|) / size (src/convolutional_layer.c:28-41), the input
 * becomes sign(x>0) in {-1,+1} (:43-49), and the ordinary im2col + GEMM runs on those tensors
 * (:451-476), so zero padding contributes 0, not -1.  Hence
 *     out[f][p] = mean_f * sum over taps inside the image of (C - 2*popcount(xbits ^ wbits))
 * followed by the usual batch-norm / bias / activation tail.
 *
 * Bit layouts (bit j of a word <-> channel 32*word + j; 1 means value > 0; channels beyond C
 * are 0 in both operands so they never count as a mismatch):
 *   xbits [batch][Cw][H][W]      one word per pixel and 32-channel slice, planes contiguous so a
 *                                 wavefront reads consecutive pixels of one slice
 *   wbits [n][size*size][Cw]
 */
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "device_math.h"
#include "hip.h"

#define XN_BLOCK 256
#define XN_FPB 16 /* filters per workgroup */

static inline hipStream_t dn_stream() { return (hipStream_t)hip_get_stream(); }

extern "C" size_t xnor_weight_words(int n, int c, int size)
{
    return (size_t)n * size * size * ((c + 31) / 32);
}

extern "C" size_t xnor_input_words(int batch, int c, int h, int w)
{
    return (size_t)batch * ((c + 31) / 32) * h * w;
}

/* One thread per filter: the |w| sum must be taken in the reference's order to round alike. */
__global__ void xnor_pack_weights_kernel(const float *weights, unsigned *wbits, float *wmean, int n, int c,
                                         int size)
{
    const int f = blockIdx.x * blockDim.x + threadIdx.x;
    if (f >= n) return;
    const int ss = size * size;
    const int K = c * ss;
    const int cw = (c + 31) / 32;
    const float *w = weights + (long)f * K;
    float mean = 0;
    for (int i = 0; i < K; ++i) mean = (float)((double)mean + fabs((double)w[i]));
    wmean[f] = mean / K;
    for (int t = 0; t < ss; ++t)
        for (int wd = 0; wd < cw; ++wd) {
            unsigned bits = 0;
            for (int j = 0; j < 32; ++j) {
                const int ch = wd * 32 + j;
                if (ch < c && w[(long)ch * ss + t] > 0) bits |= 1u << j;
            }
            wbits[((long)f * ss + t) * cw + wd] = bits;
        }
}

extern "C" void xnor_pack_weights_gpu(const float *weights, unsigned *wbits, float *wmean, int n, int c,
                                      int size)
{
    hipLaunchKernelGGL(xnor_pack_weights_kernel, dim3((n + 63) / 64), dim3(64), 0, dn_stream(), weights, wbits,
                       wmean, n, c, size);
    dn_check_launch("xnor_pack_weights_gpu");
}

/* One thread per (image, slice, pixel): 32 coalesced channel-plane reads -> one word. */
__global__ void xnor_pack_input_kernel(const float *in, unsigned *xbits, long total, int c, int hw, int cw)
{
    for (long i = blockIdx.x * (long)blockDim.x + threadIdx.x; i < total; i += (long)gridDim.x * blockDim.x) {
        const int pix = (int)(i % hw);
        long t = i / hw;
        const int wd = (int)(t % cw);
        const long b = t / cw;
        const float *src = in + (b * c + (long)wd * 32) * hw + pix;
        const int nch = min(32, c - wd * 32);
        unsigned bits = 0;
        for (int j = 0; j < nch; ++j)
            if (src[(long)j * hw] > 0) bits |= 1u << j;
        xbits[i] = bits;
    }
}

extern "C" void xnor_pack_input_gpu(const float *input, unsigned *xbits, int batch, int c, int h, int w)
{
    const int cw = (c + 31) / 32;
    const long total = (long)batch * cw * h * w;
    long blocks = (total + XN_BLOCK - 1) / XN_BLOCK;
    if (blocks > 256L * 32) blocks = 256L * 32;
    hipLaunchKernelGGL(xnor_pack_input_kernel, dim3((int)blocks), dim3(XN_BLOCK), 0, dn_stream(), input, xbits,
                       total, c, h * w, cw);
    dn_check_launch("xnor_pack_input_gpu");
}

struct xnor_args {
    const unsigned *xbits;
    const unsigned *wbits;
    const float *wmean;
    const float *biases, *scales, *mean, *var;
    float *out;
    int c, h, w, n, size, stride, pad, oh, ow, cw, bn, act;
};

/* Workgroup: XN_FPB filters x 256 output pixels of one image.  The filters' bit rows sit in
 * LDS (read as wave-uniform broadcasts); each lane owns a pixel and walks taps x slices. */
__global__ __launch_bounds__(XN_BLOCK) void xnor_conv_kernel(xnor_args a)
{
    extern __shared__ unsigned wsm[]; /* [XN_FPB][taps*cw] */
    const int ss = a.size * a.size;
    const int row = ss * a.cw;
    const int f0 = blockIdx.y * XN_FPB;
    const int nf = min(XN_FPB, a.n - f0);
    const int b = blockIdx.z;
    for (int i = threadIdx.x; i < XN_FPB * row; i += XN_BLOCK) {
        const int j = i / row;
        wsm[i] = j < nf ? a.wbits[(long)(f0 + j) * row + (i - j * row)] : 0u;
    }
    __syncthreads();
    const int P = a.oh * a.ow;
    const int p = blockIdx.x * XN_BLOCK + threadIdx.x;
    if (p >= P) return;
    const int oy = p / a.ow, ox = p - oy * a.ow;
    const int iy0 = oy * a.stride - a.pad, ix0 = ox * a.stride - a.pad;
    const long plane = (long)a.h * a.w;
    const unsigned *xb = a.xbits + (long)b * a.cw * plane;
    int mism[XN_FPB];
#pragma unroll
    for (int j = 0; j < XN_FPB; ++j) mism[j] = 0;
    int taps_inside = 0;
    for (int ky = 0; ky < a.size; ++ky) {
        const int iy = iy0 + ky;
        if (iy < 0 || iy >= a.h) continue;
        for (int kx = 0; kx < a.size; ++kx) {
            const int ix = ix0 + kx;
            if (ix < 0 || ix >= a.w) continue;
            ++taps_inside;
            const int t = ky * a.size + kx;
            for (int wd = 0; wd < a.cw; ++wd) {
                const unsigned x = xb[wd * plane + (long)iy * a.w + ix];
#pragma unroll
                for (int j = 0; j < XN_FPB; ++j) mism[j] += __popc(x ^ wsm[j * row + t * a.cw + wd]);
            }
        }
    }
#pragma unroll
    for (int j = 0; j < XN_FPB; ++j) {
        if (j >= nf) continue;
        const int f = f0 + j;
        const int dot = taps_inside * a.c - 2 * mism[j];
        const float acc = __fmul_rn(a.wmean[f], (float)dot);
        const dn_bn_row r = dn_bn_make(a.bn, a.biases[f], a.bn ? a.scales[f] : 1.f, a.bn ? a.mean[f] : 0.f,
                                       a.bn ? a.var[f] : 1.f);
        a.out[((long)b * a.n + f) * P + p] = dn_activate(dn_bn_apply(acc, r, a.bn), a.act);
    }
}

extern "C" void forward_convolutional_xnor_gpu(const float *input, const float *weights, unsigned *wbits,
                                               float *wmean, unsigned *xbits, const float *biases,
                                               const float *scales, const float *rolling_mean,
                                               const float *rolling_variance, float *output, int batch,
                                               int c, int h, int w, int n, int size, int stride, int pad,
                                               int batch_normalize, int activation)
{
    if (batch <= 0 || c <= 0 || h <= 0 || w <= 0 || n <= 0 || size <= 0 || stride <= 0 || pad < 0)
        dn_fatal("forward_convolutional_xnor_gpu: bad geometry");
    if (!input || !weights || !wbits || !wmean || !xbits || !biases || !output)
        dn_fatal("forward_convolutional_xnor_gpu: null pointer");
    if (batch_normalize && (!scales || !rolling_mean || !rolling_variance))
        dn_fatal("forward_convolutional_xnor_gpu: batch_normalize needs scales, rolling_mean, rolling_variance");
    if (size == 1 && (stride != 1 || pad != 0))
        dn_fatal("forward_convolutional_xnor_gpu: a 1x1 kernel needs stride 1 and pad 0");
    xnor_args a;
    a.oh = (h + 2 * pad - size) / stride + 1;
    a.ow = (w + 2 * pad - size) / stride + 1;
    if (a.oh <= 0 || a.ow <= 0) dn_fatal("forward_convolutional_xnor_gpu: empty output");
    a.cw = (c + 31) / 32;
    const size_t lds = sizeof(unsigned) * XN_FPB * size * size * a.cw;
    if (lds > 64 * 1024) dn_fatal("forward_convolutional_xnor_gpu: filter bits exceed the LDS budget");
    /* the reference re-binarises both operands on every forward (src/convolutional_layer.c:451-455) */
    xnor_pack_weights_gpu(weights, wbits, wmean, n, c, size);
    xnor_pack_input_gpu(input, xbits, batch, c, h, w);
    a.xbits = xbits;
    a.wbits = wbits;
    a.wmean = wmean;
    a.biases = biases;
    a.scales = scales;
    a.mean = rolling_mean;
    a.var = rolling_variance;
    a.out = output;
    a.c = c;
    a.h = h;
    a.w = w;
    a.n = n;
    a.size = size;
    a.stride = stride;
    a.pad = pad;
    a.bn = batch_normalize ? 1 : 0;
    a.act = activation;
    const int P = a.oh * a.ow;
    const int fblocks = (n + XN_FPB - 1) / XN_FPB;
    if (fblocks > 65535 || batch > 65535) dn_fatal("forward_convolutional_xnor_gpu: grid too large");
    dim3 grid((P + XN_BLOCK - 1) / XN_BLOCK, fblocks, batch);
    hipLaunchKernelGGL(xnor_conv_kernel, grid, dim3(XN_BLOCK), lds, dn_stream(), a);
    dn_check_launch("forward_convolutional_xnor_gpu");
}
